"""The C++ host-side MoE operator (MI355MoEKernel: the decode methods of the reference's
IMoEKernel).  The cases are C++ (tests/cpp/test_moe_kernel.cpp); these wrappers run the
prebuilt program: the host-logic cases anywhere, the device cases (against the oracle) on a GPU."""
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
EXE = ROOT / "tests" / "cpp" / "bin" / "test_moe_kernel"
HOST_LIB = ROOT / "llaminar_amd" / "lib" / "libllaminar_ql_host.so"


def _run(*args, timeout=300):
    assert EXE.exists(), f"{EXE} is not built: run __graft_entry__.build()"
    proc = subprocess.run([str(EXE), *args], capture_output=True, text=True, timeout=timeout)
    print(proc.stdout[-6000:])
    print(proc.stderr[-2000:])
    return proc


def test_host_library_exports_moe_methods():
    out = subprocess.run(["nm", "-DC", "--defined-only", str(HOST_LIB)], capture_output=True, text=True, check=True).stdout
    for method in ("decodeRouteSelect", "uploadGroupedExpertGateUpDescriptorTables",
                   "uploadGroupedExpertDownDescriptorTable", "groupedExpertGateUpDecodeFromRuntime",
                   "groupedExpertDownDecodeFromRuntime", "groupedExpertDecodeFromRuntime", "sharedExpertGateAdd",
                   "getWorkspaceRequirements"):
        assert f"llaminar_amd::MI355MoEKernel::{method}(" in out, method
    # every function include/llaminar_amd/dense_decoder.h declares
    import re

    text = (ROOT / "include" / "llaminar_amd" / "dense_decoder.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(llam_decoder_[a-z_]+)\s*\(", text)))
    assert len(names) >= 9, names
    for fn in names:
        assert f" T {fn}" in out, fn


def test_host_logic_cases():
    proc = _run("--cpu")
    assert proc.returncode == 0, proc.stdout[-3000:]
    assert "PASSED" in proc.stdout


@pytest.mark.gpu
def test_moe_operator_against_oracle_on_device():
    proc = _run()
    assert proc.returncode == 0, proc.stdout[-4000:] + proc.stderr[-2000:]
    assert "PASSED" in proc.stdout
