"""The C++ host-side operator (MI355QuantGemmKernel, QuantGemmRegistry).

The cases themselves are C++ (tests/cpp/test_quant_gemm_kernel.cpp), written like
the reference's operator tests; these wrappers run the prebuilt program: the
host-logic cases anywhere, the device cases (compared with the oracle) on a GPU.
"""
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
EXE = ROOT / "tests" / "cpp" / "bin" / "test_quant_gemm_kernel"
HOST_LIB = ROOT / "llaminar_amd" / "lib" / "libllaminar_ql_host.so"


def _run(*args, timeout=300):
    assert EXE.exists(), f"{EXE} is not built: run __graft_entry__.build()"
    proc = subprocess.run([str(EXE), *args], capture_output=True, text=True, timeout=timeout)
    print(proc.stdout[-6000:])
    print(proc.stderr[-2000:])
    return proc


def test_host_library_exports_operator_methods():
    assert HOST_LIB.exists(), "libllaminar_ql_host.so is not built"
    out = subprocess.run(["nm", "-DC", "--defined-only", str(HOST_LIB)], capture_output=True, text=True, check=True).stdout
    for method in ("multiply_tensor", "multiply_fused_tensor", "multiply_tensor_with_fused_swiglu",
                   "multiply_fused_verifier_rows_decode_equivalent", "multiply_fused_expert_down",
                   "quantize_activations", "multiply_with_precomputed_q8_1", "prepareWeights",
                   "releaseWeights", "exportMatrixDesc", "getWorkspaceRequirements"):
        assert f"llaminar_amd::MI355QuantGemmKernel::{method}(" in out, method
    for method in ("prepareGemmHandleLocal", "getOrCreateGemmEngine", "registerPreparedGemmHandle",
                   "gemmKernel", "registerEngine", "getEngine"):
        assert f"llaminar_amd::QuantGemmRegistry::{method}(" in out, method


def test_host_logic_cases():
    proc = _run("--cpu")
    assert proc.returncode == 0, proc.stdout[-3000:]
    assert "PASSED" in proc.stdout


@pytest.mark.gpu
def test_operator_against_oracle_on_device():
    proc = _run()
    assert proc.returncode == 0, proc.stdout[-4000:] + proc.stderr[-2000:]
    assert "PASSED" in proc.stdout
