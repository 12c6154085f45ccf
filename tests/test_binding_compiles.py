"""The Llaminar-side binding (include/llaminar_amd/binding/) compiles against the reference's
own interface headers: ITensorGemm + IWorkspaceConsumer (tensors/TensorKernels.h,
interfaces/IWorkspaceConsumer.h) and IMoEKernel (kernels/IMoEKernel.h).  Syntax check only;
skipped where the reference tree is absent (nothing of it ships or travels)."""
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
REFERENCE = Path("/root/reference/src/v2")
MPI_INCLUDE = Path("/opt/conda/include")  # <mpi.h>, pulled in by utils/MPIContext.h


@pytest.mark.skipif(not (REFERENCE / "tensors" / "TensorKernels.h").exists(), reason="reference tree not present")
def test_adapters_compile_against_the_reference_interfaces():
    cxx = shutil.which("g++")
    assert cxx, "g++ not found"
    cmd = [cxx, "-std=c++17", "-fsyntax-only", "-Wall", "-Wextra", "-Woverloaded-virtual", "-Werror",
           # the reference's SIMD headers need their instruction sets switched on to parse
           "-mavx512f", "-mavx512bw", "-mavx512vnni", "-mavx512vl", "-mavx512dq", "-mavx2", "-mfma", "-mf16c",
           # -isystem: warnings inside the reference's headers are not this check's business
           "-isystem", str(REFERENCE), "-isystem", str(MPI_INCLUDE), f"-I{ROOT / 'include'}",
           str(ROOT / "tests" / "cpp" / "adapter_check.cpp")]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-4000:]
