"""Compile the gfx950 quantized-linear library in-tree with hipcc.

Every ``*.hip`` / ``*.cpp`` source under ``llaminar_amd/csrc`` is compiled into
one shared object, ``llaminar_amd/lib/libllaminar_ql.so``.  hipcc cross-compiles
for gfx950 without a GPU, so this runs anywhere the ROCm toolchain is present.

The host-side operator (``csrc/host``) is linked into a second library,
``libllaminar_ql_host.so``, on top of the first.

Usage: ``python -m llaminar_amd.build``
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIBDIR = PKG / "lib"
LIB = LIBDIR / "libllaminar_ql.so"
HOST_LIB = LIBDIR / "libllaminar_ql_host.so"
OBJDIR = PKG / "build"

ARCH = "gfx950"
# -packed-fp32-ops is switched OFF: scalar fp32 code must not be fused into
# v_pk_*_f32 forms.  The host pass warns that it does not know the feature.
HIP_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]
# Register allocation of every kernel is reported by the compiler and checked below.
RESOURCE_FLAG = "-Rpass-analysis=kernel-resource-usage"


class SpillError(RuntimeError):
    """A kernel needs per-lane scratch memory (register spills)."""


def check_kernel_resources(remarks: str, src_name: str) -> dict[str, dict[str, int]]:
    """Parse hipcc's kernel-resource-usage remarks and refuse any kernel that spills.

    Several kernels issue their global loads as inline assembly and wait for them by
    hand many instructions later.  The compiler takes the destination registers of such
    a load as written at the point of issue.  If it has to spill, it may store such a
    register to scratch straight after the load instruction (before the data has
    arrived: the spill slot gets stale contents) and hand the register to another
    value, for instance an address; the load then lands in that value and the kernel
    reads a wild address.  The kernels are only correct with zero spills, so a spill
    fails the build instead of the GPU.
    """
    usage: dict[str, dict[str, int]] = {}
    name = None
    for line in remarks.splitlines():
        # the remark's position is printed before "remark:" or, under -save-temps, after it
        m = re.search(r"remark:(?: \S+:\d+:\d+:)? Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            usage[name] = {}
            continue
        m = re.search(r"remark:(?: \S+:\d+:\d+:)?\s+(ScratchSize \[bytes/lane\]|VGPRs Spill|SGPRs Spill|VGPRs|Dynamic Stack): (\S+)", line)
        if m and name is not None:
            v = m.group(2)
            usage[name][m.group(1)] = int(v) if v.isdigit() else int(v == "True")
    bad = [
        f"{k}: scratch {u.get('ScratchSize [bytes/lane]', 0)} B/lane, {u.get('VGPRs Spill', 0)} VGPRs spilled"
        for k, u in usage.items()
        if u.get("ScratchSize [bytes/lane]", 0) or u.get("VGPRs Spill", 0) or u.get("Dynamic Stack", 0)
    ]
    if bad:
        raise SpillError(
            f"{src_name}: kernels with register spills are refused (hand-scheduled loads are unsafe "
            "once the compiler spills):\n  " + "\n  ".join(bad)
        )
    return usage


class InFlightRegisterError(RuntimeError):
    """Compiler-generated code touches the destination register of a hand-issued load before its wait."""


_VREG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
_ASM_LOAD = re.compile(r"^\s*(global_load_\w+|buffer_load_\w+)\s+(v\d+|v\[\d+:\d+\])\s*,")
_VMEM = re.compile(r"^\s*(global_|buffer_|flat_|scratch_)(load|store|atomic)")
_VMCNT = re.compile(r"vmcnt\((\d+)\)")


def _vregs(text: str) -> set[int]:
    regs: set[int] = set()
    for m in _VREG.finditer(text):
        if m.group(1) is not None:
            regs.add(int(m.group(1)))
        else:
            regs.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return regs


def check_inflight_registers(asm: str, src_name: str) -> int:
    """Scan the device assembly for the second way the hand-scheduled loads can break.

    The kernels issue global loads inside inline assembly and wait for them (s_waitcnt
    vmcnt, also inline assembly) many instructions later.  To the compiler the destination
    registers hold their values from the point of issue, so besides spilling them it may
    COPY them (a phi move at a loop entry, a move into another allocation) or reuse them
    while the data is still on its way: the copy reads stale contents, or the load lands in
    whatever lives in the register by then.  This pass walks every function in program
    order, keeps the queue of vector memory operations that vmcnt counts (hand-issued loads
    with their destination registers, everything else as a placeholder), retires entries at
    each s_waitcnt vmcnt(N), and reports any instruction that names a register of a
    hand-issued load still in the queue.  Straight-line bookkeeping: the queue is emptied
    where control cannot fall through (s_branch, s_endpgm, s_setpc), so the pass can miss a
    hazard across a jump but does not invent one.  Returns the number of hand-issued loads
    it followed.
    """
    findings: list[str] = []
    followed = 0
    func = "?"
    queue: list[set[int] | None] = []  # oldest first; None: an operation whose registers the compiler tracks
    in_asm = False
    for raw_line in asm.splitlines():
        line = raw_line.split(";")[0].rstrip() if not raw_line.lstrip().startswith(";;#") else raw_line.strip()
        if line.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if line.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = re.match(r"^([A-Za-z_][\w$.]*):", line)
        if m and not line.startswith(".L"):
            func, queue = m.group(1), []
            continue
        text = line.strip()
        if not text or text.startswith(".") or text.endswith(":"):
            continue
        if text.startswith("s_waitcnt"):
            w = _VMCNT.search(text)
            if w:
                keep = int(w.group(1))
                queue = queue[len(queue) - keep:] if keep and keep < len(queue) else ([] if keep == 0 else queue)
            continue
        if re.match(r"^(s_branch|s_endpgm|s_setpc_b64)\b", text):
            queue = []
            continue
        touched = _vregs(text)
        load = _ASM_LOAD.match(text) if in_asm else None
        pending = set().union(*[q for q in queue if q]) if queue else set()
        if load:
            dst = _vregs(load.group(2))
            hit = (touched - dst) & pending or (dst & pending)
            if hit:
                findings.append(f"{func}: '{text}' uses v{sorted(hit)[0]} while a hand-issued load into it is in flight")
            queue.append(dst)
            followed += 1
            continue
        hit = touched & pending
        if hit:
            findings.append(f"{func}: '{text}' touches v{sorted(hit)[0]} before the wait for the hand-issued load into it")
        if _VMEM.match(text):
            queue.append(None)
    if findings:
        shown = "\n  ".join(findings[:12]) + ("" if len(findings) <= 12 else f"\n  ... and {len(findings) - 12} more")
        raise InFlightRegisterError(
            f"{src_name}: registers of hand-issued loads are touched before their s_waitcnt "
            f"(the data has not arrived; see check_inflight_registers):\n  {shown}")
    return followed


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found: the ROCm toolchain is required to build llaminar_amd")
    return exe


def sources() -> list[Path]:
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")))


def _deps_mtime() -> float:
    files = [f for f in CSRC.rglob("*") if f.is_file()] + list((ROOT / "include" / "llaminar_amd").glob("*.h*"))
    return max(f.stat().st_mtime for f in files)


def build_host(verbose: bool = True) -> Path:
    """Link the C++ operator layer against the kernel library (no device code)."""
    srcs = sorted((CSRC / "host").glob("*.cpp"))
    cmd = [hipcc(), "-std=c++17", "-O2", "-fPIC", "-shared", f"-I{ROOT / 'include'}", *map(str, srcs),
           f"-L{LIBDIR}", "-lllaminar_ql", "-Wl,-rpath,$ORIGIN", "-o", str(HOST_LIB)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"host library build failed:\n{proc.stderr}")
    if verbose:
        print(f"[llaminar_amd.build] wrote {HOST_LIB} ({HOST_LIB.stat().st_size} bytes)", flush=True)
    return HOST_LIB


def _drop_resource_remarks(lines: list[str]) -> list[str]:
    """Compiler output without the kernel-resource-usage remarks and their source excerpts."""
    out, skip = [], 0
    for l in lines:
        if "[-Rpass-analysis=kernel-resource-usage]" in l:
            skip = 2 if "Function Name" in l else 0  # the excerpt: source line and caret line
            continue
        if skip and (re.match(r"\s*\d+ \|", l) or re.match(r"\s*\|\s*\^", l)):
            skip -= 1
            continue
        skip = 0
        if re.match(r"In file included from ", l) or re.search(r"\d+ (warning|remark)s? generated", l):
            continue
        out.append(l)
    return out


def _headers_mtime() -> float:
    files = list(CSRC.glob("*.h")) + list((ROOT / "include" / "llaminar_amd").glob("*.h*"))
    return max(f.stat().st_mtime for f in files)


def _compile(src: Path, force: bool = True) -> Path:
    obj = OBJDIR / (src.stem + ".o")
    # without force an object newer than its source and every header is kept (it passed the checks below
    # when it was made)
    if not force and obj.exists() and obj.stat().st_mtime >= max(src.stat().st_mtime, _headers_mtime()):
        return obj
    # -save-temps leaves the device assembly beside the object file for check_inflight_registers
    cmd = [hipcc(), *HIP_FLAGS, RESOURCE_FLAG, "-save-temps=obj", "-c", str(src), "-o", str(obj)]
    if src.suffix == ".cpp":
        cmd.insert(1, "-x")
        cmd.insert(2, "hip")
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    lines = [l for l in proc.stderr.splitlines() if noise not in l]
    if proc.returncode == 0:
        check_kernel_resources(proc.stderr, src.name)
        for asm_file in OBJDIR.glob(f"{src.stem}-hip-amdgcn-*.s"):
            check_inflight_registers(asm_file.read_text(), src.name)
    err = "\n".join(_drop_resource_remarks(lines))
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = True, verbose: bool = True) -> Path:
    """Compile and link the library.  With force=False an up-to-date library is kept."""
    if not force and LIB.exists() and HOST_LIB.exists() and LIB.stat().st_mtime >= _deps_mtime():
        return LIB
    OBJDIR.mkdir(exist_ok=True)
    LIBDIR.mkdir(exist_ok=True)
    srcs = sources()
    if verbose:
        print(f"[llaminar_amd.build] hipcc {ARCH}: {len(srcs)} sources", flush=True)
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(lambda src: _compile(src, force), srcs))
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(LIB)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"[llaminar_amd.build] wrote {LIB} ({LIB.stat().st_size} bytes)", flush=True)
    build_host(verbose)
    return LIB


if __name__ == "__main__":
    build(force="--incremental" not in sys.argv)
