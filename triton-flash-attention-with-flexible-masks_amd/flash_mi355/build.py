"""Build the gfx950 shared library in-tree with hipcc (cross-compiles without a GPU).

    python -m flash_mi355.build          # from the package directory, or
    flash_mi355.build.build(force=True)

Every .hip file of csrc/ is compiled to an object next to the library and linked
into flash_mi355/libflash_mi355.so.  Nothing is installed outside the tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR.parent / "csrc"
INCLUDE = PKG_DIR.parent.parent / "include"
LIB_PATH = PKG_DIR / "libflash_mi355.so"
OBJ_DIR = PKG_DIR / "_obj"

SOURCES = ["fa_api.hip", "fa_aux.hip", "fa_fwd.hip", "fa_bwd_dq.hip", "fa_bwd_dkdv.hip", "fa_f32.hip"]
# measurement aid of bench.py --mfma-probe (sustained MFMA rate of the chip); a library of its own
PROBE_SOURCE = "probe_mfma.hip"
PROBE_LIB_PATH = PKG_DIR / "libfa_probe.so"
# measurement aid of bench.py --wg-trace: the same sources with -DFA_TRACE (clock stamps per
# workgroup and the extra export fa_trace_read); never loaded by the operator
TRACE_LIB_PATH = PKG_DIR / "libflash_mi355_trace.so"
TRACE_OBJ_DIR = PKG_DIR / "_obj_trace"

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # no compiler-generated packed fp32 arithmetic on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _compile(src: Path, obj: Path, extra) -> str:
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, f"-I{INCLUDE}", "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stderr[-4000:]}")
    return r.stderr


def build(force: bool = True, verbose: bool = False, extra_flags=()) -> Path:
    """Compile all kernels and link the library (and the two measurement libraries); returns its path."""
    OBJ_DIR.mkdir(exist_ok=True)
    TRACE_OBJ_DIR.mkdir(exist_ok=True)
    headers = list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h"))
    newest_hdr = max(h.stat().st_mtime for h in headers)
    jobs, trace_jobs = [], []
    for name in SOURCES:
        src = CSRC / name
        for obj_dir, todo, flags in ((OBJ_DIR, jobs, []), (TRACE_OBJ_DIR, trace_jobs, ["-DFA_TRACE"])):
            obj = obj_dir / (src.stem + ".o")
            stale = force or not obj.exists() or obj.stat().st_mtime < max(src.stat().st_mtime, newest_hdr)
            if stale:
                todo.append((src, obj, flags))
    with ThreadPoolExecutor(max_workers=8) as ex:
        logs = list(ex.map(lambda j: _compile(j[0], j[1], list(extra_flags) + j[2]), jobs + trace_jobs))
    logs = logs[:len(jobs)]
    if verbose:
        for (src, _, _), log in zip(jobs, logs):
            lines = [l for l in log.splitlines() if "packed-fp32-ops" not in l]
            if lines:
                print(f"--- {src.name}\n" + "\n".join(lines))
    probe_src = CSRC / PROBE_SOURCE
    if force or not PROBE_LIB_PATH.exists() or PROBE_LIB_PATH.stat().st_mtime < probe_src.stat().st_mtime:
        cmd = [_hipcc(), *HIPCC_FLAGS, "-shared", str(probe_src), "-o", str(PROBE_LIB_PATH)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {PROBE_SOURCE}:\n{r.stderr[-4000:]}")
    objs = [str(OBJ_DIR / (Path(n).stem + ".o")) for n in SOURCES]
    if jobs or not LIB_PATH.exists():
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *objs]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    if trace_jobs or not TRACE_LIB_PATH.exists():
        tobjs = [str(TRACE_OBJ_DIR / (Path(n).stem + ".o")) for n in SOURCES]
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(TRACE_LIB_PATH), *tobjs]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--incremental" not in sys.argv, verbose=True)
    print(path)
