"""Builds libcascmm.so (HIP, gfx950 only) in-tree with hipcc.

    python -m basedxl_amd.build

Every .hip file under csrc/ is one translation unit; they are compiled in parallel and
linked into basedxl_amd/libcascmm.so, which the ctypes loader in _lib.py opens.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libcascmm.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "warning generated" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True, jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(jobs, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    # a kernel whose launch stub the compiler left out only shows up as an undefined symbol at load time
    import ctypes
    try:
        ctypes.CDLL(LIB)
    except OSError as e:
        raise RuntimeError(f"{LIB} was linked but does not load: {e}") from None
    if verbose:
        print(f"built {LIB} from {len(srcs)} translation units")
    return LIB


def _listing(src: str) -> str:
    """Assembly listing of one translation unit's device code (kept beside the objects, redone when a
    source under csrc/ is newer)."""
    out = os.path.join(OBJ, src[:-4] + ".gfx950.s")
    newest = max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC) if f.endswith((".hip", ".h")))
    if not os.path.exists(out) or os.path.getmtime(out) < newest:
        os.makedirs(OBJ, exist_ok=True)
        tmp = f"{out}.{os.getpid()}.tmp"      # (another process may be making the same listing: rename a finished file into place)
        cmd = [HIPCC, *FLAGS, "-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", tmp]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            if os.path.exists(tmp):
                os.remove(tmp)
            raise RuntimeError(f"hipcc -S failed on {src}:\n{r.stderr[-2000:]}")
        os.replace(tmp, out)
    return out


def kernel_isa(symbol: str, jobs: int = 8) -> str:
    """gfx950 assembly of one kernel of the library, from its label to the end of its
    `.amdhsa_kernel` block (register counts, LDS and scratch sizes), compiled from the sources under
    csrc/ with the flags of the build.  `symbol` is what `cascmm_variant_kernel` returns."""
    srcs = [f for f in sources() if f.startswith("cascmm_inst_")] + [f for f in sources() if not f.startswith("cascmm_inst_")]
    with ThreadPoolExecutor(max_workers=min(jobs, len(srcs))) as ex:
        listings = list(ex.map(_listing, srcs))
    label, end = symbol + ":", ".end_amdhsa_kernel"
    for path in listings:
        with open(path) as f:
            text = f.read()
        at = text.find("\n" + label)
        if at < 0:
            continue
        meta = text.find("\t.amdhsa_kernel " + symbol + "\n", at)
        stop = text.find(end, meta if meta >= 0 else at)
        if stop < 0:
            continue
        return f"; {os.path.basename(path)}\n" + text[at + 1:stop + len(end)] + "\n"
    raise KeyError(f"no kernel {symbol} in the listings of {', '.join(srcs)}")


if __name__ == "__main__":
    build()
