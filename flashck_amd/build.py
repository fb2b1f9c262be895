"""In-tree build of the gfx950 FMHA library (libflashck_fmha.so) with hipcc.

``python -m flashck_amd.build`` compiles every translation unit under ``csrc/`` for gfx950 and links the shared
library next to this file.  hipcc cross-compiles, so no GPU is needed to build.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libflashck_fmha.so")

SOURCES = ["fmha_api.cpp", "splitkv_decode.hip", "splitkv_combine.hip", "appendkv_rope.hip", "prefill.hip",
           "prefill_pingpong.hip", "prefill_dma.hip", "validate.hip", "appendkv_fp8.hip"]

FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "--offload-arch=gfx950", "-fno-gpu-rdc",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the FMHA library cannot be built")
    return exe


def _newest_header():
    dirs = (CSRC, os.path.join(ROOT, "include", "flashck", "fmha"))
    return max(os.path.getmtime(os.path.join(d, f)) for d in dirs for f in os.listdir(d) if f.endswith((".hpp", ".h")))


def _compile(src, extra, incremental=False):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(os.path.join(CSRC, src)), _newest_header()):
        return obj, ""
    cmd = [hipcc(), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + FLAGS + extra
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    return obj, out


def build(verbose=False, extra_flags=(), incremental=False):
    """incremental: translation units whose object file is newer than the source and every header are not recompiled
    (a development convenience; the default compiles everything)."""
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 4)) as ex:
        results = list(ex.map(lambda s: _compile(s, list(extra_flags), incremental), SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    tmp = LIB + ".tmp"
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", "-o", tmp] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}")
    os.replace(tmp, LIB)
    try:
        build_header_test()
    except RuntimeError as e:  # a test program that does not build must not take the library down with it
        print(f"warning: {e}", file=sys.stderr)
    return LIB


def build_header_test():
    """tests/cpp/fmha_header_gpu: the C++ program the GPU test of the header API (include/flashck/fmha/fmha_fwd.h)
    runs.  Built here, next to the library it links, so that it exists wherever the library does; skipped when the
    test sources are not part of the tree."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "cpp", "fmha_header_gpu.cpp")
    if not os.path.exists(src):
        return None
    exe = src[:-len(".cpp")]
    cmd = [hipcc(), "-std=c++17", "-O1", "-Wall", "-I", os.path.join(root, "include"), src, "-o", exe + ".tmp", "-L", HERE,
           "-lflashck_fmha", "-Wl,-rpath,$ORIGIN/../../flashck_amd"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building {exe} failed:\n{r.stdout}")
    os.replace(exe + ".tmp", exe)
    return exe


if __name__ == "__main__":
    flags = [a for a in sys.argv[1:] if a != "--incremental"]
    print(build(verbose=True, extra_flags=flags, incremental="--incremental" in sys.argv[1:]))
