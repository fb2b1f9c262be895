"""Builds tests/emu/libflashck_fmha_emu.so: the kernel sources of flashck_amd/csrc, unchanged, compiled as C++ for the
host on top of the wave64 emulator in this directory.  Test infrastructure: only tests load the result."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "flashck_amd", "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libflashck_fmha_emu.so")
CXX = "/opt/rocm/llvm/bin/clang++"

sys.path.insert(0, ROOT)
from flashck_amd.build import SOURCES  # noqa: E402  (the same translation units as the shipped library)

FLAGS = ["-x", "c++", "-std=c++17", "-O1", "-g", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off", "-mf16c", "-mavx2",
         "-I", os.path.join(HERE, "include"), "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-I", HERE,
         "-include", os.path.join(HERE, "include", "gfx950_ops.hpp"),
         "-Wall", "-Wno-unused-function", "-Wno-unused-variable", "-Wno-unused-but-set-variable", "-Wno-unknown-pragmas"]


# FCK_EMU_GCOV=1: a second build with line and branch counters (clang --coverage, read with gcov), in its own directory
# and library, for finding the kernel and C-ABI code no test executes: tests/emu/line_coverage.py
GCOV = os.environ.get("FCK_EMU_GCOV") == "1"
if GCOV:
    OBJ = os.path.join(HERE, "build_gcov")
    LIB = os.path.join(HERE, "libflashck_fmha_emu_gcov.so")
    FLAGS = FLAGS + ["--coverage"]
# FCK_EMU_UBSAN=1: a build with the undefined-behaviour sanitizer (indexing past a fixed-size array, misaligned vector
# accesses, signed overflow, shifts out of range); a finding aborts the process with a report
UBSAN = os.environ.get("FCK_EMU_UBSAN") == "1"
if UBSAN:
    OBJ = os.path.join(HERE, "build_ubsan")
    LIB = os.path.join(HERE, "libflashck_fmha_emu_ubsan.so")
    FLAGS = FLAGS + ["-fsanitize=bounds,alignment,signed-integer-overflow,shift,null,integer-divide-by-zero", "-fno-sanitize-recover=all"]


def _sanitizer_dir():
    """where clang keeps its shared sanitizer runtimes"""
    r = subprocess.run([CXX, "-print-file-name=libclang_rt.ubsan_standalone-x86_64.so"], stdout=subprocess.PIPE, text=True)
    path = r.stdout.strip()
    if not os.path.isabs(path):   # not in the default place: search the resource directory
        res = subprocess.run([CXX, "-print-resource-dir"], stdout=subprocess.PIPE, text=True).stdout.strip()
        path = os.path.join(res, "lib", "linux", "libclang_rt.ubsan_standalone-x86_64.so")
    return os.path.dirname(path)


def _compile(path):
    obj = os.path.join(OBJ, os.path.splitext(os.path.basename(path))[0] + ".o")
    if os.path.exists(obj) and os.path.getmtime(obj) > max(
            os.path.getmtime(os.path.join(d, f)) for d in (CSRC, HERE, os.path.join(HERE, "include"), os.path.join(ROOT, "include", "flashck", "fmha"))
            for f in os.listdir(d) if f.endswith((".hip", ".hpp", ".h", ".cpp"))):
        return obj
    r = subprocess.run([CXX] + FLAGS + ["-c", path, "-o", obj], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"emulator build failed on {path}:\n{r.stdout[-6000:]}")
    return obj


class _Locked:
    """one build at a time (test workers of a parallel run all ask for the library)"""

    def __enter__(self):
        import fcntl
        os.makedirs(OBJ, exist_ok=True)
        self.f = open(os.path.join(OBJ, ".lock"), "w")
        fcntl.flock(self.f, fcntl.LOCK_EX)

    def __exit__(self, *exc):
        self.f.close()


def build():
    with _Locked():
        return _build()


def _build():
    os.makedirs(OBJ, exist_ok=True)
    paths = [os.path.join(CSRC, s) for s in SOURCES] + [os.path.join(HERE, "emu_runtime.cpp"), os.path.join(HERE, "selftest.cpp")]
    with ThreadPoolExecutor(max_workers=min(len(paths), os.cpu_count() or 4)) as ex:
        objs = list(ex.map(_compile, paths))
    if os.path.exists(LIB) and os.path.getmtime(LIB) >= max(os.path.getmtime(o) for o in objs):
        return LIB
    r = subprocess.run([CXX, "-shared", "-fPIC", "-o", LIB + ".tmp"] + objs + ["-lpthread", "-lm"] + (["--coverage"] if GCOV else []) +
                       (["-fsanitize=undefined", "-shared-libsan", "-Wl,-rpath," + _sanitizer_dir()] if UBSAN else []), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"emulator link failed:\n{r.stdout[-4000:]}")
    os.replace(LIB + ".tmp", LIB)
    return LIB


def build_pybind():
    """flash_ck/csrc/pybind.cpp bound to the emulator library: module `flash_ck_emu` in this directory."""
    import sysconfig
    from flash_ck import build as fb
    out = os.path.join(HERE, "flash_ck_emu" + sysconfig.get_config_var("EXT_SUFFIX"))
    src = os.path.join(ROOT, "flash_ck", "csrc", "pybind.cpp")
    with _Locked():
        if os.path.exists(out) and os.path.getmtime(out) > max(os.path.getmtime(src), os.path.getmtime(LIB)):
            return out
        return fb.build(name="flash_ck_emu", out=out, kernel_lib=LIB, extra=["-DFLASH_CK_HOST_TENSORS"])


if __name__ == "__main__":
    print(build())
