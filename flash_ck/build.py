"""In-tree build of the compiled module flash_ck/flash_ck<ext>.so (pybind11 + torch tensors over the C ABI of
flashck_amd/libflashck_fmha.so).  ``python -m flash_ck.build``; needs hipcc, builds without a GPU."""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def target():
    return os.path.join(HERE, "flash_ck" + sysconfig.get_config_var("EXT_SUFFIX"))


def build(name="flash_ck", out=None, kernel_lib=None, extra=()):
    """name / out / kernel_lib / extra: the test build against the emulator library (tests/emu) passes its own."""
    import torch
    from torch.utils import cpp_extension as ce
    from flashck_amd import build as lib_build
    if not os.path.exists(lib_build.LIB):
        lib_build.build()
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = out or target()
    kernel_lib = kernel_lib or lib_build.LIB
    libname = os.path.basename(kernel_lib)[3:-3]
    cmd = [lib_build.hipcc(), "-x", "c++", os.path.join(HERE, "csrc", "pybind.cpp"), "-shared", "-fPIC", "-O2", "-std=c++17", "-o", out + ".tmp",
           f"-DTORCH_EXTENSION_NAME={name}", "-DTORCH_API_INCLUDE_EXTENSION_H", "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-unused-result",
           "-I", os.path.join(ROOT, "include"), "-I", sysconfig.get_paths()["include"], "-I", "/opt/rocm/include"]
    for p in ce.include_paths():
        cmd += ["-isystem", p]
    cmd += ["-L", tlib, "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
            "-L", os.path.dirname(kernel_lib), "-l" + libname,
            f"-Wl,-rpath,{tlib}", "-Wl,-rpath," + ("$ORIGIN/../flashck_amd" if kernel_lib == lib_build.LIB else os.path.dirname(kernel_lib))]
    cmd += list(extra)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the flash_ck module failed:\n" + r.stdout[-6000:])
    os.replace(out + ".tmp", out)
    return out


if __name__ == "__main__":
    sys.path.insert(0, ROOT)
    print(build())
