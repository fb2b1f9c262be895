"""Which kernel instantiations of the device build does the test suite launch?

    python tests/emu/kernel_coverage.py            # runs the emulator suite (about ten minutes), then reports
    python tests/emu/kernel_coverage.py FILE ...   # reports on coverage files written earlier (EMU_COVERAGE=FILE)

The kernels are templates; a library of 300 instantiations can pass every test with a third of them never run.  The
emulator's launch hook appends the mangled name of every instantiation a process launches to the file EMU_COVERAGE
names; this script compares those names with the kernels of the device build (the `.amdhsa_kernel` entries of
`hipcc -S --cuda-device-only` over the sources of flashck_amd/build.py) and lists what was never launched.  Exit status 1
when something was not."""
import concurrent.futures
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

# without the six prefill cases that are hours of emulation each (they launch nothing the others do not)
SLOW = "not workload5_full and not midsize_every_row and not large_pool and not longer_than_the_page_cache"


def _demangle(names, types=False):
    r = subprocess.run(["c++filt"] + (["-t"] if types else []), input="\n".join(names), capture_output=True, text=True, check=True)
    return r.stdout.split("\n")


def _norm(name):
    name = re.sub(r"\(.*\)$", "", name.replace("void ", "").strip())   # no return type, no parameter list
    return re.sub(r"\s+", "", re.sub(r"\b\w+::", "", name))            # no namespaces, no blanks


def device_kernels():
    from flashck_amd import build
    out = set()
    with tempfile.TemporaryDirectory() as tmp:
        def one(src):
            asm = os.path.join(tmp, src + ".s")
            cmd = [build.hipcc(), "-x", "hip", "--cuda-device-only", "-S", os.path.join(build.CSRC, src), "-o", asm] + build.FLAGS
            subprocess.run(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, check=True)
            return re.findall(r"^\s*\.amdhsa_kernel\s+(\S+)", open(asm).read(), re.M)
        with concurrent.futures.ThreadPoolExecutor(8) as ex:
            for names in ex.map(one, [s for s in build.SOURCES if s.endswith(".hip")]):
                out.update(_norm(d) for d in _demangle(names) if d)
    return out


def launched(files):
    tags = set()
    for f in files:
        tags.update(open(f).read().split())
    out = set()
    for t in _demangle(sorted(tags), types=True):
        m = re.match(r"emu::KernelTag<&\(?(.*?)\)?>$", t)
        if m:
            out.add(_norm(m.group(1)))
    return out


def main(argv):
    files = argv
    if not files:
        fd, path = tempfile.mkstemp(suffix=".cov")
        os.close(fd)
        env = dict(os.environ, EMU_COVERAGE=path, FCK_EMU_FULL="1")
        cmd = [sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_emu_kernels.py"), "-q", "-n", "6", "-k", SLOW]
        r = subprocess.run(cmd, env=env, cwd=ROOT)
        if r.returncode != 0:
            return r.returncode
        files = [path]
    have, hit = device_kernels(), launched(files)
    miss = sorted(have - hit)
    print(f"kernels in the device build: {len(have)}; launched: {len(have & hit)}; never launched: {len(miss)}")
    for m in miss:
        print("  ", m)
    return 1 if miss else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
