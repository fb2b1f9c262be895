"""Which lines of the kernels and of the C ABI does the test suite never execute?

    FCK_EMU_GCOV=1 FCK_EMU_FULL=1 python -m pytest tests/test_emu_kernels.py -n 6 -k "not zy_flash and <the slow cases>"
    python tests/emu/line_coverage.py [-v]

The first command runs the GPU tests on a build of the emulator library that counts lines and branches (clang --coverage;
tests/emu/build_emu.py with FCK_EMU_GCOV=1, objects and counters in tests/emu/build_gcov); this script runs gcov over the
counters and prints, for every source of flashck_amd/csrc, how many of its lines ran, and with -v the lines that never did.
Templates are counted once per line over all instantiations."""
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OBJ = os.path.join(HERE, "build_gcov")


def main(verbose):
    data = sorted(f for f in os.listdir(OBJ) if f.endswith(".gcda"))
    if not data:
        print("no counters in tests/emu/build_gcov: run the tests with FCK_EMU_GCOV=1 first")
        return 2
    lines = {}  # source -> {line number: executions}, merged over translation units
    text = {}
    with tempfile.TemporaryDirectory() as tmp:
        for d in data:
            subprocess.run(["gcov", "-o", OBJ, os.path.join(OBJ, d)], cwd=tmp, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL,
                           env=dict(os.environ, PWD=ROOT), check=False)
            subprocess.run(["gcov", "-s", ROOT, "-o", OBJ, os.path.join(OBJ, d)], cwd=ROOT, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, check=False)
            for g in [f for f in os.listdir(ROOT) if f.endswith(".gcov")]:
                path = os.path.join(ROOT, g)
                rows = open(path, errors="replace").read().splitlines()
                os.remove(path)
                src = rows[0].split("Source:", 1)[1] if rows and "Source:" in rows[0] else g
                if "flashck_amd/csrc" not in src:
                    continue
                name = os.path.basename(src)
                for r in rows:
                    m = re.match(r"\s*([0-9]+\*?|#####|=====|-):\s*(\d+):(.*)$", r)
                    if not m or m.group(1) == "-" or int(m.group(2)) == 0:
                        continue
                    n = 0 if m.group(1) in ("#####", "=====") else int(m.group(1).rstrip("*"))
                    ln = int(m.group(2))
                    lines.setdefault(name, {})[ln] = lines.get(name, {}).get(ln, 0) + n
                    text.setdefault(name, {})[ln] = m.group(3)
    total = missed = 0
    for name in sorted(lines):
        never = sorted(ln for ln, n in lines[name].items() if n == 0)
        total += len(lines[name])
        missed += len(never)
        print(f"{name:24s} {len(lines[name]) - len(never):5d} of {len(lines[name]):5d} lines executed")
        if verbose:
            for ln in never:
                print(f"    {ln:5d}: {text[name][ln].strip()[:140]}")
    print(f"{'all':24s} {total - missed:5d} of {total:5d} lines executed ({100.0 * (total - missed) / max(total, 1):.1f} %)")
    return 0


if __name__ == "__main__":
    sys.exit(main("-v" in sys.argv[1:]))
