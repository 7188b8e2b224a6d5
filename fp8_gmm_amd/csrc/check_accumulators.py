"""Build check for the grouped-GEMM kernels: nothing but their own statements may touch an accumulation register.

The kernels address the accumulation registers (a0 .. a255) by name inside inline assembly, so the compiler does
not know that they hold the accumulators of a tile.  It stays out of them as long as it has vector registers to
spare; if it ever runs short it may park a value there and the kernel would silently compute garbage.  This script
reads the device assembly of one translation unit and fails when an instruction OUTSIDE the inline-assembly blocks
names an accumulation register, or when the kernel spills vector registers to scratch memory.

usage: check_accumulators.py <file.s> [...]
"""
import re
import sys

ACC_REGISTER = re.compile(r"(?<![\w.$])a(\d+|\[)")


def check(path):
    in_asm = False
    bad = []
    spills = 0
    for number, line in enumerate(open(path), 1):
        if "ASMSTART" in line:
            in_asm = True
            continue
        if "ASMEND" in line:
            in_asm = False
            continue
        m = re.match(r"\s*\.vgpr_spill_count:\s*(\d+)", line)
        if m:
            spills = max(spills, int(m.group(1)))
        if in_asm:
            continue
        code = line.split(";")[0]
        if ACC_REGISTER.search(code) and not code.lstrip().startswith("."):
            bad.append((number, line.rstrip()))
    for number, line in bad[:10]:
        print(f"{path}:{number}: accumulation register used outside the kernel's own statements: {line.strip()}")
    if spills:
        print(f"{path}: {spills} vector registers spilled to scratch memory")
    return not bad and not spills


if __name__ == "__main__":
    ok = all([check(p) for p in sys.argv[1:]])
    sys.exit(0 if ok else 1)
