"""Static check of the device assembly of attention.hip.

attn_fwd_w64_kernel keeps its O^T accumulators and Q fragments in accumulation registers that it
names by number inside inline asm; the compiler does not know they are live. That is sound only if
the compiler (1) never touches an accumulation register itself, which it would do to spill vector
registers, and (2) spills nothing to scratch memory (scratch traffic shares the counter the kernel
uses to wait for its own LDS-writing loads). Both are properties of the generated code, so they are
checked on it: every instantiation of the kernel, every line outside the asm blocks.

usage: check_attention_isa.py <attention device assembly (.s)>; exit status 1 on a violation.
"""
import re
import sys

KERNEL = "attn_fwd_w64_kernel"


def kernels(path):
    """{mangled name: [lines]} of every instantiation of the kernel in a device .s file."""
    out, cur = {}, None
    for line in open(path):
        m = re.match(r"^(_Z\w*%s\w*):" % KERNEL, line)
        if m:
            cur = out.setdefault(m.group(1), [])
        if cur is not None:
            cur.append(line.rstrip("\n"))
            if "s_endpgm" in line:
                cur = None
    return out


def violations(lines):
    errs, in_asm = [], False
    for i, line in enumerate(lines):
        if "ASMSTART" in line:
            in_asm = True
        elif "ASMEND" in line:
            in_asm = False
        elif not in_asm and re.search(r"\bv_accvgpr|\ba\[?\d", line.split(";")[0]):
            errs.append("accumulation register outside asm, line %d: %s" % (i, line.strip()))
        if "scratch_" in line.split(";")[0]:
            errs.append("scratch access, line %d: %s" % (i, line.strip()))
    return errs


def check(path):
    ks = kernels(path)
    if not ks:
        return ["no instantiation of %s in %s" % (KERNEL, path)]
    errs = []
    for name, lines in ks.items():
        errs += ["%s: %s" % (name, e) for e in violations(lines)]
    return errs


if __name__ == "__main__":
    e = check(sys.argv[1])
    for x in e[:10]:
        print(x)
    print("%s: %d instantiation(s) of %s, %d violation(s)" % (sys.argv[1], len(kernels(sys.argv[1])), KERNEL, len(e)))
    sys.exit(1 if e else 0)
