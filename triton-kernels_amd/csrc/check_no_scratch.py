"""Static check of a device assembly file: the named kernels must not spill to scratch memory.

The tiled GEMM runs at 254 of 256 vector registers with all 256 accumulation registers taken. A
source change that keeps a few more values alive makes the compiler spill, and a kernel that touches
scratch memory at all runs several times slower here (measured: six times), with correct results, so
no parity test would notice. The build therefore checks the generated code.

usage: check_no_scratch.py <device assembly (.s)> <kernel name substring>; exit status 1 on a violation.
"""
import re
import sys


def kernels(path, name):
    """{mangled name: [lines]} of every kernel whose mangled name contains `name`."""
    out, cur = {}, None
    for line in open(path):
        m = re.match(r"^(_Z\w*%s\w*):" % re.escape(name), line)
        if m:
            cur = out.setdefault(m.group(1), [])
        if cur is not None:
            cur.append(line.rstrip("\n"))
            if "s_endpgm" in line:
                cur = None
    return out


def check(path, name):
    ks = kernels(path, name)
    if not ks:
        return ["no kernel matching %s in %s" % (name, path)]
    errs = []
    for k, lines in ks.items():
        n = sum(1 for l in lines if "scratch_" in l.split(";")[0])
        if n:
            errs.append("%s: %d scratch accesses" % (k, n))
    return errs


if __name__ == "__main__":
    e = check(sys.argv[1], sys.argv[2])
    for x in e:
        print(x)
    print("%s: %d kernel(s) matching %s, %d with scratch accesses" % (sys.argv[1], len(kernels(sys.argv[1], sys.argv[2])), sys.argv[2], len(e)))
    sys.exit(1 if e else 0)
