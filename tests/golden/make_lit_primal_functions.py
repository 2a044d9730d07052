"""Writes tests/golden/lit_primal_functions.json: the primal functions of the reference's StableHLO differentiation
lit tests (test/lit_tests/diffrules/stablehlo/*.mlir) as data.

Only the input programs are kept (one entry per `func.func` that holds no `enzyme.` operation or type, i.e. the
function a test differentiates, not the driver that calls `enzyme.fwddiff` / `enzyme.autodiff`); RUN and CHECK lines
are dropped.  Run in the build container, where /root/reference exists:
    python tests/golden/make_lit_primal_functions.py
"""
import glob
import json
import os
import re

SRC = "/root/reference/test/lit_tests/diffrules/stablehlo"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lit_primal_functions.json")


def functions(text):
    src = "\n".join(l for l in text.split("\n") if not l.strip().startswith("//"))
    out, i = [], 0
    while True:
        j = src.find("func.func", i)
        if j < 0:
            return out
        # the body is the brace group opened at the end of the signature's last line (argument attribute
        # dictionaries and quoted symbol names hold braces of their own)
        m = re.compile(r"\{[ \t]*\n").search(src, j)
        if m is None:
            return out
        p, depth, quoted = m.start(), 0, False
        while p < len(src):
            ch = src[p]
            if ch == '"':
                quoted = not quoted
            elif not quoted and ch == "{":
                depth += 1
            elif not quoted and ch == "}":
                depth -= 1
                if depth == 0:
                    break
            p += 1
        out.append(src[j:p + 1])
        i = p + 1


def main():
    data = {}
    for f in sorted(glob.glob(os.path.join(SRC, "*.mlir"))):
        fns = [fn for fn in functions(open(f).read()) if "enzyme." not in fn and "!enzyme" not in fn]
        if fns:
            data[os.path.basename(f)] = fns
    with open(OUT, "w") as fh:
        json.dump(data, fh, indent=1, sort_keys=True)
    print("%d files, %d functions -> %s" % (len(data), sum(len(v) for v in data.values()), OUT))


if __name__ == "__main__":
    main()
