"""Extracts the known-answer vectors the reference's fusion tests hold for a
contraction followed by fused element-wise operations
(mlir/test/fusion/pr-e2e/: the FileCheck literal, the data fill named on the
RUN line, and the shapes of the migraphx.dot / convolution) into
fusion_kats.json.  Run in the build container, where /root/reference is
mounted; the JSON (data only) is what the tests read.

    python tests/golden/make_fusion_kats.py
"""
import json
import os
import re

REF = "/root/reference/mlir/test/fusion/pr-e2e"
# file, operation, fused tail as this library's epilogue spells it
FILES = [
    ("mixr-gemm/mixr-gemm-add.e2e.mlir", "gemm", {"residual": "add"}),
    ("mixr-gemm/mixr-gemm-bcast-add.e2e.mlir", "gemm", {"bias": True}),
    ("mixr-gemm/mixr-gemm-erf_f32.mlir", "gemm", {"activation": "erf"}),
    ("mixr-gemm/mixr-gemm-erf_f16.mlir", "gemm", {"activation": "erf"}),
    ("mixr-bcast-add.e2e.mlir", "conv", {"bias": True}),
]


def main():
    cases = []
    for fname, op, tail in FILES:
        text = open(os.path.join(REF, fname)).read()
        run = next(l for l in text.splitlines() if l.startswith("// RUN:"))
        rand = re.search(r"-rand (\w+)", run).group(1)
        check = next(l for l in text.splitlines() if re.search(r"// CHECK:\s", l))
        expected = [float(v) for v in re.findall(r"-?\d+(?:\.\d+)?(?:e[-+]?\d+)?", check.split("CHECK:")[1])]
        case = {"source": fname, "operation": op, "rand": rand, "tail": tail, "expected": expected}
        if op == "gemm":
            m = re.search(r"migraphx\.dot .*?<(\d+)x(\d+)x(\d+)x(f\d+),.*?<\d+x\d+x(\d+)xf\d+,", text)
            case.update(g=int(m.group(1)), m=int(m.group(2)), k=int(m.group(3)), t=m.group(4), n=int(m.group(5)))
        else:
            m = re.search(r"migraphx\.convolution .*?<(\d+)x(\d+)x(\d+)x(\d+)x(f\d+),.*?<(\d+)x\d+x(\d+)x(\d+)xf\d+,",
                          text)
            case.update(n=int(m.group(1)), c=int(m.group(2)), hi=int(m.group(3)), wi=int(m.group(4)),
                        t=m.group(5), k=int(m.group(6)), y=int(m.group(7)), x=int(m.group(8)))
        cases.append(case)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fusion_kats.json")
    with open(out, "w") as f:
        json.dump(cases, f, separators=(",", ":"))
    print("wrote %d cases to %s" % (len(cases), out))


if __name__ == "__main__":
    main()
