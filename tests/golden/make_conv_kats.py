"""Extracts the convolution known-answer vectors that the reference's own CPU
tests hold (mlir/test/rocmlir-driver/cpu_conv2d/*.mlir: the RUN line's
problem flags and the literal output vector FileCheck expects) into
conv_fwd_kats.json (forward) and conv_bwd_kats.json (backward data and
backward weight; flags carry the operation).  Run in the build container, where /root/reference is
mounted; the JSON (data only) is what the tests read.

    python tests/golden/make_conv_kats.py
"""
import json
import os
import re

REF = "/root/reference/mlir/test/rocmlir-driver/cpu_conv2d"
FILES = ["kyxc_nhwc_nhwk_fwd.mlir", "kcyx_nchw_nkhw_fwd.mlir"]
BWD_FILES = ["kyxc_nhwc_nhwk_bwd_data.mlir", "kcyx_nchw_nkhw_bwd_data.mlir",
             "kyxc_nhwc_nhwk_bwd_weight.mlir", "kcyx_nchw_nkhw_bwd_weight.mlir"]
FLAGS = ["fil_layout", "in_layout", "out_layout", "batchsize", "in_channels",
         "out_channels", "in_h", "in_w", "fil_h", "fil_w", "dilation_h",
         "dilation_w", "padding_h", "padding_w", "conv_stride_h",
         "conv_stride_w", "groupsize", "rand", "t", "operation"]


def extract(files, out_name):
    cases = []
    for fname in files:
        text = open(os.path.join(REF, fname)).read().splitlines()
        pending = None
        for line in text:
            if line.startswith("// RUN:"):
                flags = {}
                for key in FLAGS:
                    m = re.search(r"-{1,2}%s[= ]([^ ]+)" % key, line)
                    if m:
                        flags[key] = m.group(1)
                prefix = re.search(r"--check-prefix=(\w+)", line).group(1)
                pending = {"source": "%s:%s" % (fname, prefix), "flags": flags}
            m = re.match(r"// (\w+)-NEXT\{LITERAL\}:\s*\[(.*)\]", line)
            if m and pending is not None:
                pending["expected"] = [float(v) for v in m.group(2).split(",")]
                cases.append(pending)
                pending = None
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), out_name)
    with open(out, "w") as f:
        json.dump(cases, f, separators=(",", ":"))
    print("wrote %d cases to %s" % (len(cases), out))


def main():
    extract(FILES, "conv_fwd_kats.json")
    extract(BWD_FILES, "conv_bwd_kats.json")


if __name__ == "__main__":
    main()
