"""Problems through the CPU build of the kernels, checked by the end-to-end harness's own comparisons with the
oracle (tests/test_gpu_e2e_lists.py with the model as its device).  Run from the repository root:

  python -m tests.kernel_host.sweep --lists all                 # the reference's end-to-end lists, batches capped
  python -m tests.kernel_host.sweep --random 500 --kinds conv   # random problems (conv, gemm, attention, and with a
                                                                # tile drawn from the tuning space: bigconv, biggemm)
  ... --types all --rolled    every operand type and the rolled-epilogue kernels (ten minutes of compilation,
                              kept in --build-dir and used again while the sources are unchanged)
  ... --late --order 2        loads land at the wait that covers them, waves take their turns rotated

One line per problem: ok / FAIL / refused, the kernels that ran, the options string to run it again."""
import argparse
import hashlib
import os
import random
import re
import sys
import time
import traceback

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

import rocmlir_amd as rock  # noqa: E402
import tests.test_gpu_e2e_lists as lists  # noqa: E402
from oracle import rock_oracle  # noqa: E402
from tests.kernel_host import model as km  # noqa: E402

LAYOUTS = [("gkcyx", "ngchw", "ngkhw"), ("gkyxc", "nhwgc", "nhwgk"), ("kcyx", "nchw", "nkhw"), ("kyxc", "nhwc", "nhwk"),
           ("yxck", "nhwc", "nhwk"), ("gkcyx", "nghwc", "ngchw"), ("gkyxc", "ngchw", "nghwc"), ("gyxck", "hwcgn", "nghwc"),
           ("gkcyx", "hwcgn", "hwcgn"), ("kyxc", "nhwc", "nkhw"), ("kcyx", "nchw", "nhwk")]
CONV = ("-groupsize=%d -batchsize=%d -in_channels=%d -out_channels=%d -in_h=%d -in_w=%d -fil_h=%d -fil_w=%d "
        "-dilation_h=%d -dilation_w=%d -conv_stride_h=%d -conv_stride_w=%d -padding_h_l=%d -padding_h_r=%d "
        "-padding_w_l=%d -padding_w_r=%d --operation %s -fil_layout=%s -in_layout=%s -out_layout=%s -t %s -arch gfx950")


def conv_problem(R):
    while True:
        op = R.choice(["conv", "conv", "conv_bwd_data", "conv_bwd_weight"])
        t = R.choice(["f32", "f16", "f16", "bf16"] + (["i8"] if op == "conv" else []))
        fl, il, ol = R.choice(LAYOUTS)
        g = R.choice([1, 1, 1, 2, 4]) if "g" in fl else 1
        chan = lambda: R.choice([1, 2, 3, 4, 5, 7, 8, 8, 16, 16, 24, 32, 32, 40, 64, 64, 72, 96, 128])
        c, k = chan(), chan()
        hi, wi = R.randint(1, 30), R.randint(1, 30)
        y, x = R.choice([1, 1, 2, 3, 3, 5, 7]), R.choice([1, 1, 2, 3, 3, 5, 7])
        sh, sw = R.choice([1, 1, 1, 2, 2, 3]), R.choice([1, 1, 1, 2, 2, 3])
        dh, dw = R.choice([1, 1, 1, 2]), R.choice([1, 1, 1, 2])
        phl, pwl = R.choice([0, 0, 1, 1, 2, 3]), R.choice([0, 0, 1, 1, 2, 3])
        # (the backward kernels take equal padding on both sides)
        phr, pwr = (phl, pwl) if (op != "conv" or R.random() < 0.8) else (R.choice([0, 1, 2]), R.choice([0, 1, 2]))
        n = R.randint(1, 4)
        eh, ew = hi + phl + phr - (y - 1) * dh - 1, wi + pwl + pwr - (x - 1) * dw - 1
        if eh < 0 or ew < 0 or n * g * c * k * (eh // sh + 1) * (ew // sw + 1) * y * x > 6e7:
            continue
        return CONV % (g, n, g * c, g * k, hi, wi, y, x, dh, dw, sh, sw, phl, phr, pwl, pwr, op, fl, il, ol, t)


def big_conv_problem(R):
    op = R.choice(["conv", "conv", "conv_bwd_data", "conv_bwd_weight"])
    t = R.choice(["f32", "f16", "f16", "bf16"] + (["i8"] if op == "conv" else []))
    fl, il, ol = R.choice(LAYOUTS[:4] + [("kyxc", "nhwc", "nkhw")])
    c, k = R.choice([64, 128, 128, 256]), R.choice([64, 128, 128, 256, 96])
    hw, f, s = R.choice([14, 28, 28, 56, 12, 20]), R.choice([1, 3, 3]), R.choice([1, 1, 1, 2])
    return CONV % (1, R.choice([1, 2]), c, k, hw, hw, f, f, 1, 1, s, s, f // 2, f // 2, f // 2, f // 2, op, fl, il, ol, t)


def gemm_problem(R):
    t = R.choice(["f32", "f16", "f16", "bf16", "i8", "fp8_fp8", "fp8_bf8", "bf8_fp8", "bf8_bf8"])
    m, n, k = R.randint(1, 300), R.randint(1, 300), R.randint(1, 400)
    if R.random() < 0.4:
        m, n, k = (R.choice([32, 64, 128, 256]) for _ in range(3))
    return ("-g %d -m %d -n %d -k %d --operation gemm -transA=%s -transB=%s -transC=%s -t %s -arch gfx950"
            % (R.choice([1, 1, 2, 3]), m, n, k, R.choice(["true", "false"]), R.choice(["true", "false"]),
               R.choice(["false", "false", "true"]), t))


def big_gemm_problem(R):
    t = R.choice(["f32", "f16", "f16", "bf16", "i8", "fp8_fp8", "bf8_bf8"])
    return ("-g 1 -m %d -n %d -k %d --operation gemm -transA=%s -transB=%s -transC=false -t %s -arch gfx950"
            % (R.choice([256, 300, 512, 520]), R.choice([256, 300, 512, 130]), R.choice([64, 128, 200, 256]),
               R.choice(["true", "false"]), R.choice(["true", "false"]), t))


def attention_problem(R):
    t = R.choice(["f16", "f16", "f32", "i8"])
    d = R.choice([32, 64, 64, 128, 128, 40, 256]) if t != "i8" else R.choice([64, 128])
    dv = d if R.random() < 0.7 else R.choice([32, 64, 128])
    flags = " ".join(f for f in ("--with-attn-scale", "--with-attn-bias") if R.random() < 0.3)
    trans = " ".join("--trans%s=%s" % (n, R.choice(["true", "false"])) for n in ("K",) + (("Q", "V", "O") if R.random() < 0.3 else ()))
    return ("-g %d -seq_len_q %d -seq_len_k %d -head_dim_qk %d -head_dim_v %d %s %s --operation attention -t %s -arch gfx950"
            % (R.choice([1, 2, 3]), R.randint(1, 300), R.randint(1, 300), d, dv, flags, trans, t))


def with_tile(make):
    def problem(R):
        opts = make(R)
        try:
            space = rock.RockKernel(opts).tuning_space("full")
        except rock.RockError:
            return opts
        return opts + " -perf_config " + R.choice(space) if space else opts
    return problem


KINDS = {"conv": conv_problem, "gemm": gemm_problem, "attention": attention_problem,
         "bigconv": with_tile(big_conv_problem), "biggemm": with_tile(big_gemm_problem)}


def source_stamp():
    h = hashlib.sha1()
    for d in (km.CSRC, km.HOST):
        for root, _, files in sorted(os.walk(d)):
            for f in sorted(files):
                if f.endswith((".h", ".hip", ".cpp", ".py")):
                    h.update(open(os.path.join(root, f), "rb").read())
    return h.hexdigest()[:16]


def check(device, opts, gen, have):
    o = lists.parse_options(opts)
    op = o.get("operation", "")
    t = {"fp16": "f16", "fp32": "f32"}.get(o.get("t") or o.get("in_type") or "f32", o.get("t") or o.get("in_type") or "f32")
    if op == "attention" and t == "i8":   # (the int8 attention kernels come with the attention kernels, V is f16)
        t = "f16"
    if not set(t.split("_")) <= have:
        return "skipped (type %s is not in this build of the model)" % t
    try:
        rock.RockKernel(opts)
    except rock.RockError as e:
        return "refused: " + str(e)[:80]
    t0 = time.time()
    device.kernels = []
    try:
        (lists.run_gemm if op == "gemm" else lists.run_attention if op == "attention" else lists.run_conv)(
            device, rock_oracle, "cpu", gen, opts, o)
        return "ok %.1fs %s" % (time.time() - t0, device.kernels)
    except AssertionError as e:
        return "FAIL %s %s" % (device.kernels, str(e)[:400].replace("\n", " "))
    except Exception as e:   # a problem the harness cannot set up is a finding too
        traceback.print_exc(limit=4)
        return "FAIL %r" % (e,)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--lists", default="", help="comma-separated list names of tests/golden/e2e_problems.json, or all")
    ap.add_argument("--batch", type=int, default=2, help="cap on the batch size of listed convolutions")
    ap.add_argument("--shrink-gemm", action="store_true", help="listed GEMMs with M and N a quarter, K a half")
    ap.add_argument("--random", type=int, default=0, help="number of random problems")
    ap.add_argument("--kinds", default="conv,gemm,attention")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--types", default="f32,f16", help="operand types of the build, or all")
    ap.add_argument("--rolled", action="store_true", help="build the rolled-epilogue kernels too")
    ap.add_argument("--late", action="store_true", help="loads into LDS land at the wait that covers them")
    ap.add_argument("--order", type=int, default=0, help="0 ascending, 1 descending, 2 waves rotated per pass")
    ap.add_argument("--build-dir", default=os.path.join(os.environ.get("TMPDIR", "/tmp"), "rock_kernel_host"))
    a = ap.parse_args()
    names = {v: k for k, v in km._build.GEMM_TYPES.items()}
    types = km.ALL_TYPES if a.types == "all" else tuple(names[t] for t in a.types.split(","))
    d = os.path.join(a.build_dir, "%s-%s-%d" % (source_stamp(), "_".join(str(t) for t in types), a.rolled))
    so = os.path.join(d, "libkernel_host.so")
    if os.path.exists(so):
        model = km.load_model(so)
    else:
        os.makedirs(d, exist_ok=True)
        print("building the model in", d, flush=True)
        model = km.build_model(d, types=types, rolled=a.rolled)
    model.hm_set_late_loads(1 if a.late else 0)
    model.hm_set_thread_order(a.order)
    have = set()
    for t in types:
        have |= set(km._build.GEMM_TYPES[t].split("_"))
    device = km.harness_device(model, rock)
    bad = 0
    wanted = sorted(lists._BY_LIST) if a.lists == "all" else [n for n in a.lists.split(",") if n]
    for name in wanted:
        gen = torch.Generator(device="cpu")
        gen.manual_seed(1234)
        for i, opts in enumerate(lists._BY_LIST[name]):
            opts = re.sub(r"-batchsize[= ](\d+)", lambda m: "-batchsize=%d" % min(int(m.group(1)), a.batch), opts)
            if a.shrink_gemm and "--operation gemm" in opts:
                opts = re.sub(r"-(m|n) (\d+)", lambda m: "-%s %d" % (m.group(1), max(1, int(m.group(2)) // 4)), opts)
                opts = re.sub(r"-k (\d+)", lambda m: "-k %d" % max(1, int(m.group(1)) // 2), opts)
            verdict = check(device, opts, gen, have)
            bad += verdict.startswith("FAIL")
            print(name, i, verdict, "|", opts if not verdict.startswith("ok") else "", flush=True)
    R = random.Random(a.seed)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(a.seed)
    for i in range(a.random):
        opts = KINDS[R.choice(a.kinds.split(","))](R)
        verdict = check(device, opts, gen, have)
        bad += verdict.startswith("FAIL")
        print(i, verdict, "|", opts if not verdict.startswith("ok") else "", flush=True)
    print("failures:", bad)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
