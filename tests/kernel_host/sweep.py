"""Problems through the CPU build of the kernels, checked by the end-to-end harness's own comparisons with the
oracle (tests/test_gpu_e2e_lists.py with the model as its device).  Run from the repository root:

  python -m tests.kernel_host.sweep --lists all                 # the reference's end-to-end lists, batches capped
  python -m tests.kernel_host.sweep --random 500 --kinds conv   # random problems (conv, gemm, attention, and with a
                                                                # tile drawn from the tuning space: bigconv, biggemm)
  ... --types all --rolled    every operand type and the rolled-epilogue kernels (ten minutes of compilation,
                              kept in --build-dir and used again while the sources are unchanged)
  ... --late --order 2        loads land at the wait that covers them, waves take their turns rotated
  ... --owners                every launch is checked for bytes that two of its blocks change
  python -m tests.kernel_host.sweep --boundary                  # tensors just below and at 2 GiB, their last tiles only

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
    for d in (km.CSRC, km.HOST):   # the kernels' sources (not the host library's), the stand-in, the runner
        for root, _, files in sorted(os.walk(d)):
            for f in sorted(files):
                if f.endswith((".h", ".hip")) or (d == km.HOST and (f.endswith(".cpp") or f == "model.py")):
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


def _last_tiles(model, opts, fill, blocks, order_at):
    """Runs the last `blocks` blocks of every kernel of the plan, the tiles taken in plain order (order_at: byte
    offset of group_m in the contraction kernel's parameter block, checked against the sizes in front of it)."""
    import ctypes as C
    import struct
    import numpy as np
    first = rock.RockKernel(opts)
    kernels = [first] + [rock.RockKernel("%s --kernel_id %d" % (opts, i)) for i in range(1, first.kernel_count)]
    model.hm_clear()
    tensors = []
    for i, (dt, dims) in enumerate(first.arguments()):
        nbytes = max(int(np.prod(dims, dtype=np.int64)) * (1 if dt < 0 else km._DTYPE_BYTES[dt]), 16)
        at = model.hm_alloc(nbytes, b"argument %d" % i)
        tensors.append((at, nbytes, np.ctypeslib.as_array((C.c_uint8 * nbytes).from_address(at))))
    fill([v for _, _, v in tensors])
    problems = []
    for k in kernels:
        params = bytearray(k.params())
        if k.kernel_name.startswith(("rock_conv_", "rock_gemm_")):
            tiles_m, tiles_n = struct.unpack_from("<2i", params, order_at - 8)
            assert tiles_m * tiles_n in (k.grid_size, k.grid_size // max(1, struct.unpack_from("<i", params, 72)[0])), \
                "the parameter block is not laid out as this probe assumes"
            struct.pack_into("<2i", params, order_at, 1, 0)   # group_m = 1, xcd_remap = 0
        ptrs = (C.c_void_p * 8)()
        for j, (src, off) in enumerate(km.pointer_map(rock, k)):
            ptrs[j] = None if src < 0 else tensors[src][0] + off
        model.hm_set_blocks(max(0, k.grid_size - blocks), blocks)
        text = C.create_string_buffer(512)
        bad = model.hm_run(k.kernel_name.encode(), bytes(params), ptrs, k.grid_size, k.block_size, text, 512)
        model.hm_set_blocks(0, 0xFFFFFFFF)
        if bad:
            problems.append("%s: %s" % (k.kernel_name, text.value.decode()))
        problems += ["%s wrote beside argument %d" % (k.kernel_name, i) for i, (at, n, _) in enumerate(tensors)
                     if model.hm_canaries(at, n)]
    return [k.kernel_name for k in kernels], problems, [v for _, _, v in tensors]


def boundary(model):
    """The direct-to-LDS loads address a 2 GiB window behind a base pointer, and the planners send a tensor that
    does not fit to the kernels with 64-bit addressing: a convolution input and a K-major GEMM operand of just
    under and of exactly 2 GiB, the last tiles of each (highest offsets), results against the oracle / numpy."""
    import numpy as np
    bad = 0
    rng = np.random.default_rng(0)
    c = k = 64
    hw, f = 16, 3
    img = hw * hw * c
    W = rng.integers(-2, 3, k * c * f * f).astype(np.float16)
    X3 = rng.integers(-2, 3, 3 * img).astype(np.float16)   # the last three images hold data, the rest zeros
    ref = rock_oracle.conv_fwd(W.astype(np.float32), X3.astype(np.float32), "gkyxc", "nhwgc", "nhwgk", 3, 1, c, k, hw, hw,
                               f, f, stride=(1, 1), pad=(1, 1), dil=(1, 1))[0]
    ref = np.asarray(ref).reshape(3, hw * hw * k)[2].astype(np.float16)
    for n, expect in ((65534, "rock_conv_f16_64x64_fast"), (65536, "rock_conv_f16_64x64_generic")):
        opts = CONV % (1, n, c, k, hw, hw, f, f, 1, 1, 1, 1, 1, 1, 1, 1, "conv", "kyxc", "nhwc", "nhwk", "f16")

        def fill(t):
            t[0][:W.nbytes] = W.view(np.uint8)
            t[1][:] = 0
            t[1][(n - 3) * img * 2:n * img * 2] = X3.view(np.uint8)
        names, problems, out = _last_tiles(model, opts, fill, 8, 204)
        got = out[2][(n - 1) * hw * hw * k * 2:n * hw * hw * k * 2].view(np.float16)
        ok = names[-1] == expect and not problems and np.array_equal(got.astype(np.float32), ref.astype(np.float32))
        bad += not ok
        print("convolution input of %d bytes:" % (n * img * 2), "ok" if ok else "FAIL", names, problems, flush=True)
    M, K = 64, 32768
    A = rng.integers(-2, 3, (M, K)).astype(np.float16)
    for N, expect in ((32760, "rock_gemm_f16_64x64_fast_nn"), (32768, "rock_gemm_f16_64x64_generic")):
        B = rng.integers(-2, 3, (K, N), dtype=np.int8).astype(np.float16)
        opts = "-operation gemm -arch gfx950 -t f16 -g 1 -m %d -n %d -k %d -transA false -transB false" % (M, N, K)

        def fill(t):
            t[0][:A.nbytes] = A.view(np.uint8).ravel()
            t[1][:B.nbytes] = B.view(np.uint8).ravel()
        names, problems, out = _last_tiles(model, opts, fill, 2, 96)
        got = out[2][:M * N * 2].view(np.float16).reshape(M, N)[:, -64:].astype(np.float64)
        want = A.astype(np.float64) @ B[:, -64:].astype(np.float64)
        ok = names[-1] == expect and not problems and np.array_equal(got, want)
        bad += not ok
        print("GEMM operand of %d bytes:" % B.nbytes, "ok" if ok else "FAIL", names, problems, flush=True)
    return bad


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
    ap.add_argument("--owners", action="store_true", help="report a byte that two blocks of one launch change")
    ap.add_argument("--boundary", action="store_true", help="tensors just below and at 2 GiB (needs about 10 GB of memory)")
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
    model.hm_set_owner_check(1 if a.owners else 0)
    have = set()
    for t in types:
        have |= set(km._build.GEMM_TYPES[t].split("_"))
    device = km.harness_device(model, rock)
    bad = boundary(model) if a.boundary else 0
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
