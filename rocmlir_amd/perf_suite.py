"""Times lists of problems written in the reference's benchmark-config grammar.

The counterpart of mlir/utils/performance/perfRunner.py for this library: the
same three kinds of config lines are accepted,

  gemm        "-transA false -transB false -g 64 -m 1024 -n 384 -k 1024"
              (rocmlir-gen flags; getGemmConfigurations, perfRunner.py:546-588,
              adds "-t <type>")
  attention   "-transK true -t f16 -g 128 -seq_len_q 2048 -seq_len_k 2048
               -head_dim_qk 128 -head_dim_v 128"   (perfRunner.py:590-622)
  conv        "-n 256 -c 128 -H 28 -W 28 -k 128 -y 3 -x 3 -p 1 -q 1 -u 1 -v 1
               -l 1 -j 1 -g 1 -m conv -t 1"        (MIOpenDriver letters,
              perfRunner.py:261-307,387-470; layouts from --layouts; -F 1,
              2 or 4, or --direction, picks forward, backward data, backward weight)

every problem goes through the C ABI, is timed with HIP events on synthetic
data, and is reported with the reference's FLOP formulas
(perfRunner.py:313-316, 627-630, 759-777).  Problems the library has no
kernel for are listed with the library's error message, not skipped silently.

  python -m rocmlir_amd.perf_suite --op gemm --types f16,i8 FILE

With --tune quick|full|exhaustive every problem is also run under each entry of
its tuning space (what mlir/utils/performance/tuningRunner.py does over the
same lists with rocmlir-tuning-driver): the line then carries the fastest
perf_config, its kernel and time next to the built-in choice, and --table PATH
saves the winners in the reference's tab-separated ".tuning" form.
"""
import argparse
import json
import shlex
import sys
import time


def _flags(line):
    """'-a 1 -b x' -> {'a': '1', 'b': 'x'} (single or double dash)."""
    toks = shlex.split(line)
    out = {}
    i = 0
    while i < len(toks):
        t = toks[i]
        if t.startswith("-") and i + 1 < len(toks) and not toks[i + 1].startswith("--"):
            out[t.lstrip("-")] = toks[i + 1]
            i += 2
        else:
            i += 1
    return out


def _torch_dtype(torch, t):
    return {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "i8": torch.int8,
            "fp8": torch.float8_e4m3fn, "bf8": torch.float8_e5m2, "i32": torch.int32}[t]


def _rand(torch, shape, t, dev):
    if t == "i8":
        return torch.randint(-128, 128, shape, device=dev, dtype=torch.int8)
    return torch.randn(shape, device=dev).to(_torch_dtype(torch, t))


def _out_type(t):
    return {"i8": "i32", "fp8": "f32", "bf8": "f32"}.get(t, t)


def gemm_problem(line, t):
    f = _flags(line)
    t = f.get("t", t)
    opts = "-operation gemm -arch gfx950 -t %s -out_datatype %s -g %s -m %s -n %s -k %s -transA %s -transB %s" % (
        t, f.get("out_datatype", _out_type(t)), f.get("g", "1"), f["m"], f["n"], f["k"],
        f.get("transA", "false"), f.get("transB", "false"))
    g, m, n, k = int(f.get("g", 1)), int(f["m"]), int(f["n"]), int(f["k"])
    # pointer order A, B, C, bias
    shapes = [((g * m * k,), t), ((g * k * n,), t), ((g * m * n,), f.get("out_datatype", _out_type(t))), None]
    return opts, shapes, 2.0 * g * m * n * k


def attention_problem(line, t):
    f = _flags(line)
    t = f.get("t", t)
    g, sq, sk = int(f.get("g", 1)), int(f["seq_len_q"]), int(f["seq_len_k"])
    dqk, dv = int(f["head_dim_qk"]), int(f["head_dim_v"])
    opts = ("-operation attention -arch gfx950 -t %s -g %d -seq_len_q %d -seq_len_k %d -head_dim_qk %d "
            "-head_dim_v %d -transQ %s -transK %s -transV %s -transO %s -scale %.9g"
            % (t, g, sq, sk, dqk, dv, f.get("transQ", "false"), f.get("transK", "false"),
               f.get("transV", "false"), f.get("transO", "false"), dqk ** -0.5))
    # pointer order Q, K, V, bias, O
    shapes = [((g * sq * dqk,), t), ((g * sk * dqk,), t), ((g * sk * dv,), t), None, ((g * sq * dv,), t)]
    return opts, shapes, 2.0 * g * sq * sk * (dqk + dv)


_CONV_TYPES = {"conv": "f32", "convfp16": "f16", "convbfp16": "bf16", "convint8": "i8"}
_LAYOUTS = {"NCHW": ("gkcyx", "ngchw", "ngkhw"), "NHWC": ("gkyxc", "nhwgc", "nhwgk")}


def conv_problem(line, t, layout, direction_flag=None):
    if direction_flag:
        line = line + " -F " + direction_flag
    toks = shlex.split(line)
    if toks and not toks[0].startswith("-"):  # leading "convfp16"-style type word
        t = _CONV_TYPES.get(toks[0], t)
    f = _flags(line)
    direction = {"1": "conv", "2": "conv_bwd_data", "4": "conv_bwd_weight"}.get(f.get("F", "1"))
    if direction is None:
        raise ValueError("-F must be 1 (forward), 2 (backward data) or 4 (backward weight)")
    fl, il, ol = _LAYOUTS[layout]
    n, c, hi, wi, k = int(f["n"]), int(f["c"]), int(f["H"]), int(f["W"]), int(f["k"])
    y, x, g = int(f["y"]), int(f["x"]), int(f.get("g", 1))
    ph, pw, sh, sw = int(f.get("p", 0)), int(f.get("q", 0)), int(f.get("u", 1)), int(f.get("v", 1))
    dh, dw = int(f.get("l", 1)), int(f.get("j", 1))
    ho = (hi + 2 * ph - (y - 1) * dh - 1) // sh + 1
    wo = (wi + 2 * pw - (x - 1) * dw - 1) // sw + 1
    name = {"f32": "f32", "f16": "fp16", "bf16": "bf16", "i8": "i8"}[t]
    opts = ("--operation " + direction + " --arch gfx950 --in_type %s --fil_type %s --out_type %s --fil_layout %s --in_layout %s "
            "--out_layout %s --batchsize %d --groupsize %d --in_channels %d --out_channels %d --in_h %d --in_w %d "
            "--fil_h %d --fil_w %d --dilation_h %d --dilation_w %d --conv_stride_h %d --conv_stride_w %d "
            "--padding_h %d --padding_w %d"
            % (name, name, {"i8": "i32"}.get(t, name), fl, il, ol, n, g, c, k, hi, wi, y, x, dh, dw, sh, sw, ph, pw))
    # pointer order filter, input, output, bias; the written tensor comes last in `shapes`' order of use
    out_t = _out_type(t) if direction == "conv" else t
    shapes = [((k * (c // g) * y * x,), t), ((n * c * hi * wi,), t), ((n * k * ho * wo,), out_t), None]
    return opts, shapes, 2.0 * n * (c // g) * k * ho * wo * y * x


def run_problem(rock, torch, dev, opts, shapes, flops, warmup, iters, warm_ms=0.0, tune_kind=None, table=None,
                per_kernel=False):
    try:
        prog = rock.RockProgram(opts)  # every kernel of the problem and its workspace
    except rock.RockError as e:
        return {"status": "no kernel", "error": str(e).split(" [")[0]}
    # the last tensor in pointer order is left uninitialised (the forward output; for the
    # gradients every tensor holds some data, which is all timing needs); the bias slot stays empty
    last = max(i for i, s in enumerate(shapes) if s is not None)
    args = [None if s is None else
            torch.empty(s[0], device=dev, dtype=_torch_dtype(torch, s[1])) if i == last else _rand(torch, s[0], s[1], dev)
            for i, s in enumerate(shapes)]
    # the shader clock leaves its idle state only after some tens of milliseconds of load
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < warm_ms:
        for _ in range(10):
            prog.launch(*args)
        torch.cuda.synchronize()
    each = prog.benchmark_each(*args, warmup=warmup, iters=iters)
    ms = sum(t for _, t in each)
    contraction = [k.kernel_name for k in prog.kernels if k.kernel_name.startswith(("rock_conv", "rock_gemm",
                                                                                     "rock_attention"))]
    res = {"status": "ok", "kernel": contraction[-1], "kernels": len(prog.kernels), "ms": round(ms, 5),
           "tflops": round(flops / (ms * 1e-3) / 1e12, 2)}
    if len(prog.kernels) > 1:  # the list launched back to back, beside the sum of the kernels timed one by one
        res["sequence_ms"] = round(prog.benchmark_sequence(*args), 5)
    if per_kernel:
        res["kernel_ms"] = [[name, round(t, 5)] for name, t in each]
    if tune_kind:
        from .tuning import tune
        best = tune(prog, *args, table=table, warmup=warmup, iters=iters, kind=tune_kind)
        res.update({"tuned_perf_config": best[0][0], "tuned_kernel": best[0][1], "tuned_ms": round(best[0][2], 5),
                    "tuned_tflops": round(flops / (best[0][2] * 1e-3) / 1e12, 2), "candidates": len(best)})
    return res


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("file", help="config file in the reference's grammar, one problem per line")
    ap.add_argument("--op", choices=["gemm", "conv", "attention"], required=True)
    ap.add_argument("--types", default="f16", help="comma-separated element types for lines that name none")
    ap.add_argument("--layouts", default="NHWC", help="conv only: comma-separated subset of NHWC,NCHW")
    ap.add_argument("--direction", choices=["1", "2", "4"], default=None,
                    help="conv only: run every line forward (1), backward data (2) or backward weight (4)")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--warm-ms", type=float, default=30.0,
                    help="keep the GPU busy with the problem for this long before timing it (clock ramp-up)")
    ap.add_argument("--max-bytes", type=float, default=8e9, help="skip problems whose tensors exceed this")
    ap.add_argument("--extra-options", default="", help="appended to every problem string (plan switches, a perf_config)")
    ap.add_argument("--tune", choices=["quick", "full", "exhaustive"], default=None,
                    help="also time every entry of each problem's tuning space and report the fastest")
    ap.add_argument("--table", default=None, help="with --tune: save the winners as a .tuning table here")
    ap.add_argument("--per-kernel", action="store_true", help="list every kernel of a problem with its own time")
    args = ap.parse_args(argv)

    import torch
    import rocmlir_amd as rock
    rock.load_library()
    table = None
    if args.tune and args.table:
        from .tuning import TuningTable
        table = TuningTable()
    dev = torch.device("cuda:0")
    lines = [l.strip() for l in open(args.file) if l.strip() and not l.lstrip().startswith("#")]
    seen = set()
    for line in lines:
        for t in args.types.split(","):
            for layout in (args.layouts.split(",") if args.op == "conv" else [None]):
                try:
                    if args.op == "gemm":
                        opts, shapes, flops = gemm_problem(line, t)
                    elif args.op == "attention":
                        opts, shapes, flops = attention_problem(line, t)
                    else:
                        opts, shapes, flops = conv_problem(line, t, layout, args.direction)
                except (KeyError, ValueError) as e:
                    print(json.dumps({"config": line, "status": "unparsed", "error": str(e)}), flush=True)
                    continue
                if args.extra_options:
                    opts += " " + args.extra_options
                if opts in seen:
                    continue
                seen.add(opts)
                nbytes = sum(torch.empty(0, dtype=_torch_dtype(torch, s[1])).element_size() * s[0][0]
                             for s in shapes if s is not None)
                if nbytes > args.max_bytes:
                    print(json.dumps({"problem": opts, "status": "skipped", "bytes": nbytes}), flush=True)
                    continue
                res = run_problem(rock, torch, dev, opts, shapes, flops, args.warmup, args.iters, args.warm_ms,
                                  args.tune, table, args.per_kernel)
                res["problem"] = opts
                print(json.dumps(res), flush=True)
                torch.cuda.empty_cache()
    if table is not None:
        table.save(args.table)
    return 0


if __name__ == "__main__":
    sys.exit(main())
