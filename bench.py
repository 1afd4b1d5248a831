#!/usr/bin/env python3
"""Benchmark of the Rock-dialect contraction kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only-headline]

Headline workload (BASELINE.json configs[1]): int8 quantised GEMM
M=N=K=4096, A[M,K] x B[N,K]^T, int32 accumulate, f32 scale 0.01, f16 output.
A step is one launch of that kernel on inputs already resident in HBM.  The
JSON line also carries the other four BASELINE configurations (`per_config`),
the MFMA roofline of the headline kernel and the CPU validator's throughput
on the host cores (the oracle, timed on a bounded sample).

TFLOPS definitions follow the reference (mlir/utils/performance/perfRunner.py:
GEMM 2*g*m*k*n :627-630, conv 2*n*c*k*ho*wo*y*x :313-316, attention
4*g*sq*sk*d matmul-only :759-777).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published dense peaks (AMD CDNA4 data sheet), TFLOP/s or TOP/s
PEAK = {"i8": 5000.0, "fp8": 5000.0, "f16": 2500.0, "bf16": 2500.0, "f32": 157.3}


def make_configs(torch, rock, dev, seed=1):
    """The five BASELINE configurations: name -> dict(kernel launch closure,
    algorithmic ops, peak, cpu sample runner)."""
    import numpy as np
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    cfgs = {}

    def gemm_cfg(name, t, M, N, K, out_dtype=None, scale=None, make=None):
        a, b = make((M, K)), make((N, K))
        opts = ("-operation gemm -arch gfx950 -t %s -g 1 -m %d -n %d -k %d -transA false -transB true"
                " -transC false" % (t, M, N, K))
        if out_dtype:
            opts += " -out_datatype %s" % out_dtype
        if scale is not None:
            opts += " -scale %.9g" % scale
        kern = rock.RockKernel(opts)
        od = out_dtype or {"i8": "i32", "fp8": "f32"}.get(t, t)
        out = torch.empty((M, N), dtype=rock.api._torch_dtype(od), device=dev)
        cfgs[name] = dict(kernel=kern, args=(a, b, out, None), ops=2.0 * M * N * K, dtype=t,
                          peak=PEAK[t], shape=dict(op="gemm", t=t, M=M, N=N, K=K),
                          min_bytes=a.numel() * a.element_size() + b.numel() * b.element_size()
                          + out.numel() * out.element_size())

    # C1: f32 GEMM 512^3, uniform[-1,1)
    gemm_cfg("c1_gemm_f32_512", "f32", 512, 512, 512,
             make=lambda s: torch.rand(s, generator=g, device=dev) * 2 - 1)
    # C2: int8 4096^3 -> i32 -> *0.01 -> f16
    gemm_cfg("c2_gemm_i8_4096_f16out", "i8", 4096, 4096, 4096, out_dtype="f16", scale=0.01,
             make=lambda s: torch.randint(-128, 128, s, generator=g, device=dev, dtype=torch.int8))

    # C4: fp8 8192^3, normal(0,1) quantised with amax/448, f32 out * sa*sb
    def fp8(s):
        x = torch.randn(s, generator=g, device=dev)
        sc = x.abs().max() / 448.0
        fp8.scales.append(float(sc))
        return (x / sc).to(torch.float8_e4m3fn)
    fp8.scales = []
    gemm_cfg("c4_gemm_fp8_8192", "fp8", 8192, 8192, 8192, make=fp8)
    cfgs["c4_gemm_fp8_8192"]["kernel"].set_scale(fp8.scales[0] * fp8.scales[1])

    # C3: f16 NHWC conv N=256 28x28 C=128 K=128 3x3 s1 p1
    n, c, k, hw = 256, 128, 128, 28
    inp = (torch.randn(n * hw * hw * c, generator=g, device=dev) * 0.1).half()
    fil = (torch.randn(k * 9 * c, generator=g, device=dev) * 0.1).half()
    # (a program: the table's plan for this layer is a small filter conversion in front of the window-resident
    # kernel, and both are launched and timed)
    kern = rock.RockProgram(
        "--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 --fil_layout gkyxc "
        "--in_layout nhwgc --out_layout nhwgk --batchsize 256 --groupsize 1 --in_channels 128 "
        "--out_channels 128 --in_h 28 --in_w 28 --out_h 28 --out_w 28 --fil_h 3 --fil_w 3 --dilation_h 1 "
        "--dilation_w 1 --conv_stride_h 1 --conv_stride_w 1 --padding_h 1 --padding_w 1")
    out = torch.empty(n * hw * hw * k, dtype=torch.float16, device=dev)
    cfgs["c3_conv_f16_resnet3x3"] = dict(
        kernel=kern, args=(fil, inp, out, None), ops=2.0 * n * c * k * hw * hw * 9, dtype="f16",
        peak=PEAK["f16"], shape=dict(op="conv"), min_bytes=2 * (inp.numel() + fil.numel() + out.numel()))

    # C5: attention f16 [4,32,2048,128]
    G, S, D = 128, 2048, 128
    q, kk, v = (torch.randn((G, S, D), generator=g, device=dev).half() for _ in range(3))
    kern = rock.RockKernel("-operation attention -arch gfx950 -t f16 -g 128 -seq_len_q 2048 -seq_len_k 2048 "
                           "-head_dim_qk 128 -head_dim_v 128 -transK true -scale %.9g" % (128 ** -0.5))
    o = torch.empty((G, S, D), dtype=torch.float16, device=dev)
    cfgs["c5_attention_f16_2048x128"] = dict(
        kernel=kern, args=(q, kk, v, None, o), ops=4.0 * G * S * S * D, dtype="f16", peak=PEAK["f16"],
        shape=dict(op="attention"), min_bytes=2 * 4 * G * S * D)
    return cfgs


def cpu_baseline(name, budget_s, threads):
    """Times the CPU oracle (the restated rocmlir-gen -pv validator) on a
    bounded sample of the named workload; returns (ops/s, description)."""
    import numpy as np
    from oracle import rock_oracle as orc
    rng = np.random.default_rng(0)

    def timed(run, unit_ops, total_units, probe_units, what):
        t0 = time.perf_counter()
        run(probe_units)
        dt = max(time.perf_counter() - t0, 1e-4)
        units = int(min(total_units, max(probe_units, probe_units * budget_s / dt)))
        t0 = time.perf_counter()
        run(units)
        dt = time.perf_counter() - t0
        return unit_ops * units / dt, "%d of %d %s, %.1f s" % (units, total_units, what, dt)

    if name.startswith("c2"):
        M = N = K = 4096
        A = rng.integers(-128, 128, (M, K), dtype=np.int8)
        B = rng.integers(-128, 128, (N, K), dtype=np.int8)
        return timed(lambda r: orc.gemm(A, B, 1, M, N, K, transB=True, rows=(0, r), threads=threads),
                     2.0 * N * K, M, 4 * threads, "output rows of the 4096^3 int8 GEMM (i64 accumulate)")
    if name.startswith("c1"):
        A = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
        B = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
        return timed(lambda r: orc.gemm(A, B, 1, 512, 512, 512, transB=True, rows=(0, r), threads=threads),
                     2.0 * 512 * 512, 512, 512, "output rows of the 512^3 f32 GEMM")
    if name.startswith("c4"):
        M = N = K = 8192
        A = orc.round_through(rng.standard_normal((M // 8, K), dtype=np.float32) * 100, orc.FP8)
        B = orc.round_through(rng.standard_normal((N, K), dtype=np.float32) * 100, orc.FP8)
        A = np.concatenate([A] * 8)
        return timed(lambda r: orc.gemm(A, B, 1, M, N, K, transB=True, rows=(0, r), threads=threads),
                     2.0 * N * K, M, 2 * threads, "output rows of the 8192^3 fp8 GEMM (f32 accumulate)")
    if name.startswith("c3"):
        n, c, k, hw = 256, 128, 128, 28
        inp = rng.standard_normal(8 * hw * hw * c).astype(np.float32)   # 8 images stand for 256
        fil = rng.standard_normal(k * 9 * c).astype(np.float32)
        total = 8 * hw * hw * k
        return timed(lambda u: orc.conv_fwd(fil, inp, "gkyxc", "nhwgc", "nhwgk", 8, 1, c, k, hw, hw, 3, 3,
                                            pad=(1, 1), out_range=(0, u), threads=threads),
                     2.0 * c * 9, total, 4096 * threads, "outputs of the f16 3x3 conv (8 of 256 images)")
    if name.startswith("c5"):
        G, S, D = 128, 2048, 128
        q = rng.standard_normal((threads, S, D)).astype(np.float32)
        kk = rng.standard_normal((threads, S, D)).astype(np.float32)
        v = rng.standard_normal((threads, S, D)).astype(np.float32)
        return timed(lambda r: orc.attention(q, kk, v, threads, S, S, D, D, scale=D ** -0.5, transK=True,
                                             q_rows=(0, r), threads=threads),
                     4.0 * S * D * threads, S, 8, "query rows x %d heads of the f16 attention" % threads)
    raise KeyError(name)


def vendor_gemms(torch, rock, dev, n):
    """Same shapes, same tensors: the vendor library's GEMM and this library's, n launches each."""
    torch.manual_seed(1)

    def ours(t, od, m, k, a, b):
        kern = rock.RockKernel("-operation gemm -arch gfx950 -t %s -g 1 -m %d -n %d -k %d -transB true "
                               "-out_datatype %s" % (t, m, m, k, od))
        out = torch.empty((m, m), dtype=rock.api._torch_dtype(od), device=dev)
        for _ in range(n):
            kern.launch(a, b, out, None)
        torch.cuda.synchronize()

    for m in (8192, 4096):
        a = torch.randn(m, m, device=dev, dtype=torch.float16)
        b = torch.randn(m, m, device=dev, dtype=torch.float16)
        for _ in range(n):
            torch.matmul(a, b.t())
        torch.cuda.synchronize()
        ours("f16", "f16", m, m, a, b)
    a = torch.randn(8192, 8192, device=dev).to(torch.float8_e4m3fn)
    b = torch.randn(8192, 8192, device=dev).to(torch.float8_e4m3fn)
    one = torch.ones((), device=dev)
    for od, name in ((torch.bfloat16, "bf16"), (torch.float32, "f32")):
        for _ in range(n):
            torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=od)
        torch.cuda.synchronize()
        ours("fp8", name, 8192, 8192, a, b)
    a = torch.randint(-128, 128, (4096, 4096), dtype=torch.int8, device=dev)
    b = torch.randint(-128, 128, (4096, 4096), dtype=torch.int8, device=dev)
    for _ in range(n):
        torch._int_mm(a, b.t())
    torch.cuda.synchronize()
    ours("i8", "i32", 4096, 4096, a, b)
    print(json.dumps({"vendor_gemms": n}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--prewarm", type=int, default=500,
                    help="untimed launches before the warm-up steps (reported as \"prewarm\" in the JSON "
                         "line): the shader clock needs some tens of "
                         "milliseconds of load to leave its idle state (measured on the headline kernel: "
                         "1.87 POP/s with none, 1.89 after 100, 2.13 after 400, flat from there to 10000)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-headline", action="store_true", help="skip the other four configs")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--traffic-bytes", type=float, default=134.7e6,
                    help="HBM bytes per launch of the headline kernel: FETCH_SIZE + WRITE_SIZE of "
                         "rocprofv3 --pmc runs of this command, each scaled by the same counter's reading "
                         "for a plain copy (--calibrate-copy); the default is the committed measurement "
                         "(profiles/gemm_i8_256x256_c2_hbm_traffic.txt)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="only run a plain device-to-device copy of MIB MiB five times (the known-size "
                         "kernel that FETCH_SIZE / WRITE_SIZE readings are scaled by) and exit")
    ap.add_argument("--vendor-gemms", type=int, default=0, metavar="N",
                    help="only launch, N times each, the GEMMs of the vendor libraries shipped with torch "
                         "(torch.matmul f16, torch._scaled_mm fp8, torch._int_mm int8) and this library's "
                         "kernels on the same shapes and data, and exit: the command that rocprofv3 traces "
                         "for the side-by-side table of kernel geometry and counters under profiles/")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every box has one); --gpus %d is not "
                 "supported -- the path shards without exchange (GEMM by rows, conv by batch, attention "
                 "by batch x heads) but no multi-GPU "
                 "figure is produced here" % args.gpus)

    import torch
    import rocmlir_amd as rock
    rock.load_library()  # fails loudly when the HIP library has not been built
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        src = torch.ones(args.calibrate_copy << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": src.numel(), "launches": 5}))
        return
    if args.vendor_gemms:
        vendor_gemms(torch, rock, dev, args.vendor_gemms)
        return
    cfgs = make_configs(torch, rock, dev)
    head_name = "c2_gemm_i8_4096_f16out"
    head = cfgs[head_name]
    K, W = args.steps, args.warmup

    # ---- the timed region: W warm-up steps, then exactly K steps
    stream = torch.cuda.current_stream()
    for _ in range(args.prewarm):  # bring the clocks up before anything is measured (about 35 ms)
        head["kernel"].launch(*head["args"], stream=stream)
    torch.cuda.synchronize()
    for _ in range(W):
        head["kernel"].launch(*head["args"], stream=stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        head["kernel"].launch(*head["args"], stream=stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / K
    value = head["ops"] / (wall / K) / 1e12

    # ---- kernel-only duration: HIP events on the launch stream
    kern_ms = head["kernel"].benchmark(*head["args"], warmup=10, iters=max(K, 50), stream=stream)
    achieved = head["ops"] / (kern_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": head["peak"], "unit": "TFLOP/s",
                "frac": round(achieved / head["peak"], 4), "traffic": args.traffic_bytes,
                "kernel": head["kernel"].kernel_name, "kernel_ms": round(kern_ms, 5),
                "hbm_gbps_algorithmic": round(head["min_bytes"] / (kern_ms * 1e-3) / 1e9, 1)}

    # what the matrix cores alone sustain on this box (register-only MFMA chains):
    # with constant operands, and with random bit patterns (lower clocks, power)
    rates = {}

    def issue_rate(dt):
        if dt not in rates:
            rates[dt] = {"constant_operands": round(rock.mfma_rate(dt, False, stream), 1),
                         "random_operands": round(rock.mfma_rate(dt, True, stream), 1)}
        return rates[dt]

    roofline["mfma_issue_rate_measured"] = issue_rate(head["dtype"])
    roofline["frac_of_measured_random_operand_rate"] = round(
        achieved / roofline["mfma_issue_rate_measured"]["random_operands"], 4)

    # The other four configurations, each first run for about 30 ms so that it
    # is timed at the clocks a loaded GPU settles at.  The headline's entry
    # repeats the event-timed figure above, so that its LAST max(K, 50)
    # dispatches in a kernel trace of this command are exactly the timed ones.
    per_config = {}
    if not args.only_headline:
        for name, c in cfgs.items():
            iters = 200 if name.startswith("c1") else max(10, min(K, 30))
            if name == head_name:
                ms = kern_ms
            else:
                t_load = time.perf_counter()
                while time.perf_counter() - t_load < 0.03:
                    for _ in range(20):
                        c["kernel"].launch(*c["args"], stream=stream)
                    torch.cuda.synchronize()
                ms = c["kernel"].benchmark(*c["args"], warmup=3, iters=iters, stream=stream)
            tf = c["ops"] / (ms * 1e-3) / 1e12
            per_config[name] = {"kernel": c["kernel"].kernel_name,
                                **({"kernels": [k.kernel_name for k in c["kernel"].kernels]}
                                   if hasattr(c["kernel"], "kernels") else {}),
                                "kernel_ms": round(ms, 5),
                                "tflops": round(tf, 2), "peak": c["peak"], "frac_of_mfma_peak": round(tf / c["peak"], 4),
                                "hbm_gbps_algorithmic": round(c["min_bytes"] / (ms * 1e-3) / 1e9, 1),
                                "mfma_issue_rate_measured": issue_rate(c["dtype"])}

    cores = os.cpu_count() or 1
    threads = min(16, cores)  # the box's CPU share for one GPU
    cpu = None
    if not args.no_cpu:
        from oracle import rock_oracle as orc
        threads = min(threads, orc.max_threads())
        rate, sample = cpu_baseline(head_name, args.cpu_seconds, threads)
        cpu = {"value": round(rate / 1e12, 6), "unit": "TOP/s", "cores": threads, "kind": "port",
               "sample": sample, "gflops": round(rate / 1e9, 2)}
        if not args.only_headline:
            for name in per_config:
                if name == head_name:
                    per_config[name]["cpu_validator_gflops"] = cpu["gflops"]
                    continue
                r, s = cpu_baseline(name, 3.0, threads)
                per_config[name]["cpu_validator_gflops"] = round(r / 1e9, 2)
                per_config[name]["cpu_sample"] = s
                per_config[name]["cpu_cores"] = threads

    line = {
        "metric": "TFLOPS/TOPS per config on 1 MI355X; % of MFMA peak; CPU -pv ref GFLOPS",
        "value": round(value, 2), "unit": "TOP/s", "n_gpus": 1, "steps": K, "warmup": W,
        "prewarm": args.prewarm, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "i8", "data": "synthetic",
        "config": {"workload": "configs[1]: int8 quantised GEMM M=N=K=4096, A[M,K] x B[N,K]^T, i32 accumulate, "
                               "f32 scale 0.01, f16 output", "kernel": head["kernel"].kernel_name,
                   "perf_config": head["kernel"].perf_config},
        "roofline": roofline, "cpu_baseline": cpu, "per_config": per_config,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
