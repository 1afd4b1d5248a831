"""GPU parity: the element-wise tail fused behind GEMM and convolution
(activation functions, clip, a residual tensor) through the C ABI.

Pinned by the literal vectors of the reference's fusion tests
(tests/golden/fusion_kats.json), then exactly with integer-valued data where
every step is exact (add, mul, relu, clip), and to the reference verifier's
RMS gate for the transcendental activations against numpy / scipy."""
import json
import math
import os

import numpy as np
import pytest
import scipy.special
import torch

from tests.gpu_util import CODE, TORCH, check_float, quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _kats():
    with open(os.path.join(HERE, "golden", "fusion_kats.json")) as f:
        return json.load(f)


def _fill(oracle, n, rand):
    """The reference's data fill for `-rand none` / `-rand N` (integers)."""
    return np.ones(n, np.float32) if rand == "none" else oracle.fill_rand(n, -5, 5, False)


@pytest.mark.parametrize("case", _kats(), ids=lambda c: c["source"])
def test_fusion_reference_golden_vectors(rock, oracle, gpu, case):
    t, tail = case["t"], dict(case["tail"])
    if case["rand"] != "none":
        oracle.seed(int(case["rand"]))
    kw = {}
    if case["operation"] == "gemm":
        g, m, n, k = case["g"], case["m"], case["n"], case["k"]
        a = _fill(oracle, g * m * k, case["rand"]).reshape(g, m, k)   # arguments are filled in order
        b = _fill(oracle, g * k * n, case["rand"]).reshape(g, k, n)
        if tail.pop("bias", False):
            kw["bias"] = torch.from_numpy(_fill(oracle, n, case["rand"])).to(gpu)
        if "residual" in tail:
            kw["residual_op"] = tail.pop("residual")
            kw["residual"] = to_gpu(quantise(_fill(oracle, g * m * n, case["rand"]), t)[0], t, gpu).reshape(g, m, n)
        out = rock.gemm(to_gpu(quantise(a, t)[0], t, gpu), to_gpu(quantise(b, t)[0], t, gpu), **kw, **tail)
        got = to_f32(out, t)
        assert got.size == len(case["expected"])
    else:
        n, c, k, hi, wi = case["n"], case["c"], case["k"], case["hi"], case["wi"]
        inp = _fill(oracle, n * c * hi * wi, case["rand"])
        fil = _fill(oracle, k * c * case["y"] * case["x"], case["rand"])
        if tail.pop("bias", False):
            kw["bias"] = torch.from_numpy(_fill(oracle, k, case["rand"])).to(gpu)
        out = rock.conv2d(to_gpu(quantise(fil, t)[0], t, gpu), to_gpu(quantise(inp, t)[0], t, gpu),
                          fil_layout="gkcyx", in_layout="ngchw", out_layout="ngkhw", batchsize=n, in_channels=c,
                          out_channels=k, in_h=hi, in_w=wi, fil_h=case["y"], fil_w=case["x"], **kw, **tail)
        got = to_f32(out, t)
        assert got.size == n * k * hi * wi
        got = got[:len(case["expected"])] if np.all(got == got[0]) else got
    # FileCheck compares the printed text: six significant digits
    assert [float("%.6g" % v) for v in got] == case["expected"]


def _gemm_inputs(rng, t, G, M, N, K, integer):
    if t == "i8":
        A = rng.integers(-128, 128, (G, M, K)).astype(np.float32)
        B = rng.integers(-128, 128, (G, N, K)).astype(np.float32)
    elif integer:
        A = rng.integers(-2, 3, (G, M, K)).astype(np.float32)
        B = rng.integers(-2, 3, (G, N, K)).astype(np.float32)
    else:
        A = rng.uniform(-1, 1, (G, M, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (G, N, K)).astype(np.float32)
    return A, B


# (kernel family, G M N K, transB, perf_config)
KERNELS = [
    ("fast_256x256", (1, 300, 520, 128), True, "v2:256,256,8,128,16,8,1,1,1"),
    ("fast_128x128", (2, 130, 136, 64), True, "v2:128,128,8,64,16,8,1,1,1"),
    ("fast_64x64", (1, 70, 72, 96), True, "v2:64,64,8,32,16,8,1,1,1"),
    ("generic", (2, 70, 45, 97), True, None),
    ("split_k", (1, 32, 48, 1024), True, None),
    ("k_major", (1, 144, 208, 208), False, None),
]


@pytest.mark.parametrize("kernel", KERNELS, ids=lambda k: k[0])
@pytest.mark.parametrize("t,od", [("f32", "f32"), ("f16", "f16"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "f16"),
                                  ("fp8", "f32")])
@pytest.mark.parametrize("op", ["add", "mul"])
def test_gemm_residual_and_relu_exact(rock, oracle, gpu, kernel, t, od, op):
    """relu(scale * acc + bias op residual): integer data keeps every step exact."""
    name, (G, M, N, K), tB, pc = kernel
    rng = np.random.default_rng(61)
    A, B = _gemm_inputs(rng, t, G, M, N, K, True)
    rawA, Aq = quantise(A, t)
    rawB, Bq = quantise(B if tB else np.ascontiguousarray(B.transpose(0, 2, 1)), t)
    res = rng.integers(-3, 4, (G, M, N)).astype(np.float32)
    raw_res, res_q = quantise(res, od) if od != "i32" else (res.astype(np.int32), res)
    info = {}
    kw = dict(scale=0.5, relu=True) if od != "i32" else {}
    out = rock.gemm(to_gpu(rawA, t, gpu), to_gpu(rawB, t, gpu), transB=tB, out_dtype=od,
                    residual=to_gpu(raw_res, od, gpu).reshape(G, M, N), residual_op=op, perf_config=pc,
                    info=info, layout_conversion=name != "generic", **kw)
    if name not in ("generic", "split_k", "k_major"):
        assert name.split("_")[1] in info["kernel_name"]
    else:
        assert {"generic": "generic", "split_k": "splitk", "k_major": "_fast_nn"}[name] in info["kernel_name"]
    acc = oracle.gemm(rawA, rawB, G, M, N, K, False, tB, False) if t == "i8" else \
        oracle.gemm(Aq, Bq, G, M, N, K, False, tB, False)
    acc = np.asarray(acc, np.float64).reshape(G, M, N)
    if od == "i32":
        want = acc + res if op == "add" else acc * res
        assert np.array_equal(out.cpu().numpy().astype(np.float64), want)
        return
    v = (acc * 0.5).astype(np.float32)
    v = v + res_q.reshape(G, M, N) if op == "add" else v * res_q.reshape(G, M, N)
    want = np.maximum(v, 0.0).astype(np.float32)
    assert np.array_equal(to_f32(out, od), oracle.round_through(want.ravel(), CODE[od]))


@pytest.mark.parametrize("kernel", KERNELS, ids=lambda k: k[0])
@pytest.mark.parametrize("t,od", [("f32", "f32"), ("f16", "f16"), ("bf16", "f32"), ("i8", "i32"), ("fp8", "f32")])
@pytest.mark.parametrize("transC", [False, True], ids=["c", "ct"])
def test_gemm_accumulating_store_exact(rock, oracle, gpu, kernel, t, od, transC):
    """-store-method atomic_add (rocmlir-gen.cpp:295-331): C += A B, twice in a row into the same tensor, on
    every kernel family; integer data keeps every sum exact."""
    name, (G, M, N, K), tB, pc = kernel
    rng = np.random.default_rng(65)
    A, B = _gemm_inputs(rng, t, G, M, N, K, True)
    rawA, Aq = quantise(A, t)
    rawB, Bq = quantise(B if tB else np.ascontiguousarray(B.transpose(0, 2, 1)), t)
    c0 = rng.integers(-5, 6, (G, N, M) if transC else (G, M, N)).astype(np.float32)
    raw_c, c0q = quantise(c0, od) if od != "i32" else (c0.astype(np.int32), c0)
    out = to_gpu(raw_c, od, gpu).reshape(c0.shape).clone()
    info = {}
    for _ in range(2):
        got = rock.gemm(to_gpu(rawA, t, gpu), to_gpu(rawB, t, gpu), transB=tB, transC=transC, out_dtype=od, out=out,
                        accumulate=True, perf_config=pc, info=info, layout_conversion=name != "generic")
        assert got.data_ptr() == out.data_ptr()
    torch.cuda.synchronize()
    assert info["kernel_name"].endswith("_e") or "generic" in info["kernel_name"]
    acc = oracle.gemm(rawA, rawB, G, M, N, K, False, tB, False) if t == "i8" else \
        oracle.gemm(Aq, Bq, G, M, N, K, False, tB, False)
    acc = np.asarray(acc, np.float64).reshape(G, M, N)
    if transC:
        acc = acc.transpose(0, 2, 1)
    if od == "i32":
        assert np.array_equal(out.cpu().numpy().astype(np.float64), c0.astype(np.float64) + 2.0 * acc)
        return
    want = c0q.reshape(c0.shape).astype(np.float32)
    for _ in range(2):   # each pass: f32 sum of the accumulator and the stored value, rounded to the output type
        want = oracle.round_through((acc.astype(np.float32) + want).ravel(), CODE[od]).reshape(c0.shape)
    assert np.array_equal(to_f32(out, od), want.ravel())


def test_gemm_clip_exact(rock, oracle, gpu):
    rng = np.random.default_rng(63)
    A, B = _gemm_inputs(rng, "f16", 1, 128, 128, 64, True)
    rawA, Aq = quantise(A, "f16")
    rawB, Bq = quantise(B, "f16")
    out = rock.gemm(to_gpu(rawA, "f16", gpu), to_gpu(rawB, "f16", gpu), transB=True, clip=(-2.5, 6.0))
    acc = oracle.gemm(Aq, Bq, 1, 128, 128, 64, False, True, False)
    assert np.array_equal(to_f32(out, "f16"), np.clip(acc, -2.5, 6.0).astype(np.float32))


ACTIVATIONS = {
    "sigmoid": lambda v: 1.0 / (1.0 + np.exp(-v)),
    "tanh": np.tanh,
    "erf": scipy.special.erf,
    "gelu": lambda v: 0.5 * v * (1.0 + scipy.special.erf(v / math.sqrt(2.0))),
    "exp": np.exp,
    "relu": lambda v: np.maximum(v, 0.0),
}


@pytest.mark.parametrize("act", sorted(ACTIVATIONS))
@pytest.mark.parametrize("t,od", [("f32", "f32"), ("f16", "f16"), ("bf16", "bf16"), ("i8", "f16")])
def test_gemm_activation_real_values(rock, oracle, gpu, act, t, od):
    """act(scale * acc + bias) on real-valued data against numpy / scipy in
    float64, the reference's RMS gate for the output type."""
    G, M, N, K = 2, 200, 264, 128
    rng = np.random.default_rng(65)
    A, B = _gemm_inputs(rng, t, G, M, N, K, False)
    rawA, Aq = quantise(A, t)
    rawB, Bq = quantise(B, t)
    bias = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    scale = 2e-5 if t == "i8" else 0.25
    out = rock.gemm(to_gpu(rawA, t, gpu), to_gpu(rawB, t, gpu), transB=True, out_dtype=od, scale=scale,
                    bias=torch.from_numpy(bias).to(gpu), activation=act)
    acc = oracle.gemm(rawA, rawB, G, M, N, K, False, True, False) if t == "i8" else \
        oracle.gemm(Aq, Bq, G, M, N, K, False, True, False)
    v = np.asarray(acc, np.float64).reshape(G, M, N) * scale + bias[None, None, :]
    check_float(to_f32(out, od), ACTIVATIONS[act](v).astype(np.float32).ravel(), od)


NHWC = ("gkyxc", "nhwgc", "nhwgk")
NCHW = ("gkcyx", "ngchw", "ngkhw")


@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=["nhwc", "nchw"])
@pytest.mark.parametrize("t,od", [("f16", "f16"), ("f32", "f32"), ("i8", "i32"), ("i8", "f16")])
@pytest.mark.parametrize("shape", [(4, 64, 64, 14, 14, 3, 1), (2, 32, 48, 9, 9, 1, 0), (2, 3, 16, 12, 12, 3, 1),
                                   (3, 128, 96, 14, 16, 3, 1, "v2:224,128,8,224,32,8,1,1,1")],
                         ids=["3x3", "1x1", "padded-channels", "window-resident"])
def test_conv_bias_residual_relu_exact(rock, oracle, gpu, layouts, t, od, shape):
    """The ResNet block tail relu(conv + bias + shortcut), every layout route
    (vector kernel, conversion plan, pointwise-as-GEMM falls back because of the bias,
    the window-resident kernel behind its filter conversion)."""
    n, c, k, hi, wi, y, pad = shape[:7]
    perf = shape[7] if len(shape) > 7 else None
    fl, il, ol = layouts
    rng = np.random.default_rng(67)
    lim = 128 if t == "i8" else 3
    fil = rng.integers(-lim, lim, (1, k, c, y, y)).astype(np.float32)
    inp = rng.integers(-lim, lim, (n, 1, c, hi, wi)).astype(np.float32)

    def to_layout(x, canonical, layout):
        return np.ascontiguousarray(x.transpose([canonical.index(ch) for ch in layout])).ravel()

    raw_f, fq = quantise(to_layout(fil, "gkcyx", fl), t)
    raw_i, iq = quantise(to_layout(inp, "ngchw", il), t)
    ho, wo = hi + 2 * pad - y + 1, wi + 2 * pad - y + 1
    res = rng.integers(-4, 5, n * k * ho * wo).astype(np.float32)       # laid out like the output
    raw_res, res_q = quantise(res, od) if od != "i32" else (res.astype(np.int32), res)
    bias = rng.integers(-3, 4, k).astype(np.float32)
    bias_t = torch.from_numpy(bias.astype(np.int32) if od == "i32" else bias).to(gpu)
    kw = dict(scale=0.25, relu=True) if od != "i32" else {}
    info = {}
    out = rock.conv2d(to_gpu(raw_f, t, gpu), to_gpu(raw_i, t, gpu), fil_layout=fl, in_layout=il, out_layout=ol,
                      batchsize=n, in_channels=c, out_channels=k, in_h=hi, in_w=wi, fil_h=y, fil_w=y,
                      padding=(pad, pad), out_dtype=od, bias=bias_t, residual=to_gpu(raw_res, od, gpu), info=info,
                      perf_config=perf, **kw)
    if perf and layouts is NHWC:
        assert info["kernels"][-1].startswith("rock_conv_%s_direct224" % t) and len(info["kernels"]) == 2
    acc, _, _ = oracle.conv_fwd(raw_f if t == "i8" else fq, raw_i if t == "i8" else iq, fl, il, ol, n, 1, c, k, hi, wi,
                                y, y, (1, 1), (pad, pad), (1, 1))
    acc = np.asarray(acc, np.float64)
    # bias per output channel, in the output's layout
    kpos = ol.index("k")
    shape5 = [dict(n=n, g=1, k=k, h=ho, w=wo)[ch] for ch in ol]
    bshape = [1] * 5
    bshape[kpos] = k
    b_full = np.broadcast_to(bias.reshape(bshape), shape5).ravel()
    if od == "i32":
        assert np.array_equal(out.cpu().numpy().astype(np.float64), acc + b_full + res)
        return
    v = (acc * 0.25).astype(np.float32) + b_full
    want = np.maximum(v + res_q, 0.0).astype(np.float32)
    assert np.array_equal(to_f32(out, od), oracle.round_through(want, CODE[od]))
    assert info["kernel_name"].startswith("rock_conv_")


def test_conv_pointwise_gemm_route_with_residual(rock, oracle, gpu):
    """NCHW 1x1 without bias keeps the GEMM route; the residual is laid out like the output."""
    n, c, k, hi, wi = 3, 64, 48, 8, 8
    rng = np.random.default_rng(69)
    fil = rng.integers(-2, 3, k * c).astype(np.float32)
    inp = rng.integers(-2, 3, n * c * hi * wi).astype(np.float32)
    res = rng.integers(-4, 5, n * k * hi * wi).astype(np.float32)
    raw_f, fq = quantise(fil, "f16")
    raw_i, iq = quantise(inp, "f16")
    raw_r, rq = quantise(res, "f16")
    info = {}
    out = rock.conv2d(to_gpu(raw_f, "f16", gpu), to_gpu(raw_i, "f16", gpu), fil_layout="gkcyx", in_layout="ngchw",
                      out_layout="ngkhw", batchsize=n, in_channels=c, out_channels=k, in_h=hi, in_w=wi, fil_h=1,
                      fil_w=1, residual=to_gpu(raw_r, "f16", gpu), activation="relu", info=info)
    assert info["kernel_name"].startswith("rock_gemm_") and info["kernels"] == [info["kernel_name"]]
    acc, _, _ = oracle.conv_fwd(fq, iq, "gkcyx", "ngchw", "ngkhw", n, 1, c, k, hi, wi, 1, 1, (1, 1), (0, 0), (1, 1))
    want = np.maximum(acc + rq, 0.0).astype(np.float32)
    assert np.array_equal(to_f32(out, "f16"), oracle.round_through(want, CODE["f16"]))
