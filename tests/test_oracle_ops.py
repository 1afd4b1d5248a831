"""Pins the oracle's GEMM / convolution / attention / epilogue / verifier
restatements: the reference's own golden vectors, closed forms, library
routines (numpy float64 matmul, torch conv2d, torch softmax) and invariants."""
import ctypes
import itertools
import json
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


# ----------------------------------------------------------------- GEMM
def _store(mat, trans):
    """logical [G,R,C] -> storage order of the reference ([G,C,R] if trans)."""
    return np.ascontiguousarray(mat.transpose(0, 2, 1) if trans else mat)


@pytest.mark.parametrize("tA,tB,tC", list(itertools.product([0, 1], repeat=3)))
def test_gemm_f32_all_transposes_vs_float64(oracle, tA, tB, tC):
    rng = np.random.default_rng(10 + 4 * tA + 2 * tB + tC)
    G, M, N, K = 3, 7, 5, 11
    A = rng.uniform(-1, 1, (G, M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (G, K, N)).astype(np.float32)
    got = oracle.gemm(_store(A, tA), _store(B, tB), G, M, N, K, tA, tB, tC)
    want = np.matmul(A.astype(np.float64), B.astype(np.float64))
    want = _store(want, tC).ravel()
    assert np.allclose(got, want, rtol=0, atol=2e-6)
    # a transposed operand or a wrong index breaks this by O(1)


def test_gemm_reduction_order_is_k_ascending_mul_then_add(oracle):
    # values chosen so that any other association or an fma changes the result
    a = np.array([[1e8, 1.0, -1e8, 1.0]], np.float32)
    b = np.ones((4, 1), np.float32)
    got = oracle.gemm(a, b, 1, 1, 1, 4)
    acc = np.float32(0)
    for k in range(4):
        acc = np.float32(np.float32(a[0, k] * b[k, 0]) + acc)
    assert got[0] == acc == 1.0
    x = np.float32(1 + 2 ** -12)
    got = oracle.gemm(np.array([[x, 1.0]], np.float32), np.array([[x], [-1.0]], np.float32), 1, 1, 1, 2)
    assert got[0] == np.float32(np.float32(x * x) - np.float32(1.0))  # no fma


def test_gemm_fixed_pattern_closed_form(oracle):
    # the reference's "-rand fixed" data: {0.5,-1,0.75} cycled by flat index
    M = N = K = 6
    A = oracle.fill_fixed(M * K).reshape(M, K)
    B = oracle.fill_fixed(K * N).reshape(K, N)
    assert A.ravel()[:4].tolist() == [0.5, -1.0, 0.75, 0.5]
    got = oracle.gemm(A, B, 1, M, N, K).reshape(M, N)
    # K=6 is a multiple of 3, so every row of A is the pattern twice and every
    # column of B is constant: column j of B holds pat[j % 3]
    pat = np.array([0.5, -1.0, 0.75])
    for j in range(N):
        assert np.allclose(got[:, j], 2 * pat.sum() * pat[j % 3])


def test_gemm_i8_exact_and_widened(oracle):
    rng = np.random.default_rng(11)
    G, M, N, K = 2, 9, 8, 300
    A = rng.integers(-128, 128, (G, M, K), dtype=np.int8)
    B = rng.integers(-128, 128, (G, N, K), dtype=np.int8)  # stored [G,N,K]: transB
    got = oracle.gemm(A, B, G, M, N, K, transB=True).reshape(G, M, N)
    want = np.einsum("gmk,gnk->gmn", A.astype(np.int64), B.astype(np.int64))
    assert np.array_equal(got, want)
    # -128 * -128 = 16384 does not fit in i8: proves operands are widened first
    one = oracle.gemm(np.array([[-128]], np.int8), np.array([[-128]], np.int8), 1, 1, 1, 1)
    assert one[0] == 16384


def test_gemm_all_ones_quant_case(oracle):
    # mixr-gemm-reshape-case1-quant.e2e.mlir:6 -- all-ones 5x4 . 4x3 int8 -> fifteen 4s
    got = oracle.gemm(np.ones((5, 4), np.int8), np.ones((4, 3), np.int8), 1, 5, 3, 4)
    assert got.tolist() == [4] * 15


def test_gemm_row_sample(oracle):
    rng = np.random.default_rng(12)
    A = rng.standard_normal((16, 8)).astype(np.float32)
    B = rng.standard_normal((8, 4)).astype(np.float32)
    full = oracle.gemm(A, B, 1, 16, 4, 8).reshape(16, 4)
    part = oracle.gemm(A, B, 1, 16, 4, 8, rows=(5, 9), threads=2).reshape(16, 4)
    assert np.array_equal(part[5:9], full[5:9]) and not part[:5].any() and not part[9:].any()


# ----------------------------------------------------------------- convolution
def _golden_cases():
    with open(os.path.join(HERE, "golden", "conv_fwd_kats.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c["source"])
@pytest.mark.parametrize("dtype", ["f32", "i8"])
def test_conv_reference_golden_vectors(oracle, case, dtype):
    """mlir/test/rocmlir-driver/cpu_conv2d/*_fwd.mlir: all-ones data (-rand
    none), literal expected output."""
    f = case["flags"]
    n, c, k = int(f["batchsize"]), int(f["in_channels"]), int(f["out_channels"])
    hi, wi, y, x = int(f["in_h"]), int(f["in_w"]), int(f["fil_h"]), int(f["fil_w"])
    lay = {"kyxc": "gkyxc", "kcyx": "gkcyx", "nhwc": "nhwgc", "nchw": "ngchw",
           "nhwk": "nhwgk", "nkhw": "ngkhw"}
    np_t = np.int8 if dtype == "i8" else np.float32
    fil = np.ones(k * c * y * x, np_t)
    inp = np.ones(n * c * hi * wi, np_t)
    out, ho, wo = oracle.conv_fwd(
        fil, inp, lay[f["fil_layout"]], lay[f["in_layout"]], lay[f["out_layout"]],
        n, 1, c, k, hi, wi, y, x,
        stride=(int(f["conv_stride_h"]), int(f["conv_stride_w"])),
        pad=(int(f["padding_h"]), int(f["padding_w"])),
        dil=(int(f["dilation_h"]), int(f["dilation_w"])))
    assert out.size == len(case["expected"])
    assert np.array_equal(out.astype(np.float64), np.array(case["expected"]))


def _to_layout(t, canonical, layout):
    """tensor with axes in `canonical` letter order -> flat array in `layout` order"""
    perm = [canonical.index(ch) for ch in layout]
    return np.ascontiguousarray(t.transpose(perm)).ravel()


CONV_CASES = [
    # n g c k hi wi y x stride pad dil
    (2, 1, 3, 4, 9, 7, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 2, 4, 6, 8, 8, 3, 2, (2, 1), (0, 1), (1, 2)),
    (3, 4, 2, 2, 5, 6, 1, 1, (1, 1), (0, 0), (1, 1)),
    (1, 1, 5, 3, 11, 11, 5, 5, (2, 3), (2, 2), (1, 1)),
    (2, 1, 3, 2, 4, 4, 2, 2, (1, 1), (1, 1), (2, 2)),
    (1, 1, 2, 3, 14, 14, 14, 14, (1, 1), (1, 1), (1, 1)),
]
LAYOUTS = [("gkcyx", "ngchw", "ngkhw"), ("gkyxc", "nhwgc", "nhwgk"), ("gyxck", "hwcgn", "hwkgn"),
           ("gkcyx", "nhwgc", "ngkhw")]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("layouts", LAYOUTS)
def test_conv_vs_torch_conv2d(oracle, case, layouts):
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    rng = np.random.default_rng(1000 + 16 * CONV_CASES.index(case) + LAYOUTS.index(layouts))
    fil = rng.integers(-3, 4, (g, k, c, y, x)).astype(np.float32)   # exact in f32
    inp = rng.integers(-3, 4, (n, g, c, hi, wi)).astype(np.float32)
    fl, il, ol = layouts
    out, ho, wo = oracle.conv_fwd(_to_layout(fil, "gkcyx", fl), _to_layout(inp, "ngchw", il),
                                  fl, il, ol, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    ref = torch.nn.functional.conv2d(
        torch.from_numpy(inp.reshape(n, g * c, hi, wi)).double(),
        torch.from_numpy(fil.reshape(g * k, c, y, x)).double(),
        stride=stride, padding=pad, dilation=dil, groups=g).numpy()
    assert ref.shape == (n, g * k, ho, wo)
    want = _to_layout(ref.reshape(n, g, k, ho, wo), "ngkhw", ol)
    assert np.array_equal(out.astype(np.float64), want)
    # int8 path on the same integers
    out8, _, _ = oracle.conv_fwd(_to_layout(fil, "gkcyx", fl).astype(np.int8),
                                 _to_layout(inp, "ngchw", il).astype(np.int8),
                                 fl, il, ol, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(out8.astype(np.float64), want)


CONV3D_CASES = [
    (2, 2, 3, 4, (5, 6, 7), (3, 2, 3), (1, 2, 2), (1, 0, 2), (1, 2, 1)),
    (1, 1, 4, 5, (6, 6, 6), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    (2, 1, 2, 3, (7, 5, 9), (1, 3, 5), (2, 1, 3), (0, 1, 2), (1, 1, 1)),
]
CONV3D_LAYOUTS = [("gkc012", "ngc012", "ngk012"), ("gk012c", "n012gc", "n012gk"), ("g012ck", "n2g01c", "ngk201")]


ASYM_CASES = [  # (n g c k hi wi y x stride pad_left pad_right dil)
    (2, 1, 3, 4, 6, 7, 2, 2, (1, 1), (0, 0), (1, 1), (1, 1)),
    (1, 2, 2, 3, 9, 8, 3, 3, (2, 2), (0, 1), (1, 2), (1, 1)),
    (2, 1, 4, 2, 7, 7, 3, 2, (1, 1), (2, 0), (0, 1), (1, 2)),
]


@pytest.mark.parametrize("case", ASYM_CASES)
@pytest.mark.parametrize("layouts", LAYOUTS[:2])
def test_conv_asymmetric_padding_vs_torch(oracle, case, layouts):
    """Different padding on the two sides of an axis (--padding_h_l / _r): torch
    conv2d over an explicitly zero-padded image is the independent answer."""
    n, g, c, k, hi, wi, y, x, stride, pad_l, pad_r, dil = case
    rng = np.random.default_rng(4000 + 16 * ASYM_CASES.index(case) + LAYOUTS.index(layouts))
    fil = rng.integers(-3, 4, (g, k, c, y, x)).astype(np.float32)
    inp = rng.integers(-3, 4, (n, g, c, hi, wi)).astype(np.float32)
    fl, il, ol = layouts
    out, ho, wo = oracle.conv_fwd(_to_layout(fil, "gkcyx", fl), _to_layout(inp, "ngchw", il),
                                  fl, il, ol, n, g, c, k, hi, wi, y, x, stride, pad_l, dil, pad_r=pad_r)
    padded = torch.nn.functional.pad(torch.from_numpy(inp.reshape(n, g * c, hi, wi)).double(),
                                     (pad_l[1], pad_r[1], pad_l[0], pad_r[0]))
    ref = torch.nn.functional.conv2d(padded, torch.from_numpy(fil.reshape(g * k, c, y, x)).double(),
                                     stride=stride, dilation=dil, groups=g).numpy()
    assert ref.shape == (n, g * k, ho, wo)
    assert np.array_equal(out, _to_layout(ref.reshape(n, g, k, ho, wo).astype(np.float32), "ngkhw", ol))


@pytest.mark.parametrize("case", CONV3D_CASES)
@pytest.mark.parametrize("layouts", CONV3D_LAYOUTS, ids=lambda l: l[1])
def test_conv3d_vs_torch_conv3d(oracle, case, layouts):
    """torch.nn.functional.conv3d (a library routine) on integer-valued data in
    float64: every sum exact, so a wrong index, stride or padding side shows."""
    n, g, c, k, ins, fs, stride, pad, dil = case
    rng = np.random.default_rng(3000 + 16 * CONV3D_CASES.index(case) + CONV3D_LAYOUTS.index(layouts))
    fil = rng.integers(-3, 4, (g, k, c) + fs).astype(np.float32)
    inp = rng.integers(-3, 4, (n, g, c) + ins).astype(np.float32)
    fl, il, ol = layouts
    out, outs = oracle.conv3d(_to_layout(fil, "gkc012", fl), _to_layout(inp, "ngc012", il), fl, il, ol,
                              n, g, c, k, ins, fs, stride, pad, dil)
    ref = torch.nn.functional.conv3d(torch.from_numpy(inp.reshape((n, g * c) + ins)).double(),
                                     torch.from_numpy(fil.reshape((g * k, c) + fs)).double(),
                                     stride=stride, padding=pad, dilation=dil, groups=g).numpy()
    assert ref.shape == (n, g * k) + outs
    assert np.array_equal(out.astype(np.float64), _to_layout(ref.reshape((n, g, k) + outs), "ngk012", ol))


def test_conv3d_with_depth_one_is_the_2d_oracle(oracle):
    n, g, c, k, hi, wi, y, x = 2, 2, 3, 4, 6, 7, 3, 2
    rng = np.random.default_rng(17)
    fil = rng.integers(-3, 4, g * k * c * y * x).astype(np.float32)
    inp = rng.integers(-3, 4, n * g * c * hi * wi).astype(np.float32)
    want, ho, wo = oracle.conv_fwd(fil, inp, "gkcyx", "ngchw", "ngkhw", n, g, c, k, hi, wi, y, x, (2, 1), (1, 0), (1, 2))
    got, outs = oracle.conv3d(fil, inp, "gkc012", "ngc012", "ngk012", n, g, c, k, (hi, wi, 1), (y, x, 1),
                              (2, 1, 1), (1, 0, 0), (1, 2, 1))
    assert outs == (ho, wo, 1) and np.array_equal(got, want)


@pytest.mark.parametrize("case", CONV3D_CASES)
@pytest.mark.parametrize("layouts", CONV3D_LAYOUTS, ids=lambda l: l[1])
def test_conv3d_gradients_vs_torch_autograd(oracle, case, layouts):
    """Both 3-D gradients against torch's autograd of conv3d (library routines)
    on integer-valued data in float64: every sum is exact, so a wrong index,
    a transposed operand or a missed padding check shows."""
    n, g, c, k, ins, fs, stride, pad, dil = case
    rng = np.random.default_rng(4000 + 16 * CONV3D_CASES.index(case) + CONV3D_LAYOUTS.index(layouts))
    outs = tuple(oracle.conv_out_dim(ins[a], fs[a], pad[a], pad[a], stride[a], dil[a]) for a in range(3))
    fil = rng.integers(-3, 4, (g, k, c) + fs).astype(np.float32)
    inp = rng.integers(-3, 4, (n, g, c) + ins).astype(np.float32)
    dout = rng.integers(-3, 4, (n, g, k) + outs).astype(np.float32)
    fl, il, ol = layouts
    x = torch.from_numpy(inp.reshape((n, g * c) + ins)).double().requires_grad_()
    w = torch.from_numpy(fil.reshape((g * k, c) + fs)).double().requires_grad_()
    y = torch.nn.functional.conv3d(x, w, stride=stride, padding=pad, dilation=dil, groups=g)
    y.backward(torch.from_numpy(dout.reshape((n, g * k) + outs)).double())
    dx = oracle.conv3d_bwd_data(_to_layout(fil, "gkc012", fl), _to_layout(dout, "ngk012", ol), fl, il, ol,
                                n, g, c, k, ins, fs, stride, pad, dil)
    dw = oracle.conv3d_bwd_weight(_to_layout(inp, "ngc012", il), _to_layout(dout, "ngk012", ol), fl, il, ol,
                                  n, g, c, k, ins, fs, stride, pad, dil)
    assert np.array_equal(dx.astype(np.float64), _to_layout(x.grad.numpy().reshape((n, g, c) + ins), "ngc012", il))
    assert np.array_equal(dw.astype(np.float64), _to_layout(w.grad.numpy().reshape((g, k, c) + fs), "gkc012", fl))


def test_conv3d_gradients_with_depth_one_are_the_2d_oracle(oracle):
    n, g, c, k, hi, wi, y, x = 2, 2, 3, 4, 6, 7, 3, 2
    rng = np.random.default_rng(18)
    ho, wo = oracle.conv_out_dim(hi, y, 1, 1, 2, 1), oracle.conv_out_dim(wi, x, 0, 0, 1, 2)
    fil = rng.integers(-3, 4, g * k * c * y * x).astype(np.float32)
    inp = rng.integers(-3, 4, n * g * c * hi * wi).astype(np.float32)
    dout = rng.integers(-3, 4, n * g * k * ho * wo).astype(np.float32)
    want_dx, _, _ = oracle.conv_bwd_data(fil, dout, "gkcyx", "ngchw", "ngkhw", n, g, c, k, hi, wi, y, x, (2, 1), (1, 0),
                                         (1, 2))
    want_dw, _, _ = oracle.conv_bwd_weight(inp, dout, "gkcyx", "ngchw", "ngkhw", n, g, c, k, hi, wi, y, x, (2, 1),
                                           (1, 0), (1, 2))
    a3 = ("gkc012", "ngc012", "ngk012", n, g, c, k, (hi, wi, 1), (y, x, 1), (2, 1, 1), (1, 0, 0), (1, 2, 1))
    assert np.array_equal(oracle.conv3d_bwd_data(fil, dout, *a3), want_dx)
    assert np.array_equal(oracle.conv3d_bwd_weight(inp, dout, *a3), want_dw)


def _bwd_golden_cases():
    with open(os.path.join(HERE, "golden", "conv_bwd_kats.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _bwd_golden_cases(), ids=lambda c: c["source"])
def test_conv_backward_reference_golden_vectors(oracle, case):
    """mlir/test/rocmlir-driver/cpu_conv2d/*_bwd_data.mlir, *_bwd_weight.mlir:
    all-ones data (-rand none), the literal gradient FileCheck expects."""
    f = case["flags"]
    n, c, k = int(f["batchsize"]), int(f["in_channels"]), int(f["out_channels"])
    hi, wi, y, x = int(f["in_h"]), int(f["in_w"]), int(f["fil_h"]), int(f["fil_w"])
    lay = {"kyxc": "gkyxc", "kcyx": "gkcyx", "nhwc": "nhwgc", "nchw": "ngchw",
           "nhwk": "nhwgk", "nkhw": "ngkhw"}
    geom = dict(stride=(int(f["conv_stride_h"]), int(f["conv_stride_w"])),
                pad=(int(f["padding_h"]), int(f["padding_w"])),
                dil=(int(f["dilation_h"]), int(f["dilation_w"])))
    ho = oracle.conv_out_dim(hi, y, geom["pad"][0], geom["pad"][0], geom["stride"][0], geom["dil"][0])
    wo = oracle.conv_out_dim(wi, x, geom["pad"][1], geom["pad"][1], geom["stride"][1], geom["dil"][1])
    layouts = (lay[f["fil_layout"]], lay[f["in_layout"]], lay[f["out_layout"]])
    dy = np.ones(n * k * ho * wo, np.float32)
    if f["operation"] == "conv_bwd_data":
        got, _, _ = oracle.conv_bwd_data(np.ones(k * c * y * x, np.float32), dy, *layouts,
                                         n, 1, c, k, hi, wi, y, x, **geom)
    else:
        got, _, _ = oracle.conv_bwd_weight(np.ones(n * c * hi * wi, np.float32), dy, *layouts,
                                           n, 1, c, k, hi, wi, y, x, **geom)
    assert got.size == len(case["expected"])
    assert np.array_equal(got.astype(np.float64), np.array(case["expected"]))


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("layouts", LAYOUTS)
def test_conv_backward_vs_torch_grad(oracle, case, layouts):
    """torch.nn.grad.conv2d_input / conv2d_weight (library routines) on
    integer-valued data in float64: every sum exact."""
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    rng = np.random.default_rng(2000 + 16 * CONV_CASES.index(case) + LAYOUTS.index(layouts))
    ho = oracle.conv_out_dim(hi, y, pad[0], pad[0], stride[0], dil[0])
    wo = oracle.conv_out_dim(wi, x, pad[1], pad[1], stride[1], dil[1])
    fil = rng.integers(-3, 4, (g, k, c, y, x)).astype(np.float32)
    inp = rng.integers(-3, 4, (n, g, c, hi, wi)).astype(np.float32)
    dy = rng.integers(-3, 4, (n, g, k, ho, wo)).astype(np.float32)
    fl, il, ol = layouts
    t_in = torch.from_numpy(inp.reshape(n, g * c, hi, wi)).double()
    t_fil = torch.from_numpy(fil.reshape(g * k, c, y, x)).double()
    t_dy = torch.from_numpy(dy.reshape(n, g * k, ho, wo)).double()
    dx, _, _ = oracle.conv_bwd_data(_to_layout(fil, "gkcyx", fl), _to_layout(dy, "ngkhw", ol), fl, il, ol,
                                    n, g, c, k, hi, wi, y, x, stride, pad, dil)
    ref = torch.nn.grad.conv2d_input(t_in.shape, t_fil, t_dy, stride=stride, padding=pad, dilation=dil,
                                     groups=g).numpy()
    assert np.array_equal(dx.astype(np.float64), _to_layout(ref.reshape(n, g, c, hi, wi), "ngchw", il))
    dw, _, _ = oracle.conv_bwd_weight(_to_layout(inp, "ngchw", il), _to_layout(dy, "ngkhw", ol), fl, il, ol,
                                      n, g, c, k, hi, wi, y, x, stride, pad, dil)
    ref = torch.nn.grad.conv2d_weight(t_in, t_fil.shape, t_dy, stride=stride, padding=pad, dilation=dil,
                                      groups=g).numpy()
    assert np.array_equal(dw.astype(np.float64), _to_layout(ref.reshape(g, k, c, y, x), "gkcyx", fl))


def test_conv_i8_widens_before_multiply(oracle):
    # deliberate deviation from rocmlir-gen.cpp:1955-1960 (i8 multiply wraps)
    out, _, _ = oracle.conv_fwd(np.array([-128], np.int8), np.array([-128], np.int8),
                                "gkcyx", "ngchw", "ngkhw", 1, 1, 1, 1, 1, 1, 1, 1)
    assert out[0] == 16384


def test_conv_output_range_sample(oracle):
    rng = np.random.default_rng(5)
    fil = rng.standard_normal(4 * 3 * 3 * 3).astype(np.float32)
    inp = rng.standard_normal(2 * 3 * 6 * 6).astype(np.float32)
    full, _, _ = oracle.conv_fwd(fil, inp, "gkyxc", "nhwgc", "nhwgk", 2, 1, 3, 4, 6, 6, 3, 3, pad=(1, 1))
    part, _, _ = oracle.conv_fwd(fil, inp, "gkyxc", "nhwgc", "nhwgk", 2, 1, 3, 4, 6, 6, 3, 3, pad=(1, 1),
                                 out_range=(10, 50), threads=3)
    assert np.array_equal(part[10:50], full[10:50]) and not part[:10].any() and not part[50:].any()


# ----------------------------------------------------------------- attention
def test_softmax_reference_vector(oracle):
    # migraphx_softmax.cpu.e2e.mlir:8-9
    got = oracle.softmax(np.array([[0, 2, 3, 1]], np.float32))[0]
    assert np.allclose(got, [0.0320586, 0.236883, 0.643914, 0.0871443], rtol=1e-5)


def _attn_ref64(Q, K, V, scale, bias=None):
    S = np.einsum("gid,gjd->gij", Q.astype(np.float64), K.astype(np.float64)) * scale
    if bias is not None:
        S = S + bias
    P = torch.softmax(torch.from_numpy(S), dim=-1).numpy()
    return np.einsum("gij,gje->gie", P, V.astype(np.float64))


@pytest.mark.parametrize("tQ,tK,tV,tO", [(0, 0, 0, 0), (0, 1, 0, 0), (1, 1, 1, 1), (1, 0, 1, 0), (0, 1, 1, 1)])
def test_attention_vs_float64_all_layouts(oracle, tQ, tK, tV, tO):
    rng = np.random.default_rng(20 + tQ + 2 * tK + 4 * tV + 8 * tO)
    G, sq, sk, dqk, dv = 2, 9, 27, 8, 5
    Q = rng.standard_normal((G, sq, dqk)).astype(np.float32)
    K = rng.standard_normal((G, sk, dqk)).astype(np.float32)   # logical [G,sk,d]
    V = rng.standard_normal((G, sk, dv)).astype(np.float32)
    bias = rng.standard_normal((G, sq, sk)).astype(np.float32)
    scale = 0.37
    # storage: K is [G,d,sk] by default, [G,sk,d] with transK
    got = oracle.attention(_store(Q, tQ), _store(K, not tK), _store(V, tV), G, sq, sk, dqk, dv,
                           scale=scale, bias_t=bias, transQ=tQ, transK=tK, transV=tV, transO=tO)
    want = _store(_attn_ref64(Q, K, V, scale, bias), tO).ravel()
    assert np.allclose(got, want, rtol=0, atol=3e-6)


def test_attention_where_mask_vs_float64(oracle):
    """migraphx.where(mask, scale * Q K^T [+ bias], other) in front of the softmax (mixr-attn-where.mlir:11):
    against torch.where + softmax in float64; an all-ones mask changes nothing, an all-zero mask makes the
    weights softmax(other) whatever Q and K hold (an additive mask, or a select on the wrong side, fails both)."""
    rng = np.random.default_rng(33)
    G, sq, sk, d, dv = 2, 7, 19, 8, 5
    Q = rng.standard_normal((G, sq, d)).astype(np.float32)
    K = rng.standard_normal((G, sk, d)).astype(np.float32)
    V = rng.standard_normal((G, sk, dv)).astype(np.float32)
    bias = rng.standard_normal((G, sq, sk)).astype(np.float32)
    other = rng.standard_normal((G, sq, sk)).astype(np.float32) * 3
    mask = (rng.random((G, sq, sk)) < 0.6).astype(np.int8)
    mask[0, 0, :] = 0          # a fully masked row
    mask[1, 2, :] = 1          # an untouched row
    att = lambda **kw: oracle.attention(Q, K, V, G, sq, sk, d, dv, transK=True, **kw).reshape(G, sq, dv)
    for b in (None, bias):
        S = np.einsum("gid,gjd->gij", Q.astype(np.float64), K.astype(np.float64)) * 0.3
        if b is not None:
            S = S + b
        S = torch.where(torch.from_numpy(mask != 0), torch.from_numpy(S), torch.from_numpy(other.astype(np.float64)))
        want = np.einsum("gij,gje->gie", torch.softmax(S, dim=-1).numpy(), V.astype(np.float64))
        assert np.allclose(att(scale=0.3, bias_t=b, mask=mask, other=other), want, rtol=0, atol=3e-6)
    assert np.array_equal(att(scale=0.3, mask=np.ones_like(mask), other=other), att(scale=0.3))
    only_other = np.einsum("gij,gje->gie", torch.softmax(torch.from_numpy(other.astype(np.float64)), dim=-1).numpy(),
                           V.astype(np.float64))
    assert np.allclose(att(scale=0.3, mask=np.zeros_like(mask), other=other), only_other, rtol=0, atol=3e-6)


def test_attention_program_vs_float64_and_the_fixed_chain(oracle):
    """The pre-softmax region as postfix code (RockOps.td:208-254).  The reference's two trees -- (x * t0) -> exp
    -> + t1 (mixr-attention-padded-scale-bias-exp.mlir:12-15) and x * (t0 - t1) + (t2 + t3)
    (...-complex-tree-elemwise.mlir:17-23), at their 7 x 7 x 3 shape and a larger one -- against torch in float64
    written out operation by operation; the programs that spell the fixed chain (scale tensor, scale, bias, where)
    against the C oracle, which takes those as arguments; operand order of the non-commutative tokens by hand."""
    rng = np.random.default_rng(35)
    for G, sq, sk, d, dv in ((1, 7, 7, 3, 3), (2, 9, 21, 8, 5)):
        Q = rng.standard_normal((G, sq, d)).astype(np.float32)
        K = rng.standard_normal((G, d, sk)).astype(np.float32)
        V = rng.standard_normal((G, sk, dv)).astype(np.float32)
        t = [rng.standard_normal((G, sq, sk)).astype(np.float32) * 0.5 for _ in range(4)]
        q64, k64, v64 = (torch.from_numpy(a.astype(np.float64)) for a in (Q, K, V))
        t64 = [torch.from_numpy(a.astype(np.float64)) for a in t]
        s64 = q64 @ k64
        want = torch.softmax(torch.exp(s64 * t64[0]) + t64[1], dim=-1) @ v64
        got = oracle.attention_program(Q, K, V, G, sq, sk, d, dv, "x,t0,mul,exp,t1,add", t[:2])
        assert np.allclose(got.reshape(G, sq, dv), want.numpy(), rtol=0, atol=5e-6)
        want = torch.softmax(s64 * (t64[0] - t64[1]) + (t64[2] + t64[3]), dim=-1) @ v64
        got = oracle.attention_program(Q, K, V, G, sq, sk, d, dv, "x,t0,t1,sub,mul,t2,t3,add,add", t)
        assert np.allclose(got.reshape(G, sq, dv), want.numpy(), rtol=0, atol=5e-6)
        # the fixed chain, spelt as programs, against the C oracle's arguments (K stored [G, sk, d] there)
        Kt = np.ascontiguousarray(K.transpose(0, 2, 1))
        mask = (rng.random((G, sq, sk)) < 0.5).astype(np.int8)
        ref = oracle.attention(Q, Kt, V, G, sq, sk, d, dv, scale=0.3, scale_t=t[0], bias_t=t[1], transK=True)
        got = oracle.attention_program(Q, K, V, G, sq, sk, d, dv, "x,t0,mul,c:0.3,mul,t1,add", t[:2])
        assert np.allclose(got, ref, rtol=0, atol=2e-6)
        ref = oracle.attention(Q, Kt, V, G, sq, sk, d, dv, scale=0.3, mask=mask, other=t[2], transK=True)
        got = oracle.attention_program(Q, K, V, G, sq, sk, d, dv, "t0,x,c:0.3,mul,t1,where", [mask, t[2]])
        assert np.allclose(got, ref, rtol=0, atol=2e-6)
    # operand order: a b sub = a - b, a b div = a / b, c a b where = c ? a : b; unary tokens by their values
    x = np.array([[4.0, -2.0]], np.float32)
    run = lambda prog, *ins: oracle.run_attention_program(prog, x, ins).tolist()
    assert run("x,c:1,sub") == [[3.0, -3.0]] and run("c:1,x,sub") == [[-3.0, 3.0]]
    assert run("x,c:2,div") == [[2.0, -1.0]] and run("c:8,x,div") == [[2.0, -4.0]]
    assert run("x,c:10,c:20,where") == [[10.0, 10.0]] and run("t0,c:10,c:20,where", np.array([[0, 1]], np.int8)) == [[20.0, 10.0]]
    assert run("x,relu") == [[4.0, 0.0]] and run("x,neg,abs") == [[4.0, 2.0]]
    assert run("x,c:0,max,x,c:0,min,add") == [[4.0, -2.0]]
    assert np.allclose(run("x,sigmoid"), [[1 / (1 + np.exp(-4.0)), 1 / (1 + np.exp(2.0))]], atol=1e-7)
    assert np.allclose(run("x,c:4,div,tanh"), np.tanh([[1.0, -0.5]]), atol=1e-7)
    assert np.allclose(run("x,c:4,div,erf"), [[0.8427007929, -0.5204998778]], atol=1e-7)


def test_attention_invariants(oracle):
    rng = np.random.default_rng(21)
    G, sq, sk, d, dv = 1, 4, 16, 8, 6
    Q = rng.standard_normal((G, sq, d)).astype(np.float32)
    K = rng.standard_normal((G, sk, d)).astype(np.float32)
    V = rng.standard_normal((G, sk, dv)).astype(np.float32)
    att = lambda q, k, v, **kw: oracle.attention(q, k, v, G, sq, sk, d, dv, transK=True, **kw).reshape(G, sq, dv)
    # rows of P sum to one
    assert np.allclose(att(Q, K, np.ones_like(V)), 1.0, atol=1e-6)
    # Q = 0 -> uniform weights -> column mean of V
    assert np.allclose(att(np.zeros_like(Q), K, V), V.mean(axis=1, keepdims=True), atol=1e-6)
    # permuting keys and values together changes nothing (up to summation order)
    perm = rng.permutation(sk)
    assert np.allclose(att(Q, K, V), att(Q, K[:, perm], V[:, perm]), atol=1e-6)
    # scale tensor of constant s == scalar scale s
    st = np.full((G, sq, sk), 0.25, np.float32)
    assert np.array_equal(att(Q, K, V, scale_t=st), att(Q, K, V, scale=0.25))
    # query-row sample
    part = oracle.attention(Q, K, V, G, sq, sk, d, dv, transK=True, q_rows=(1, 3)).reshape(G, sq, dv)
    assert np.array_equal(part[:, 1:3], att(Q, K, V)[:, 1:3]) and not part[:, 0].any()


# ----------------------------------------------------------------- epilogue
def test_dequantize_formula(oracle):
    # (float(acc) - float(zp)) * scale, MIGraphXToTosa.cpp:874-902
    acc = np.array([0, 1, -7, 100, 2 ** 26 + 3, -(2 ** 26) - 5], np.int64)
    got = oracle.dequantize(acc, 0.01, 3)
    want = (acc.astype(np.int32).astype(np.float32) - np.float32(3)) * np.float32(0.01)
    assert np.array_equal(got, want)
    assert got[1] == np.float32(-0.02)
    # 2^26+3 is not representable in f32: the int->float conversion rounds to even
    assert oracle.dequantize(np.array([2 ** 26 + 3], np.int64), 1.0)[0] == np.float32(2 ** 26 + 4)


def test_quantize_formula(oracle):
    # clamp(round_even(x * (1/scale)) + zp, -128, 127), MIGraphXToTosa.cpp:904-982
    x = np.array([0.0, 0.25, 0.75, 1.25, -0.25, -0.75, 100.0, -100.0, 63.4], np.float32)
    got = oracle.quantize_i8(x, 0.5, 1)
    assert got.tolist() == [1, 1, 3, 3, 1, -1, 127, -128, 127]
    assert oracle.quantize_i8(np.array([63.4], np.float32), 0.5, 0)[0] == 127
    assert oracle.quantize_i8(np.array([63.2], np.float32), 0.5, 0)[0] == 126


def test_per_channel_quantisation_formulas(oracle):
    """One scale and zero point per output channel (MIGraphXToTosa.cpp:874-982 with broadcast tensors, as in
    mixr-resnet-fusion-case-1-quantization.mlir:8-9): hand-computed values, channel c must see only element c
    of each vector (a transposed or shifted index fails), and constant vectors reduce to the per-tensor routines."""
    acc = np.array([[10, -20, 7], [3, 4, -5]], np.int64)
    scale = np.array([0.5, 0.25, 2.0], np.float32)
    zp = np.array([2, 0, -1], np.int32)
    got = oracle.dequantize_per_channel(acc, scale, zp)
    assert got.tolist() == [[4.0, -5.0, 16.0], [0.5, 1.0, -8.0]]
    assert oracle.dequantize_per_channel(acc, scale).tolist() == [[5.0, -5.0, 14.0], [1.5, 1.0, -10.0]]
    x = np.array([[1.0, 1.0, 1.0], [-3.3, 0.3, 300.0]], np.float32)
    qs = np.array([0.5, 0.25, 2.0], np.float32)
    qz = np.array([0, 10, -100], np.int32)
    # 1/0.5 = 2, 1/0.25 = 4, 1/2 = 0.5: round_even(x * inv) + zp, clamped
    assert oracle.quantize_i8_per_channel(x, qs, qz).tolist() == [[2, 14, -100], [-7, 11, 50]]
    assert oracle.quantize_i8_per_channel(x, qs).tolist() == [[2, 4, 0], [-7, 1, 127]]
    rng = np.random.default_rng(5)
    big = rng.integers(-2 ** 20, 2 ** 20, (37, 11)).astype(np.int64)
    assert np.array_equal(oracle.dequantize_per_channel(big, np.full(11, 0.013, np.float32), np.full(11, -4, np.int32)),
                          oracle.dequantize(big, 0.013, -4))
    xf = rng.standard_normal((37, 11)).astype(np.float32) * 50
    assert np.array_equal(oracle.quantize_i8_per_channel(xf, np.full(11, 0.37, np.float32), np.full(11, 5, np.int32)),
                          oracle.quantize_i8(xf, 0.37, 5))
    # column by column against the per-tensor routine with that column's values
    sc = rng.uniform(0.01, 2.0, 11).astype(np.float32)
    zz = rng.integers(-9, 9, 11).astype(np.int32)
    d = oracle.dequantize_per_channel(big, sc, zz)
    q = oracle.quantize_i8_per_channel(xf, sc, zz)
    for c in range(11):
        assert np.array_equal(d[:, c], oracle.dequantize(big[:, c].copy(), sc[c], int(zz[c])))
        assert np.array_equal(q[:, c], oracle.quantize_i8(xf[:, c].copy(), sc[c], int(zz[c])))


def test_scale_bias(oracle):
    x = np.arange(6, dtype=np.float32).reshape(2, 3)
    got = oracle.scale_bias(x, 2, 3, 0.5, np.array([1, 2, 3], np.float32))
    assert np.array_equal(got, x * 0.5 + np.array([1, 2, 3], np.float32))


# ----------------------------------------------------------------- verifier / fill
def test_verify_float_metrics_by_hand(oracle):
    val = np.array([1.0, 2.0, 0.0, -4.0], np.float32)
    gpu = np.array([1.0, 2.5, 0.5, -4.0], np.float32)
    r = oracle.verify_float(gpu, val, thr_rms=1.0, thr_abs=1.0, thr_rel=1.0)
    # RMS = sqrt(0.25 + 0.25) / (maxMag=4 * sqrt(4))   (conv-validation-wrappers.cpp:199-200)
    assert r.rms == pytest.approx(np.sqrt(0.5) / 8.0)
    assert r.max_abs_diff == 0.5
    assert r.max_rel_diff == 0.25           # val == 0 is excluded from relDiff
    assert r.ave_abs_diff == 0.25
    assert r.passed()
    r = oracle.verify_float(gpu, val, thr_rms=0.01, thr_abs=1.0, thr_rel=0.1)
    assert (r.pass_rms, r.pass_abs, r.pass_rel) == (0, 1, 0)


def test_verify_float_inf_reference_is_fp16_max(oracle):
    r = oracle.verify_float(np.array([65504.0], np.float32), np.array([np.inf], np.float32))
    assert r.max_abs_diff == 0.0 and r.pass_abs


def test_verify_int(oracle):
    gpu = np.array([1, 2, -5, 7], np.int32)
    val = np.array([1, 3, -5, 2 ** 31 + 7], np.int64)
    fails, ovf, mad = oracle.verify_int(gpu, val)
    assert (fails, ovf, mad) == (2, 1, 2 ** 31)
    assert oracle.verify_int(gpu, gpu.astype(np.int64)) == (0, 0, 0)


def test_fill_rand_follows_libc_rand(oracle):
    libc = ctypes.CDLL(None)
    libc.rand.restype = ctypes.c_int
    oracle.seed(7)
    ints = oracle.fill_rand(20, -5, 5, as_float=False)
    libc.srand(7)
    want = [float((libc.rand() % 10) - 5) for _ in range(20)]
    assert ints.tolist() == want and ints.min() >= -5 and ints.max() < 5
    oracle.seed(7)
    fl = oracle.fill_rand(20, -1, 1, as_float=True)
    libc.srand(7)
    want = [np.float32(np.float32(2 * float(libc.rand()) / 2147483647.0) + np.float32(-1)) for _ in range(20)]
    assert fl.tolist() == [float(w) for w in want]
    assert oracle.fill_fixed(5, is_int=True).tolist() == [1, -1, 2, 1, -1]
    # min == max: constant (0.1x for floats), conv-validation-wrappers.cpp:41-45
    assert oracle.fill_rand(3, 1, 1, as_float=True).tolist() == [np.float32(0.1)] * 3


def test_rand_fill_reproduces_the_reference_erf_vector():
    """mixr-gemm-erf_f32.mlir runs `-rand 3` (srand(3), integers in [-5, 5),
    arguments filled in order) through dot + erf and FileChecks the printed
    result: reproducing it pins the fill's generator, range and order."""
    import json
    import math
    import os
    from oracle import rock_oracle as o
    here = os.path.dirname(os.path.abspath(__file__))
    case = next(c for c in json.load(open(os.path.join(here, "golden", "fusion_kats.json")))
                if c["source"].endswith("erf_f32.mlir"))
    o.seed(int(case["rand"]))
    a = o.fill_rand(case["m"] * case["k"], -5, 5, False)
    b = o.fill_rand(case["k"] * case["n"], -5, 5, False)
    c = o.gemm(a, b, 1, case["m"], case["n"], case["k"])
    assert [float("%.6g" % math.erf(v)) for v in np.asarray(c).ravel()] == case["expected"]
