"""GPU parity: per-channel (broadcast-vector) quantisation scales and zero points in the epilogue of GEMM and
forward convolution, through the C ABI, bit for bit against the oracle's restatement of the reference's
dequantizelinear / quantizelinear lowering with channel tensors (MIGraphXToTosa.cpp:874-982;
mlir/test/fusion/resnet50-e2e/mixr-resnet-fusion-case-1-quantization.mlir).

Every step is one IEEE operation on exact int32 accumulators (subtract, multiply, reciprocal, multiply, round to
even, add, clamp), so the kernels must reproduce the oracle exactly on every tile, with real-valued scales."""
import numpy as np
import pytest
import torch

from tests.gpu_util import CODE, quantise, to_f32, to_gpu
from tests.test_gpu_conv import NCHW, NHWC, _run as _run_conv

pytestmark = pytest.mark.gpu


def _vectors(n, seed, gpu, zp_dtype=np.int32):
    rng = np.random.default_rng(seed)
    sv = rng.uniform(1e-4, 3e-3, n).astype(np.float32)
    zv = rng.integers(-60, 60, n).astype(zp_dtype)
    qsv = rng.uniform(0.05, 1.5, n).astype(np.float32)
    qzv = rng.integers(-20, 20, n).astype(zp_dtype)
    dev = lambda a: torch.from_numpy(a).to(gpu)  # noqa: E731
    return (sv, zv, qsv, qzv), (dev(sv), dev(zv), dev(qsv), dev(qzv))


def _gemm(rock, oracle, gpu, M, N, K, seed, **kw):
    rng = np.random.default_rng(seed)
    A = rng.integers(-128, 128, (1, M, K)).astype(np.int8)
    B = rng.integers(-128, 128, (1, N, K)).astype(np.int8)
    info = {}
    out = rock.gemm(torch.from_numpy(A).to(gpu), torch.from_numpy(B).to(gpu), transB=True, info=info, **kw)
    torch.cuda.synchronize()
    ref = oracle.gemm(A, B, 1, M, N, K, False, True, False).reshape(M, N)
    return out, ref, info


TILES = [("v2:256,256,8,128,16,16,1,1,1", "256x256_fast_e"), ("v2:256,128,8,128,16,16,1,1,1", "256x128_fast_e"),
         ("v2:128,128,8,64,16,16,1,1,1", "128x128_fast_e"), ("v2:64,64,8,32,16,16,1,1,1", "64x64_fast_e"),
         ("v2:32,32,4,32,32,16,4,1,1", "32x32_splitk_e")]


@pytest.mark.parametrize("perf,suffix", TILES, ids=[s for _, s in TILES])
@pytest.mark.parametrize("zp_dtype", [np.int32, np.int8], ids=["zp-i32", "zp-i8"])
def test_gemm_per_channel_dequantise_every_tile(rock, oracle, gpu, perf, suffix, zp_dtype):
    """(float(acc) - float(zp[n])) * scale[n] -> f16, on the rolled-epilogue twin of every tile (ragged M and N)."""
    M, N, K = 520, 390, 256
    (sv, zv, _, _), (dsv, dzv, _, _) = _vectors(N, 71, gpu, zp_dtype)
    out, ref, info = _gemm(rock, oracle, gpu, M, N, K, 72, out_dtype="f16", scale=dsv, zero_point=dzv, perf_config=perf)
    assert info["kernel_name"] == "rock_gemm_i8_" + suffix
    want = oracle.round_through(oracle.dequantize_per_channel(ref, sv, zv.astype(np.int32)), CODE["f16"])
    assert np.array_equal(to_f32(out, "f16").reshape(M, N), want)


@pytest.mark.parametrize("perf,suffix", TILES, ids=[s for _, s in TILES])
def test_gemm_per_channel_requantise_every_tile(rock, oracle, gpu, perf, suffix):
    """dequantise per channel -> + bias -> relu -> quantise per channel back to int8 (scale and zero point
    vectors on both sides)."""
    M, N, K = 300, 270, 384
    (sv, zv, qsv, qzv), (dsv, dzv, dqsv, dqzv) = _vectors(N, 73, gpu)
    bias = np.random.default_rng(74).integers(-40, 40, N).astype(np.float32)
    out, ref, info = _gemm(rock, oracle, gpu, M, N, K, 75, out_dtype="i8", scale=dsv, zero_point=dzv,
                           bias=torch.from_numpy(bias).to(gpu), relu=True, quant_scale=dqsv, out_zero_point=dqzv,
                           perf_config=perf)
    assert info["kernel_name"] == "rock_gemm_i8_" + suffix
    x = np.maximum(oracle.dequantize_per_channel(ref, sv, zv) + bias[None, :], np.float32(0))
    want = oracle.quantize_i8_per_channel(x, qsv, qzv)
    assert np.array_equal(out.cpu().numpy().reshape(M, N), want)


def test_gemm_per_channel_mixed_with_scalars_and_element_wise_kernel(rock, oracle, gpu):
    """Only some of the four values as vectors (the others stay scalars), K-major storage, and the element-wise
    kernel (operands that are not whole chunks, conversion declined)."""
    M, N, K = 70, 45, 97
    (sv, _, qsv, _), (dsv, _, dqsv, _) = _vectors(N, 76, gpu)
    rng = np.random.default_rng(77)
    A = rng.integers(-128, 128, (1, M, K)).astype(np.int8)
    B = rng.integers(-128, 128, (1, K, N)).astype(np.int8)
    ref = oracle.gemm(A, B, 1, M, N, K, False, False, False).reshape(M, N)
    for convert in (True, False):
        info = {}
        out = rock.gemm(torch.from_numpy(A).to(gpu), torch.from_numpy(B).to(gpu), out_dtype="i8", scale=dsv, zero_point=-7,
                        quant_scale=0.25, out_zero_point=3, layout_conversion=convert, info=info)
        torch.cuda.synchronize()
        assert ("_generic" in info["kernel_name"]) == (not convert)
        want = oracle.quantize_i8(oracle.dequantize_per_channel(ref, sv, np.full(N, -7, np.int32)), 0.25, 3)
        assert np.array_equal(out.cpu().numpy().reshape(M, N), want)
        out = rock.gemm(torch.from_numpy(A).to(gpu), torch.from_numpy(B).to(gpu), out_dtype="i8", scale=0.002,
                        quant_scale=dqsv, layout_conversion=convert)
        torch.cuda.synchronize()
        want = oracle.quantize_i8_per_channel(oracle.dequantize(ref, 0.002, 0), qsv)
        assert np.array_equal(out.cpu().numpy().reshape(M, N), want)


def test_gemm_f16_per_channel_scale(rock, oracle, gpu):
    """A float problem: acc * scale[n], f32 accumulators exact on small integers."""
    M, N, K = 200, 136, 128
    rng = np.random.default_rng(78)
    A = rng.integers(-2, 3, (1, M, K)).astype(np.float32)
    B = rng.integers(-2, 3, (1, N, K)).astype(np.float32)
    sv = rng.uniform(0.1, 2.0, N).astype(np.float32)
    rawA, Aq = quantise(A, "f16")
    rawB, Bq = quantise(B, "f16")
    out = rock.gemm(to_gpu(rawA, "f16", gpu), to_gpu(rawB, "f16", gpu), transB=True, out_dtype="f32",
                    scale=torch.from_numpy(sv).to(gpu))
    torch.cuda.synchronize()
    ref = oracle.gemm(Aq, Bq, 1, M, N, K, False, True, False).reshape(M, N)
    assert np.array_equal(to_f32(out, "f32").reshape(M, N), ref * sv[None, :])


def _channels_last(flat, layouts, n, gk, ho, wo):
    """The oracle's flat output as [pixels][channels]."""
    if layouts[2] == "nhwgk":
        return flat.reshape(n * ho * wo, gk), lambda a: a.reshape(-1)
    a = flat.reshape(n, gk, ho * wo).transpose(0, 2, 1).reshape(n * ho * wo, gk)
    return a, lambda b: b.reshape(n, ho * wo, gk).transpose(0, 2, 1).reshape(-1)


@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=["nhwc", "nchw"])
@pytest.mark.parametrize("shape,perf,kernel", [
    ((2, 1, 64, 72, 14, 14, 3, 3, (1, 1), (1, 1)), None, None),
    ((2, 2, 32, 40, 9, 9, 3, 3, (2, 2), (1, 1)), "v2:64,64,8,32,16,16,1,1,1", "64x64_fast_e"),
    ((4, 1, 128, 128, 28, 28, 3, 3, (1, 1), (1, 1)), "v2:224,128,8,224,32,16,1,1,1", "direct224_e"),
    ((1, 1, 20, 12, 7, 7, 3, 3, (1, 1), (0, 0)), None, "generic")],
    ids=["table", "64x64-groups-stride2", "window-resident", "element-wise"])
def test_conv_per_channel_requantise(rock, oracle, gpu, layouts, shape, perf, kernel):
    n, g, c, k, hi, wi, y, x, stride, pad = shape
    (sv, zv, qsv, qzv), (dsv, dzv, dqsv, dqzv) = _vectors(g * k, 81, gpu)
    info = {}
    extra = {"perf_config": perf} if perf else {}
    if kernel == "generic":
        extra["layout_conversion"] = False
    bias = np.random.default_rng(80).integers(-30, 30, g * k).astype(np.float32)
    out, _, ref = _run_conv(rock, oracle, gpu, "i8", n, g, c, k, hi, wi, y, x, stride, pad, (1, 1), layouts, True, 82,
                            out_dtype="i8", scale=dsv, zero_point=dzv, quant_scale=dqsv, out_zero_point=dqzv, info=info,
                            bias=torch.from_numpy(bias).to(gpu), **extra)
    # (behind layout conversions the window-resident kernel, a plan with a workspace of its own, is not offered)
    if kernel and not (layouts is NCHW and kernel.startswith("direct224")):
        assert info["kernel_name"].endswith(kernel), info
    ho = (hi + 2 * pad[0] - y) // stride[0] + 1
    wo = (wi + 2 * pad[1] - x) // stride[1] + 1
    acc, back = _channels_last(ref, layouts, n, g * k, ho, wo)
    want = back(oracle.quantize_i8_per_channel(oracle.dequantize_per_channel(acc, sv, zv) + bias[None, :], qsv, qzv))
    assert np.array_equal(out.cpu().numpy().ravel(), want)


@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=["nhwc", "nchw"])
@pytest.mark.parametrize("perf", [None, "v2:64,64,8,32,16,16,1,1,1", "v2:64,64,8,32,16,16,1,0,1"],
                         ids=["table", "64x64", "64x64-rolled"])
def test_grouped_conv_bias_runs_over_all_groups_channels(rock, oracle, gpu, layouts, perf):
    """The bias of a grouped convolution has groups * k entries: group g's tile adds entries g*k ... g*k+k-1
    (f16, small integers, exact)."""
    n, g, c, k, hw = 2, 4, 16, 24, 10
    bias = np.random.default_rng(85).integers(-9, 10, g * k).astype(np.float32)
    extra = {"perf_config": perf} if perf else {}
    out, od, ref = _run_conv(rock, oracle, gpu, "f16", n, g, c, k, hw, hw, 3, 3, (1, 1), (1, 1), (1, 1), layouts, True,
                             86, bias=torch.from_numpy(bias).to(gpu), **extra)
    acc, back = _channels_last(ref, layouts, n, g * k, hw, hw)
    assert np.array_equal(to_f32(out, od), back(acc + bias[None, :]))


def test_reference_resnet_quantisation_chain(rock, oracle, gpu):
    """mixr-resnet-fusion-case-1-quantization.mlir: int8 NCHW convolution 128 -> 128, 3x3, stride 2, padding 1 over
    56 x 56, dequantised and re-quantised with the SAME <1x128x1x1xf32> scale vector, int8 result."""
    n, g, c, k, hi, wi = 1, 1, 128, 128, 56, 56
    sv = np.random.default_rng(83).uniform(0.5, 4.0, k).astype(np.float32)
    dsv = torch.from_numpy(sv).to(gpu)
    info = {}
    out, _, ref = _run_conv(rock, oracle, gpu, "i8", n, g, c, k, hi, wi, 3, 3, (2, 2), (1, 1), (1, 1), NCHW, True, 84,
                            out_dtype="i8", scale=dsv, quant_scale=dsv, info=info)
    assert info["kernels"][-1].startswith("rock_conv_i8_") and info["kernels"][-1].endswith("_e")
    acc, back = _channels_last(ref, NCHW, n, k, 28, 28)
    want = back(oracle.quantize_i8_per_channel(oracle.dequantize_per_channel(acc, sv), sv))
    assert np.array_equal(out.cpu().numpy().ravel(), want)
    # dequantising and re-quantising with one scale gives the saturated accumulator back (x * s * (1/s) rounds to x
    # or a neighbour; int8 accumulators of full-range data saturate almost everywhere)
    sat = np.clip(acc, -128, 127)
    assert np.mean(np.abs(back(sat).astype(np.int32) - want.astype(np.int32)) <= 1) == 1.0
