"""GPU parity: GEMM through the C ABI vs the CPU oracle.

Integer-valued operands make every product and partial sum exact in the
accumulator, so the result must match the oracle bit for bit for every
element type; real-valued operands are held to the reference verifier's RMS
gate (3e-5 for f32 results, 1e-3 for f16).  int8 -> int32 is always
bit-exact."""
import itertools

import numpy as np
import pytest
import torch

from tests.gpu_util import CODE, check_float, quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu

FLOAT_TYPES = ["f32", "f16", "bf16", "fp8", "bf8"]


def _store(mat, trans):
    return np.ascontiguousarray(mat.transpose(0, 2, 1) if trans else mat)


def _run_case(rock, oracle, gpu, t, G, M, N, K, tA, tB, tC, integer, seed, out_dtype=None, **epi):
    ta, tb = (t.split("_") + [t])[:2] if "_" in t else (t, t)
    rng = np.random.default_rng(seed)
    if ta == "i8":
        A = rng.integers(-128, 128, (G, M, K)).astype(np.float32)
        B = rng.integers(-128, 128, (G, K, N)).astype(np.float32)
    elif integer:
        A = rng.integers(-2, 3, (G, M, K)).astype(np.float32)
        B = rng.integers(-2, 3, (G, K, N)).astype(np.float32)
    else:
        A = rng.uniform(-1, 1, (G, M, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (G, K, N)).astype(np.float32)
    rawA, Aq = quantise(_store(A, tA), ta)
    rawB, Bq = quantise(_store(B, tB), tb)
    out = rock.gemm(to_gpu(rawA, ta, gpu), to_gpu(rawB, tb, gpu), transA=tA, transB=tB, transC=tC,
                    out_dtype=out_dtype, **epi)
    torch.cuda.synchronize()
    od = out_dtype or {"i8": "i32", "fp8": "f32", "bf8": "f32"}.get(ta, ta)
    assert out.shape == ((G, N, M) if tC else (G, M, N))
    if ta == "i8":
        ref = oracle.gemm(rawA, rawB, G, M, N, K, tA, tB, tC)
    else:
        ref = oracle.gemm(Aq, Bq, G, M, N, K, tA, tB, tC)
    return out, od, ref


# every transpose combination x every operand type, ragged sizes (GemmVariants.toml:5-40)
@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8", "fp8", "bf8", "fp8_bf8", "bf8_fp8"])
@pytest.mark.parametrize("tA,tB,tC", list(itertools.product([False, True], repeat=3)))
@pytest.mark.parametrize("convert", [True, False], ids=["padded-copies", "element-wise"])
def test_gemm_transposes_exact(rock, oracle, gpu, t, tA, tB, tC, convert):
    """Nothing here is a whole 16-byte chunk: by default the operands are
    copied into zero-padded K-contiguous ones and a vector kernel multiplies
    the copies; `layout_conversion=False` keeps the element-wise kernel."""
    info = {}
    out, od, ref = _run_case(rock, oracle, gpu, t, 2, 70, 45, 97, tA, tB, tC, True, 100,
                             layout_conversion=convert, info=info)
    assert ("_generic" in info["kernel_name"]) == (not convert), info
    assert len(info["kernels"]) == (2 if convert else 1), info
    got = to_f32(out, od)
    if t == "i8":
        fails, ovf, mad = oracle.verify_int(out.cpu().numpy().ravel(), ref)
        assert (fails, ovf) == (0, 0), (fails, mad)
    else:
        assert np.array_equal(got, ref)


# K-major operands (A stored [K,M] and/or B stored [K,N], the reference's
# default B): the transposing-read kernels, every tile, ragged tiles and K tails.
KM_STORAGE = {"nn": (False, False), "tn": (True, False), "tt": (True, True)}
KM_SHAPES = [(1, 256, 256, 256), (2, 144, 208, 208), (1, 304, 80, 1008), (1, 64, 48, 80)]


@pytest.mark.parametrize("tile", ["256,256", "128,128", "64,64"])
@pytest.mark.parametrize("storage", sorted(KM_STORAGE))
@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8", "fp8", "bf8", "fp8_bf8"])
def test_gemm_k_major_operands_exact(rock, oracle, gpu, t, storage, tile):
    tA, tB = KM_STORAGE[storage]
    for G, M, N, K in KM_SHAPES:
        if storage == "tn":
            K -= 3   # both operands K-major: any K, the tail rows are zero-filled
        info = {}
        out, od, ref = _run_case(rock, oracle, gpu, t, G, M, N, K, tA, tB, False, True, 11,
                                 perf_config="v2:%s,8,64,16,8,1,1,1" % tile, info=info)
        assert info["kernel_name"] == "rock_gemm_%s_%s_fast_%s" % (t, tile.replace(",", "x"), storage)
        if t == "i8":
            assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0, (G, M, N, K)
        else:  # exact sums; only the narrowing to the output type rounds
            assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od])), (G, M, N, K)


def test_gemm_k_major_real_values_with_epilogue(rock, oracle, gpu):
    """Default reference layout (no transposes), real-valued f16 data, scale +
    bias + ReLU into f32: the reference's RMS gate."""
    info = {}
    bias = torch.linspace(-1.0, 1.0, 320, device=gpu)
    out, od, ref = _run_case(rock, oracle, gpu, "f16", 1, 384, 320, 512, False, False, False, False, 13,
                             out_dtype="f32", scale=0.5, bias=bias, relu=True, info=info)
    assert info["kernel_name"].endswith("_fast_nn")
    want = np.maximum(ref.reshape(384, 320) * 0.5 + bias.cpu().numpy()[None, :], 0.0)
    check_float(to_f32(out, od), want.ravel(), od)


# (G, M, N, K, transA, transB): odd K (PrGemm.toml's -k 769), N = 60 under the default
# [K, N] storage, an unaligned M of a K-major A; one or both operands need a padded copy
RAGGED = [(3, 100, 136, 769, False, True), (1, 64, 60, 64, False, False), (2, 50, 64, 72, True, True),
          (1, 130, 60, 300, True, False), (1, 257, 129, 1025, False, True)]


@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8", "fp8", "bf8"])
@pytest.mark.parametrize("G,M,N,K,tA,tB", RAGGED)
def test_gemm_ragged_operands_run_on_vector_kernels(rock, oracle, gpu, t, G, M, N, K, tA, tB):
    info = {}
    out, od, ref = _run_case(rock, oracle, gpu, t, G, M, N, K, tA, tB, False, True, 19, info=info)
    # a vector kernel (tiled, or the K split over a block's waves), behind as many copies as
    # operands needed one (none where a row happens to be whole chunks for this element size)
    assert "_generic" not in info["kernel_name"] and len(info["kernels"]) in (1, 2), info
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:  # exact sums; only the narrowing to the output type rounds
        assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od]))


def test_gemm_ragged_with_bias_residual_and_real_values(rock, oracle, gpu):
    """The padded-copy plan keeps the epilogue's pointers in place: bias
    vector, residual tensor, ReLU; real-valued f16 data to the RMS gate."""
    G, M, N, K = 1, 200, 60, 769
    rng = np.random.default_rng(23)
    bias = torch.from_numpy(rng.uniform(-1, 1, N).astype(np.float32)).to(gpu)
    res_raw, res_q = quantise(rng.uniform(-1, 1, (G, M, N)).astype(np.float32), "f16")
    info = {}
    out, od, ref = _run_case(rock, oracle, gpu, "f16", G, M, N, K, False, True, False, False, 21,
                             bias=bias, residual=to_gpu(res_raw, "f16", gpu).reshape(G, M, N), relu=True, info=info)
    assert "_generic" not in info["kernel_name"] and len(info["kernels"]) == 2
    want = np.maximum(ref.reshape(M, N) + bias.cpu().numpy()[None, :] + res_q.reshape(M, N), 0.0)
    check_float(to_f32(out, od), want.ravel(), od)


SHAPES = [
    (1, 1, 1, 1), (1, 16, 16, 16), (1, 64, 64, 128), (1, 65, 63, 129), (3, 128, 96, 200),
    (1, 256, 256, 512), (1, 300, 520, 272), (2, 512, 128, 64), (1, 1000, 24, 48),
]


@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8", "fp8", "bf8"])
@pytest.mark.parametrize("G,M,N,K", SHAPES)
def test_gemm_nt_shapes_exact(rock, oracle, gpu, t, G, M, N, K):
    """A[M,K] x B[N,K]^T (the BASELINE layout); K-contiguous rows take the
    vector-load kernels whenever K*elemsize is a multiple of 16."""
    out, od, ref = _run_case(rock, oracle, gpu, t, G, M, N, K, False, True, False, True, 7)
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        assert np.array_equal(to_f32(out, od), ref)


@pytest.mark.parametrize("tile", ["256,256", "256,128", "128,128", "64,64"])
@pytest.mark.parametrize("t", ["f16", "i8", "fp8", "f32"])
def test_gemm_every_tile_variant(rock, oracle, gpu, t, tile):
    out, od, ref = _run_case(rock, oracle, gpu, t, 1, 520, 390, 384, False, True, False, True, 9,
                             perf_config="v2:%s,8,64,16,8,1,1,1" % tile)
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        assert np.array_equal(to_f32(out, od), ref)


@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8", "fp8", "bf8"])
@pytest.mark.parametrize("G,M,N,K", [(2, 96, 70, 1040), (1, 33, 31, 4096), (1, 512, 512, 512)])
def test_gemm_split_k_over_waves(rock, oracle, gpu, t, G, M, N, K):
    """Few output tiles and a long K: 32x32 tile per block, K divided over the
    block's waves and summed through LDS (ragged M, N and K tail included)."""
    out, od, ref = _run_case(rock, oracle, gpu, t, G, M, N, K, False, True, False, True, 15,
                             perf_config="v2:32,32,4,32,32,16,4,1,1")
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:  # exact f32 sums, one rounding to the output type
        assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od]))


@pytest.mark.parametrize("t", FLOAT_TYPES)
def test_gemm_real_values_within_reference_gate(rock, oracle, gpu, t):
    out, od, ref = _run_case(rock, oracle, gpu, t, 2, 200, 136, 512, False, True, False, False, 11)
    check_float(to_f32(out, od), ref, od)


def test_gemm_odd_k_padded(rock, oracle, gpu):
    # PrGemm.toml:31-52 style: -g 3 -m 1024 -k 769 -n 1024, scaled down in M/N
    out, od, ref = _run_case(rock, oracle, gpu, "f16", 3, 256, 192, 769, False, True, False, False, 13)
    check_float(to_f32(out, od), ref, od)


# ---- epilogue -------------------------------------------------------------------
def test_quantised_gemm_i8_to_f16_bit_exact(rock, oracle, gpu):
    """BASELINE config 2 in miniature: i32 accumulators exact, then
    f16(rne(float(acc) * scale)) -- every step is a single IEEE operation, so
    the f16 result must equal the oracle's bit for bit."""
    G, M, N, K = 1, 384, 256, 512
    out, od, ref = _run_case(rock, oracle, gpu, "i8", G, M, N, K, False, True, False, True, 21,
                             out_dtype="f16", scale=0.01)
    want = oracle.round_through(oracle.dequantize(ref, 0.01, 0), CODE["f16"])
    assert np.array_equal(to_f32(out, "f16"), want)


def test_quantised_gemm_zero_point_and_f32_out(rock, oracle, gpu):
    out, od, ref = _run_case(rock, oracle, gpu, "i8", 1, 100, 60, 200, False, True, False, True, 22,
                             out_dtype="f32", scale=0.125, zero_point=-37)
    assert np.array_equal(to_f32(out, "f32"), oracle.dequantize(ref, 0.125, -37))


def test_gemm_bias_relu_requantise_to_i8(rock, oracle, gpu):
    """dequantize -> +bias -> relu -> quantize back to int8
    (tosa-to-rock-quantization.e2e.mlir chain)."""
    G, M, N, K = 1, 96, 80, 64
    rng = np.random.default_rng(23)
    bias = rng.integers(-50, 50, N).astype(np.float32)
    out, od, ref = _run_case(rock, oracle, gpu, "i8", G, M, N, K, False, True, False, True, 23,
                             out_dtype="i8", scale=0.001, bias=torch.from_numpy(bias).to(gpu), relu=True,
                             quant_scale=0.5, out_zero_point=-3)
    x = oracle.scale_bias(oracle.dequantize(ref, 0.001, 0).reshape(M, N), M, N, 1.0, bias)
    x = np.maximum(x, 0.0)
    want = oracle.quantize_i8(x, 0.5, -3)
    assert np.array_equal(out.cpu().numpy().ravel(), want.ravel())


def test_gemm_i32_bias(rock, oracle, gpu):
    rng = np.random.default_rng(24)
    bias = rng.integers(-1000, 1000, 48).astype(np.int32)
    out, od, ref = _run_case(rock, oracle, gpu, "i8", 1, 40, 48, 64, False, True, False, True, 24,
                             bias=torch.from_numpy(bias).to(gpu))
    assert np.array_equal(out.cpu().numpy().reshape(40, 48), ref.reshape(40, 48) + bias)


def test_fp8_gemm_rescaled_by_both_scales(rock, oracle, gpu):
    """BASELINE config 4 in miniature: normal(0,1) quantised with amax/448,
    f32 result multiplied by sa*sb."""
    M = N = K = 512
    rng = np.random.default_rng(25)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    sa, sb = np.float32(np.abs(A).max() / 448), np.float32(np.abs(B).max() / 448)
    rawA, Aq = quantise(A / sa, "fp8")
    rawB, Bq = quantise(B / sb, "fp8")
    s = float(np.float32(sa * sb))
    out = rock.gemm(to_gpu(rawA, "fp8", gpu), to_gpu(rawB, "fp8", gpu), transB=True, scale=s)
    ref = oracle.scale_bias(oracle.gemm(Aq, Bq, 1, M, N, K, transB=True), M, N, s)
    res = check_float(to_f32(out, "f32"), ref, "f32")
    # and the quantised product is close to the unquantised one (sanity of the scales)
    exact = (A.astype(np.float64) @ B.astype(np.float64).T).ravel()
    assert np.abs(to_f32(out, "f32") - exact).max() < 0.08 * np.abs(exact).max()


@pytest.mark.parametrize("od", ["f16", "bf16", "fp8", "bf8"])
def test_float_output_casts(rock, oracle, gpu, od):
    out, _, ref = _run_case(rock, oracle, gpu, "f16", 1, 64, 48, 64, False, True, False, True, 26,
                            out_dtype=od, scale=0.25)
    want = oracle.round_through(oracle.scale_bias(ref, 64, 48, 0.25), CODE[od])
    assert np.array_equal(to_f32(out, od), want)


def test_fp8_output_saturates(rock, oracle, gpu):
    out, _, ref = _run_case(rock, oracle, gpu, "f16", 1, 32, 32, 256, False, True, False, True, 27,
                            out_dtype="fp8", scale=100.0)
    want = oracle.round_through(oracle.scale_bias(ref, 32, 32, 100.0), CODE["fp8"])
    got = to_f32(out, "fp8")
    assert np.abs(ref * 100).max() > 448 and np.abs(got).max() == 448.0
    assert np.array_equal(got, want)


def test_mfma_rate_probe(rock, gpu):
    """The issue-rate probe runs and reports something physically sensible:
    positive, not above the published dense peak by more than clock headroom,
    and not faster on random operands than on constants."""
    peak = {"i8": 5000.0, "fp8": 5000.0, "f16": 2500.0, "bf16": 2500.0, "f32": 157.3}
    for dt, pk in peak.items():
        const = rock.mfma_rate(dt, False)
        rnd = rock.mfma_rate(dt, True)
        assert 0.2 * pk < const < 1.1 * pk, (dt, const)
        assert 0.2 * pk < rnd <= const * 1.05, (dt, rnd, const)


@pytest.mark.parametrize("t,od", [("f16", "f16"), ("bf16", "f32"), ("f32", "f32"), ("fp8", "f32")])
@pytest.mark.parametrize("tA,tB", [(False, False), (True, False), (True, True)])
def test_gemm_split_over_blocks_exact(rock, oracle, gpu, t, od, tA, tB):
    """Few output tiles, long K, K-major storage: the reduction is cut into batch
    entries whose f32 partial results the reduction kernel adds (two kernels)."""
    G, M, N, K = 1, 128, 192, 8192
    info = {}
    out, od_, ref = _run_case(rock, oracle, gpu, t, G, M, N, K, tA, tB, False, True, 17, out_dtype=od, info=info)
    assert info["kernels"][1] == "rock_reduce_splits" and "_fast_" in info["kernels"][0]
    assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od]))
    # the split can be declined
    info = {}
    out, _, _ = _run_case(rock, oracle, gpu, t, G, M, N, K, tA, tB, False, True, 17, out_dtype=od, info=info,
                          split_k=False)
    assert len(info["kernels"]) == 1
    assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od]))


# Transposed C with rows of whole 16-byte chunks leaves the tiled kernels as
# 16-byte vectors of consecutive m (the path NCHW-style convolution outputs
# take as well): every output element size, every tile, a batch, ragged N.
@pytest.mark.parametrize("tile", ["256,256", "128,128", "64,64"])
@pytest.mark.parametrize("t,od", [("f16", "f16"), ("f16", "f32"), ("bf16", "bf16"), ("f16", "fp8"), ("f16", "bf8"),
                                  ("i8", "i32"), ("i8", "f16"), ("f32", "f32")])
def test_gemm_transposed_output_vector_store_exact(rock, oracle, gpu, t, od, tile):
    G, M, N, K = 2, 304, 88, 96
    info = {}
    epi = dict(scale=0.25) if od != "i32" else {}
    out, _, ref = _run_case(rock, oracle, gpu, t, G, M, N, K, False, True, True, True, 131, out_dtype=od,
                            perf_config="v2:%s,8,64,16,8,1,1,1" % tile, info=info, **epi)
    assert "_fast" in info["kernel_name"] and tile.replace(",", "x") in info["kernel_name"]
    if od == "i32":
        assert np.array_equal(out.cpu().numpy().ravel(), ref.ravel())
    else:
        want = oracle.round_through(np.asarray(ref, np.float32) * np.float32(0.25), CODE[od])
        assert np.array_equal(to_f32(out, od), want)


def test_gemm_transposed_output_requantised_to_i8(rock, oracle, gpu):
    G, M, N, K = 1, 128, 80, 64
    out, od, ref = _run_case(rock, oracle, gpu, "i8", G, M, N, K, False, True, True, True, 133, out_dtype="i8",
                             scale=0.001, quant_scale=0.5, out_zero_point=-3)
    want = oracle.quantize_i8(oracle.dequantize(ref, 0.001, 0), 0.5, -3)
    assert np.array_equal(out.cpu().numpy().ravel(), want.ravel())
