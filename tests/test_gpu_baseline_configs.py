"""The five BASELINE.json configurations at full size on the GPU.

The CPU oracle checks bounded samples (whole rows / output ranges, always
including tile-boundary rows); size-independent properties check the rest:
row sums of the full int8 product in exact integer arithmetic, row sums of the
fp8 product in float64, rows of the softmax summing to one.  The two large
floating-point configurations are, besides, compared element by element with
torch's own f32 computation on the same inputs -- a second opinion over the
rows the oracle's samples do not reach, under the same gates."""
import numpy as np
import pytest
import torch

from tests.gpu_util import CODE, check_float, quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu


def _row_ranges(M, tile=256, width=4, extra=0, seed=0):
    """a few whole rows at the start, around tile boundaries and at the end, and `extra` more ranges drawn at
    random (seeded) over the whole matrix"""
    picks = [0, tile - width // 2, M // 2 - width // 2, M - tile - width // 2, M - width]
    picks += [int(p) for p in np.random.default_rng(seed).integers(0, M - width, extra)]
    return [(max(0, p), min(M, max(0, p) + width)) for p in picks]


def test_c1_f32_gemm_512(rock, oracle, gpu):
    """f32 GEMM C = A * B^T, M=N=K=512, uniform[-1,1); RMS <= 3e-5."""
    rng = np.random.default_rng(1)
    A = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    B = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    out = rock.gemm(torch.from_numpy(A).to(gpu), torch.from_numpy(B).to(gpu), transB=True)
    ref = oracle.gemm(A, B, 1, 512, 512, 512, transB=True)
    res = check_float(to_f32(out, "f32"), ref, "f32", rms=3e-5)
    assert res.max_abs_diff < 1e-4


def test_c2_int8_gemm_4096_quantised(rock, oracle, gpu):
    """int8 4096^3: int32 accumulators bit-exact; f16(acc * 0.01) bit-exact."""
    M = N = K = 4096
    rng = np.random.default_rng(2)
    A = rng.integers(-128, 128, (M, K), dtype=np.int8)
    B = rng.integers(-128, 128, (N, K), dtype=np.int8)
    dA, dB = torch.from_numpy(A).to(gpu), torch.from_numpy(B).to(gpu)
    acc = rock.gemm(dA, dB, transB=True)                          # i32 out
    f16 = rock.gemm(dA, dB, transB=True, out_dtype="f16", scale=0.01)
    torch.cuda.synchronize()
    acc_h = acc.cpu().numpy()
    f16_h = to_f32(f16, "f16").reshape(M, N)
    for r0, r1 in _row_ranges(M, 256, 8):
        ref = oracle.gemm(A, B, 1, M, N, K, transB=True, rows=(r0, r1)).reshape(M, N)[r0:r1]
        fails, ovf, _ = oracle.verify_int(acc_h[r0:r1], ref)
        assert (fails, ovf) == (0, 0)
        want = oracle.round_through(oracle.dequantize(ref, 0.01, 0), CODE["f16"])
        assert np.array_equal(f16_h[r0:r1], want)
    # every element: exact row and column sums of the whole accumulator matrix
    A64, B64 = A.astype(np.int64), B.astype(np.int64)
    assert np.array_equal(acc_h.astype(np.int64).sum(axis=1), A64 @ B64.sum(axis=0))
    assert np.array_equal(acc_h.astype(np.int64).sum(axis=0), B64 @ A64.sum(axis=0))
    # the f16 output is the same function of the accumulators everywhere
    full = oracle.round_through(oracle.dequantize(acc_h.astype(np.int64), 0.01, 0), CODE["f16"])
    assert np.array_equal(f16_h, full.reshape(M, N))


def test_c3_f16_conv_resnet(rock, oracle, gpu):
    """f16 NHWC conv N=256 28x28 C=128 K=128 3x3 s1 p1; RMS <= 1e-3."""
    n, c, k, hw = 256, 128, 128, 28
    rng = np.random.default_rng(3)
    raw_i, iq = quantise((rng.standard_normal(n * hw * hw * c) * 0.1).astype(np.float32), "f16")
    raw_f, fq = quantise((rng.standard_normal(k * 9 * c) * 0.1).astype(np.float32), "f16")
    out = rock.conv2d(to_gpu(raw_f, "f16", gpu), to_gpu(raw_i, "f16", gpu), fil_layout="gkyxc",
                      in_layout="nhwgc", out_layout="nhwgk", batchsize=n, in_channels=c, out_channels=k,
                      in_h=hw, in_w=hw, fil_h=3, fil_w=3, padding=(1, 1))
    got = to_f32(out, "f16")
    total = n * hw * hw * k
    span = 28 * 128 * 3          # three output image rows: includes padded borders
    starts = [0, 256 * 128 - span // 2, total // 3, total // 2 + 12345 * 128, total - span]
    for s in starts:
        ref, _, _ = oracle.conv_fwd(fq, iq, "gkyxc", "nhwgc", "nhwgk", n, 1, c, k, hw, hw, 3, 3,
                                    pad=(1, 1), out_range=(s, s + span))
        check_float(got[s:s + span], ref[s:s + span], "f16", rms=1e-3)
    assert np.isfinite(got).all()
    # linearity in the filter: conv(2*w) == 2*conv(w) exactly in binary floating point
    raw_f2, _ = quantise(fq * 2.0, "f16")
    out2 = rock.conv2d(to_gpu(raw_f2, "f16", gpu), to_gpu(raw_i, "f16", gpu), fil_layout="gkyxc",
                       in_layout="nhwgc", out_layout="nhwgk", batchsize=n, in_channels=c, out_channels=k,
                       in_h=hw, in_w=hw, fil_h=3, fil_w=3, padding=(1, 1))
    got2 = to_f32(out2, "f16")
    normal = np.abs(got) >= 2.0 ** -13           # doubling is exact unless f16 goes subnormal
    assert np.array_equal(got2[normal], 2.0 * got[normal])
    assert np.abs(got2[~normal] - 2.0 * got[~normal]).max() <= 2.0 ** -23


def test_c4_fp8_gemm_8192(rock, oracle, gpu):
    """fp8 e4m3fn 8192^3, per-tensor scales amax/448, f32 out * sa*sb; RMS <= 3e-5
    against the f32-accumulated oracle on the same quantised inputs."""
    M = N = K = 8192
    rng = np.random.default_rng(4)
    A = rng.standard_normal((M, K), dtype=np.float32)
    B = rng.standard_normal((N, K), dtype=np.float32)
    sa, sb = np.float32(np.abs(A).max() / 448), np.float32(np.abs(B).max() / 448)
    rawA, Aq = quantise(A / sa, "fp8")
    rawB, Bq = quantise(B / sb, "fp8")
    del A, B
    s = float(np.float32(sa * sb))
    out = rock.gemm(to_gpu(rawA, "fp8", gpu), to_gpu(rawB, "fp8", gpu), transB=True, scale=s)
    got = to_f32(out, "f32").reshape(M, N)
    for r0, r1 in _row_ranges(M, 256, 4, extra=27, seed=40):      # 128 of the 8192 rows
        ref = oracle.gemm(Aq, Bq, 1, M, N, K, transB=True, rows=(r0, r1)).reshape(M, N)[r0:r1]
        check_float(got[r0:r1], oracle.scale_bias(ref, r1 - r0, N, s), "f32", rms=3e-5)
    # every element against torch's f32 product of the same quantised values (in two halves: 2 x 128 MiB)
    dAq, dBq = torch.from_numpy(Aq).to(gpu), torch.from_numpy(Bq).to(gpu)
    for half in range(2):
        rows = slice(half * M // 2, (half + 1) * M // 2)
        second = (dAq[rows] @ dBq.T) * s
        diff = (out.reshape(M, N)[rows] - second).double()
        rms = float(diff.pow(2).mean().sqrt() / (second.abs().max() * 1.0))
        assert rms <= 3e-5, rms
        del second, diff
    # every element: row sums in float64 (sum_n C[m,n] = s * A[m,:] . sum_n B[n,:])
    want = (Aq.astype(np.float64) @ Bq.astype(np.float64).sum(axis=0)) * s
    rows = got.astype(np.float64).sum(axis=1)
    assert np.abs(rows - want).max() <= 2e-4 * np.abs(got).max() * np.sqrt(N)


def test_c5_f16_attention_2048(rock, oracle, gpu):
    """softmax(Q K^T / sqrt(128)) V, f16 [4,32,2048,128]; RMS <= 1e-3, max-abs <= 0.02."""
    G, S, D = 128, 2048, 128
    rng = np.random.default_rng(5)
    rq, Qq = quantise(rng.standard_normal((G, S, D), dtype=np.float32), "f16")
    rk, Kq = quantise(rng.standard_normal((G, S, D), dtype=np.float32), "f16")
    rv, Vq = quantise(rng.standard_normal((G, S, D), dtype=np.float32), "f16")
    scale = 1.0 / np.sqrt(128.0)
    dQ, dK, dV = (to_gpu(x, "f16", gpu) for x in (rq, rk, rv))
    out = rock.attention(dQ, dK, dV, scale=scale, transK=True)
    got = to_f32(out, "f16").reshape(G, S, D)
    # block starts, boundaries, the tail, and a dozen seeded positions: 64 of the 2048 query rows of every head
    starts = [0, 126, 1023, 2044] + [int(x) for x in np.random.default_rng(50).integers(0, S - 4, 12)]
    for q0 in starts:
        ref = oracle.attention(Qq, Kq, Vq, G, S, S, D, D, scale=scale, transK=True,
                               q_rows=(q0, q0 + 4)).reshape(G, S, D)[:, q0:q0 + 4]
        check_float(got[:, q0:q0 + 4].ravel(), ref.ravel(), "f16", rms=1e-3, max_abs=0.02)
    assert np.isfinite(got).all()
    # every element against torch's f32 softmax attention on the same f16 values, sixteen heads at a time
    for g0 in range(0, G, 16):
        q32, k32, v32 = (x[g0:g0 + 16].float() for x in (dQ, dK, dV))
        second = torch.softmax((q32 @ k32.transpose(1, 2)) * scale, dim=-1) @ v32
        diff = (out.reshape(G, S, D)[g0:g0 + 16].float() - second.half().float())
        assert float(diff.abs().max()) <= 0.02
        assert float(diff.double().pow(2).mean().sqrt() / second.abs().max()) <= 1e-3
        del second, diff
    # rows of P sum to one: V = ones gives ones everywhere
    ones = torch.ones_like(dV)
    got1 = to_f32(rock.attention(dQ, dK, ones, scale=scale, transK=True), "f16")
    assert np.abs(got1 - 1.0).max() <= 2e-3
