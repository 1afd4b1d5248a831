"""GPU parity: fused attention through the C ABI vs the f32 CPU oracle.

Gates: the oracle is rounded through the 16-bit output type, then relative
RMS <= 1e-3 and max-abs <= 0.02 (the reference's f16 attention tolerances are
RMS 0.015 / abs 0.02 / rel 0.02, PrAttentionF16.toml:3; bf16 keeps only 8
mantissa bits, so its gate is RMS 8e-3 / abs 0.06)."""
import numpy as np
import pytest
import torch

from tests.gpu_util import check_float, quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu
GATE = {"f16": (1e-3, 0.02), "bf16": (8e-3, 0.06)}


def _store(mat, trans):
    return np.ascontiguousarray(mat.transpose(0, 2, 1) if trans else mat)


def _run(rock, oracle, gpu, t, G, sq, sk, dqk, dv, scale, seed, tQ=False, tK=True, tV=False, tO=False,
         bias=False, vones=False, scale_tensor=False, info=None, mask=False, limit=None, conversion=True):
    rng = np.random.default_rng(seed)
    Q = rng.standard_normal((G, sq, dqk)).astype(np.float32)
    K = rng.standard_normal((G, sk, dqk)).astype(np.float32)
    V = np.ones((G, sk, dv), np.float32) if vones else rng.standard_normal((G, sk, dv)).astype(np.float32)
    rq, Qq = quantise(_store(Q, tQ), t)
    rk, Kq = quantise(_store(K, not tK), t)     # default storage is [G,d,seq_k]
    rv, Vq = quantise(_store(V, tV), t)
    bq = braw = None
    if bias:
        braw, bq = quantise(rng.standard_normal((G, sq, sk)).astype(np.float32), t)
    sq_ = sraw = None
    if scale_tensor:
        sraw, sq_ = quantise(rng.uniform(-1.5, 1.5, (G, sq, sk)).astype(np.float32), t)
    mk = oraw = oq = None
    if mask:  # about a third of the scores replaced; some rows wholly (row 0 of every g), some not at all (row 1)
        mk = (rng.uniform(0, 1, (G, sq, sk)) > 0.35).astype(np.int8)
        mk[:, 0, :] = 0
        if sq > 1:
            mk[:, 1, :] = 1
        oraw, oq = quantise(rng.uniform(-6.0, 1.0, (G, sq, sk)).astype(np.float32), t)
    out = rock.attention(to_gpu(rq, t, gpu), to_gpu(rk, t, gpu), to_gpu(rv, t, gpu), scale=scale,
                         bias=to_gpu(braw, t, gpu) if bias else None,
                         scale_tensor=to_gpu(sraw, t, gpu) if scale_tensor else None,
                         mask=torch.from_numpy(mk).to(gpu) if mask else None,
                         other=to_gpu(oraw, t, gpu) if mask else None,
                         transQ=tQ, transK=tK, transV=tV, transO=tO, info=info, score_workspace_limit=limit,
                         layout_conversion=conversion)
    torch.cuda.synchronize()
    ref = oracle.attention(Qq, Kq, Vq, G, sq, sk, dqk, dv, scale=scale, bias_t=bq, scale_t=sq_,
                           transQ=tQ, transK=tK, transV=tV, transO=tO, mask=mk, other=oq)
    return to_f32(out, t), ref


def _run_i8(rock, oracle, gpu, G, sq, sk, dqk, dv, bias=False, info=None, limit=None):
    """int8 Q and K, f16 V: the GPU result and the oracle's, which gets the same scores through a bias that
    carries -zero_point * scale."""
    rng = np.random.default_rng(57)
    Q = rng.integers(-128, 128, (G, sq, dqk)).astype(np.int8)
    K = rng.integers(-128, 128, (G, sk, dqk)).astype(np.int8)
    V = rng.standard_normal((G, sk, dv)).astype(np.float32)
    rv, Vq = quantise(V, "f16")
    zp, scale = 37, float(np.float16(3.0e-4))
    braw = bq = None
    if bias:
        braw, bq = quantise(rng.standard_normal((G, sq, sk)).astype(np.float32), "f16")
    out = rock.attention(torch.from_numpy(Q).to(gpu), torch.from_numpy(K).to(gpu), to_gpu(rv, "f16", gpu),
                         scale=scale, zero_point=zp, bias=to_gpu(braw, "f16", gpu) if bias else None, transK=True,
                         info=info, score_workspace_limit=limit)
    torch.cuda.synchronize()
    shift = np.full((G, sq, sk), -zp * scale, np.float32) + (bq.reshape(G, sq, sk) if bias else 0.0)
    ref = oracle.attention(Q.astype(np.float32), K.astype(np.float32), Vq, G, sq, sk, dqk, dv, scale=scale,
                           bias_t=shift.astype(np.float32), transK=True)
    return to_f32(out, "f16"), ref


# PrAttentionF16.toml:20-67 shapes (+ ragged ones)
SHAPES = [
    (1, 384, 384, 64, 64), (2, 64, 64, 64, 64), (1, 256, 256, 128, 128), (3, 128, 27, 64, 32),
    (1, 1, 1, 8, 8), (2, 100, 333, 40, 72), (1, 300, 64, 128, 64), (2, 33, 130, 16, 128),
]


@pytest.mark.parametrize("t", ["f16", "bf16"])
@pytest.mark.parametrize("G,sq,sk,dqk,dv", SHAPES)
def test_attention_shapes(rock, oracle, gpu, t, G, sq, sk, dqk, dv):
    got, ref = _run(rock, oracle, gpu, t, G, sq, sk, dqk, dv, 1.0 / np.sqrt(dqk), 41)
    check_float(got, ref, t, rms=GATE[t][0], max_abs=GATE[t][1])


@pytest.mark.parametrize("tQ,tK,tV,tO", [(0, 0, 0, 0), (1, 1, 0, 0), (0, 1, 1, 0), (0, 1, 0, 1), (1, 0, 1, 1),
                                         (1, 1, 1, 1), (0, 0, 1, 0), (1, 0, 0, 0)])
def test_attention_transposed_operands(rock, oracle, gpu, tQ, tK, tV, tO):
    """Every storage of rocmlir-gen.cpp:2149-2200 ends on a fused vector kernel: K [G, d, seq_k] on the
    "_kt" kernels, transposed Q / V / O through conversion kernels around the fused one."""
    info = {}
    got, ref = _run(rock, oracle, gpu, "f16", 2, 72, 96, 64, 64, 0.125, 43, bool(tQ), bool(tK), bool(tV), bool(tO),
                    info=info)
    fused = "rock_attention_f16_d64x64_fast" + ("" if tK else "_kt")
    assert info["kernels"] == ["rock_relayout_b2"] * (tQ + tV) + [fused] + ["rock_relayout_b2"] * tO
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])


@pytest.mark.parametrize("t", ["f16", "bf16"])
@pytest.mark.parametrize("G,sq,sk,dqk,dv,bias", [
    (1, 384, 384, 64, 64, False), (2, 64, 64, 64, 64, False), (1, 256, 256, 128, 128, False),
    (2, 100, 328, 40, 72, False), (1, 300, 72, 128, 64, True), (2, 33, 136, 16, 128, False),
    (1, 1, 8, 8, 8, False), (2, 130, 200, 192, 256, False), (1, 129, 64, 256, 136, True),
    (1, 384, 384, 64, 64, True)])
def test_attention_default_key_layout(rock, oracle, gpu, t, G, sq, sk, dqk, dv, bias):
    """K stored [G, d, seq_k], the reference's default (rocmlir-gen.cpp:2164-2165; PrAttentionF16.toml:10-13
    runs every case both ways): one fused kernel that takes its K fragments through the transposing LDS
    read; ragged tiles, head-dimension padding, head dimensions up to 256, with and without bias."""
    info = {}
    got, ref = _run(rock, oracle, gpu, t, G, sq, sk, dqk, dv, 1.0 / np.sqrt(dqk), 47, tK=False, bias=bias, info=info)
    dmax = 64 if max(dqk, dv) <= 64 else 128 if max(dqk, dv) <= 128 else 256
    assert info["kernels"] == ["rock_attention_%s_d%dx%d_fast%s_kt" % (t, dmax, dmax, "_bias" if bias or dmax == 256 else "")]
    check_float(got, ref, t, rms=GATE[t][0], max_abs=GATE[t][1])


def test_attention_default_key_layout_unaligned_rows(rock, oracle, gpu):
    """seq_k = 27 under the default storage: rows of keys are not whole 16-byte chunks, K is copied to
    [G, seq_k, d] in front of the fused kernel (cross attention case of PrAttentionF16.toml:64-67)."""
    info = {}
    got, ref = _run(rock, oracle, gpu, "f16", 2, 128, 27, 64, 32, 0.125, 48, tK=False, bias=True, scale_tensor=True,
                    info=info)
    assert info["kernels"] == ["rock_relayout_b2", "rock_attention_f16_d64x64_fast_bias"]
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])


@pytest.mark.parametrize("conversion", [True, False], ids=["padded-copies", "as-they-lie"])
def test_attention_odd_head_dims(rock, oracle, gpu, conversion):
    """Head dimensions that are not whole 16-byte chunks (20 and 12): Q, K and V are copied into rows padded with
    zeros, the fused kernel runs on the padded problem and a last copy keeps the columns of O that exist; without
    conversions the element-wise kernel reads the tensors as they lie."""
    info = {}
    got, ref = _run(rock, oracle, gpu, "f16", 2, 50, 70, 20, 12, 0.3, 44, info=info, conversion=conversion)
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])
    assert info["kernels"] == (["rock_relayout_b2"] * 3 + ["rock_attention_f16_d64x64_fast", "rock_relayout_b2"]
                               if conversion else ["rock_attention_f16_d64x64_generic"])


def test_attention_with_bias(rock, oracle, gpu):
    # cross attention with scale and bias: seq_q 128, seq_k 27, d_qk 64, d_v 32
    got, ref = _run(rock, oracle, gpu, "f16", 2, 128, 27, 64, 32, 0.125, 45, bias=True)
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("shape", [(2, 128, 27, 64, 32), (1, 300, 200, 128, 128), (2, 50, 70, 20, 12)],
                         ids=["cross", "d128", "odd-head-dims"])
def test_attention_with_scale_tensor(rock, oracle, gpu, shape, bias):
    """-with-attn-scale: a [G,seq_q,seq_k] tensor multiplied into the scores
    before the softmax (rocmlir-gen.cpp:2185-2196, 2368-2382), alone and with a bias."""
    G, sq, sk, dqk, dv = shape
    got, ref = _run(rock, oracle, gpu, "f16", G, sq, sk, dqk, dv, 0.125, 49, bias=bias, scale_tensor=True)
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])


@pytest.mark.parametrize("case", [
    # the reference's own case: 12 heads, 256 x 256 scores, head dimension 256, scale 0.125 (mixr-attn-where.mlir:4-13)
    dict(id="mixr-attn-where", t="f16", shape=(12, 256, 256, 256, 256), kernels=["rock_attention_f16_d256x256_fast_bias"]),
    dict(id="d128-ragged-bias", t="f16", shape=(2, 300, 200, 128, 128), bias=True, kernels=["rock_attention_f16_d128x128_fast_bias"]),
    dict(id="d64-scale-tensor-bf16", t="bf16", shape=(3, 128, 27, 64, 32), scale_tensor=True,
         kernels=["rock_attention_bf16_d64x64_fast_bias"]),
    dict(id="default-key-layout", t="f16", shape=(2, 130, 136, 64, 64), tK=False, kernels=["rock_attention_f16_d64x64_fast_bias_kt"]),
    dict(id="generic", t="f16", shape=(2, 50, 70, 20, 12), conversion=False, kernels=["rock_attention_f16_d64x64_generic"]),
    dict(id="odd-head-dims", t="f16", shape=(2, 50, 70, 20, 12), count=5),
    dict(id="transposed-q-o", t="f16", shape=(2, 96, 80, 64, 64), tQ=True, tO=True, count=3),
    dict(id="three-kernels-d320", t="f16", shape=(2, 100, 150, 320, 192), bias=True, count=3),
    dict(id="three-kernels-f32", t="f32", shape=(2, 96, 80, 64, 64), bias=True, scale_tensor=True, count=3),
], ids=lambda c: c["id"])
def test_attention_where_mask(rock, oracle, gpu, case):
    """migraphx.where(mask, scores, other) in front of the softmax (mixr-attn-where.mlir:11): a zero in the int8
    mask replaces the score -- after scale tensor, scale and bias -- by other's element.  Every kernel family that
    takes pre-softmax tensors, rows masked wholly and not at all."""
    t = case["t"]
    G, sq, sk, dqk, dv = case["shape"]
    info = {}
    got, ref = _run(rock, oracle, gpu, t, G, sq, sk, dqk, dv, 0.125, 71, tQ=case.get("tQ", False),
                    tK=case.get("tK", True), tO=case.get("tO", False), bias=case.get("bias", False),
                    scale_tensor=case.get("scale_tensor", False), mask=True, info=info,
                    conversion=case.get("conversion", True))
    if "kernels" in case:
        assert info["kernels"] == case["kernels"]
    else:
        assert len(info["kernels"]) == case["count"]
    gate = {"f16": GATE["f16"], "bf16": GATE["bf16"], "f32": (3e-5, 1e-4)}[t]
    check_float(got, ref, t, rms=gate[0], max_abs=gate[1])


@pytest.mark.parametrize("t", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("shape", [(2, 200, 333, 256, 256), (1, 130, 520, 512, 512), (3, 64, 100, 40, 72)],
                         ids=["d256", "d512", "small"])
def test_attention_three_kernel_form(rock, oracle, gpu, t, shape):
    """Head dimensions above 256, and every f32 problem: GEMM, row softmax, GEMM.
    The 16-bit types up to head dimension 256 run on one fused kernel."""
    G, sq, sk, dqk, dv = shape
    if t != "f32" and dqk <= 128:
        pytest.skip("the fused kernel takes this one")
    gate = {"f16": GATE["f16"], "bf16": GATE["bf16"], "f32": (3e-5, 1e-4)}[t]
    info = {}
    got, ref = _run(rock, oracle, gpu, t, G, sq, sk, dqk, dv, 1.0 / np.sqrt(dqk), 51, info=info)
    if t != "f32" and dqk <= 256:
        assert info["kernels"] == ["rock_attention_%s_d256x256_fast_bias" % t]
    else:
        assert len(info["kernels"]) == 3
    check_float(got, ref, t, rms=gate[0], max_abs=gate[1])


@pytest.mark.parametrize("shape,bias,scale_tensor", [((2, 300, 333, 192, 256), False, False),
                                                      ((1, 129, 64, 256, 136), True, False),
                                                      ((2, 64, 200, 160, 160), True, True)])
def test_attention_head_dims_up_to_256_fused(rock, oracle, gpu, shape, bias, scale_tensor):
    """Head dimensions between 129 and 256 (ragged ones, different for QK and
    V, with and without the pre-softmax tensors): one kernel, no score workspace."""
    G, sq, sk, dqk, dv = shape
    info = {}
    got, ref = _run(rock, oracle, gpu, "f16", G, sq, sk, dqk, dv, 1.0 / np.sqrt(dqk), 61, bias=bias,
                    scale_tensor=scale_tensor, info=info)
    assert info["kernels"] == ["rock_attention_f16_d256x256_fast_bias"]
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])


@pytest.mark.parametrize("case", [
    dict(id="row-chunks", t="f16", shape=(3, 200, 333, 320, 192), limit=200 << 10, kernels=18),   # 128 + 72 rows per group
    dict(id="group-chunks", t="f16", shape=(3, 200, 333, 320, 192), limit=600 << 10, kernels=6),  # 2 groups + 1
    dict(id="f32-transposed", t="f32", shape=(2, 150, 96, 64, 64), limit=40 << 10, kernels=12, tQ=True, tK=False,
         tV=True, tO=True),
    dict(id="i8-rows", t="i8", shape=(2, 300, 136, 320, 64), limit=100 << 10, kernels=18),
    # chunks of one group's rows with many keys: the second GEMM's reduction in 4 shares, a fourth kernel per chunk
    dict(id="row-chunks-split-keys", t="f16", shape=(2, 200, 2048, 320, 192), limit=1 << 20, kernels=16, tO=True),
    dict(id="whole-f32-split-keys", t="f32", shape=(1, 130, 4096, 64, 72), limit=None, kernels=4),
], ids=lambda c: c["id"])
def test_attention_three_kernel_form_in_chunks(rock, oracle, gpu, case):
    """A score matrix above the workspace bound is worked off chunk by chunk (whole groups, or query rows of one
    group), three kernels each; pre-softmax tensors and the result are addressed at the chunk's rows."""
    t = case["t"]
    G, sq, sk, dqk, dv = case["shape"]
    info = {}
    if t == "i8":
        got, ref = _run_i8(rock, oracle, gpu, G, sq, sk, dqk, dv, info=info, limit=case["limit"])
        t = "f16"
    else:
        got, ref = _run(rock, oracle, gpu, t, G, sq, sk, dqk, dv, 0.1, 57, tQ=case.get("tQ", False),
                        tK=case.get("tK", True), tV=case.get("tV", False), tO=case.get("tO", False), bias=True,
                        scale_tensor=True, mask=True, info=info, limit=case["limit"])
    assert len(info["kernels"]) == case["kernels"], info["kernels"]
    gate = {"f16": GATE["f16"], "f32": (3e-5, 1e-4)}[t]
    check_float(got, ref, t, rms=gate[0], max_abs=gate[1])


@pytest.mark.parametrize("case", [
    # the reference's two trees at their own shape (mixr-attention-padded-scale-bias-exp.mlir:5-16,
    # mixr-attention-padded-complex-tree-elemwise.mlir:5-24: f32, 7 x 7 scores, head dimension 3, K [G, d, seq_k])
    dict(id="exp-tree-7x7", t="f32", shape=(1, 7, 7, 3, 3), program="x,t0,mul,exp,t1,add", n_in=2),
    dict(id="complex-tree-7x7", t="f32", shape=(1, 7, 7, 3, 3), program="x,t0,t1,sub,mul,t2,t3,add,add", n_in=4),
    dict(id="exp-tree-f16", t="f16", shape=(3, 130, 200, 64, 72), program="x,t0,mul,exp,t1,add", n_in=2),
    dict(id="complex-tree-bf16", t="bf16", shape=(2, 100, 333, 40, 128), program="x,t0,t1,sub,mul,t2,t3,add,add", n_in=4),
    dict(id="mask-tanh-chunks", t="f16", shape=(2, 200, 136, 64, 64), program="t0,x,c:0.125,mul,tanh,c:5,mul,t1,where",
         n_in=2, mask_first=True, limit=60 << 10, kernels=12),
    dict(id="long-rows-f32", t="f32", shape=(1, 40, 4500, 32, 32), program="x,c:0.2,mul,t0,max,sigmoid,neg", n_in=1),
], ids=lambda c: c["id"])
def test_attention_pre_softmax_program(rock, oracle, gpu, case):
    """-attn_elementwise: an element-wise tree over the scores and further [G, seq_q, seq_k] tensors in front of
    the softmax (the region of rock.attention, RockOps.td:208-254), interpreted by the row softmax of the
    three-kernel form; against the numpy restatement, itself pinned by torch in float64."""
    t = case["t"]
    G, sq, sk, dqk, dv = case["shape"]
    rng = np.random.default_rng(73)
    rq, Qq = quantise(rng.standard_normal((G, sq, dqk)).astype(np.float32), t)
    rk, Kq = quantise(rng.standard_normal((G, dqk, sk)).astype(np.float32), t)      # the default storage of K
    rv, Vq = quantise(rng.standard_normal((G, sk, dv)).astype(np.float32), t)
    dev_in, ref_in = [], []
    for i in range(case["n_in"]):
        if i == 0 and case.get("mask_first"):
            m = (rng.random((G, sq, sk)) < 0.7).astype(np.int8)
            dev_in.append(torch.from_numpy(m).to(gpu))
            ref_in.append(m)
        else:
            raw, val = quantise((rng.standard_normal((G, sq, sk)) * 0.4).astype(np.float32), t)
            dev_in.append(to_gpu(raw, t, gpu).reshape(G, sq, sk))
            ref_in.append(val)
    info = {}
    out = rock.attention(to_gpu(rq, t, gpu), to_gpu(rk, t, gpu), to_gpu(rv, t, gpu), program=case["program"],
                         inputs=dev_in, info=info, score_workspace_limit=case.get("limit"))
    torch.cuda.synchronize()
    assert len(info["kernels"]) == case.get("kernels", 3) and "rock_softmax_rows" in info["kernels"]
    ref = oracle.attention_program(Qq, Kq, Vq, G, sq, sk, dqk, dv, case["program"], ref_in)
    gate = {"f16": GATE["f16"], "bf16": GATE["bf16"], "f32": (3e-5, 1e-4)}[t]
    check_float(to_f32(out, t), ref, t, rms=gate[0], max_abs=gate[1])


def test_attention_three_kernel_form_with_bias_and_scale_tensor(rock, oracle, gpu):
    got, ref = _run(rock, oracle, gpu, "f16", 2, 100, 150, 320, 192, 0.07, 53, bias=True, scale_tensor=True)
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])
    got, ref = _run(rock, oracle, gpu, "f32", 2, 96, 80, 64, 64, 0.125, 55, tQ=True, tK=False, tV=True, tO=True,
                    bias=True)
    check_float(got, ref, "f32", rms=3e-5, max_abs=1e-4)


@pytest.mark.parametrize("shape", [(1, 64, 64, 32, 32), (2, 100, 130, 64, 48), (1, 200, 77, 256, 64)],
                         ids=["mixr", "ragged", "d256"])
@pytest.mark.parametrize("bias", [False, True])
def test_attention_int8_first_gemm(rock, oracle, gpu, shape, bias):
    """-t i8 (mixr-attention-first-gemm-i8-f16.mlir): Q K^T in int8 -> int32,
    dequantised with a zero point and an f16-valued scale before the softmax,
    f16 V and output.  The oracle gets the same scores through a bias that
    carries -zero_point * scale."""
    G, sq, sk, dqk, dv = shape
    info = {}
    got, ref = _run_i8(rock, oracle, gpu, G, sq, sk, dqk, dv, bias=bias, info=info)
    if dqk <= 128:  # fused: the int32 score tile is dequantised in registers
        dmax = 64 if max(dqk, dv) <= 64 else 128
        assert info["kernels"] == ["rock_attention_i8_d%dx%d_%s" % (dmax, dmax, "fast_bias" if bias else "fast")]
    else:
        assert len(info["kernels"]) == 3
    check_float(got, ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])


def test_attention_int8_first_gemm_fused_at_size(rock, oracle, gpu):
    """Head dimension 128, several key tiles and query blocks, ragged in both:
    the fused int8 kernel against the oracle, and on K stored the other way
    round."""
    G, sq, sk, dqk, dv = 3, 300, 333, 128, 128
    rng = np.random.default_rng(59)
    Q = rng.integers(-128, 128, (G, sq, dqk)).astype(np.int8)
    K = rng.integers(-128, 128, (G, sk, dqk)).astype(np.int8)
    rv, Vq = quantise(rng.standard_normal((G, sk, dv)).astype(np.float32), "f16")
    zp, scale = -5, float(np.float16(2.0e-4))
    info, info3 = {}, {}
    q, k, v = torch.from_numpy(Q).to(gpu), torch.from_numpy(K).to(gpu), to_gpu(rv, "f16", gpu)
    out = rock.attention(q, k, v, scale=scale, zero_point=zp, transK=True, info=info)
    # K stored [G, d, seq_k] (as mixr-attention-first-gemm-i8.mlir:7 holds it): copied in front of the same kernel
    out3 = rock.attention(q, k.transpose(1, 2).contiguous(), v, scale=scale, zero_point=zp, transK=False, info=info3)
    torch.cuda.synchronize()
    assert info["kernels"] == ["rock_attention_i8_d128x128_fast"]
    assert info3["kernels"] == ["rock_relayout_b1", "rock_attention_i8_d128x128_fast"]
    assert torch.equal(out, out3)
    shift = np.full((G, sq, sk), -zp * scale, np.float32)
    ref = oracle.attention(Q.astype(np.float32), K.astype(np.float32), Vq, G, sq, sk, dqk, dv, scale=scale,
                           bias_t=shift, transK=True)
    check_float(to_f32(out, "f16"), ref, "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])
    check_float(to_f32(out, "f16"), to_f32(out3, "f16"), "f16", rms=GATE["f16"][0], max_abs=GATE["f16"][1])


def test_attention_rows_of_p_sum_to_one(rock, oracle, gpu):
    # V = ones -> O = ones exactly up to the final rounding (size-independent property)
    got, ref = _run(rock, oracle, gpu, "f16", 2, 200, 520, 128, 128, 0.0884, 46, vones=True)
    assert np.abs(got - 1.0).max() <= 2e-3


def test_attention_large_scores_do_not_overflow(rock, oracle, gpu):
    # scale 4 pushes scores to ~ +-150: exp must stay finite through the running max
    got, ref = _run(rock, oracle, gpu, "f16", 1, 64, 256, 64, 64, 4.0, 47)
    check_float(got, ref, "f16", rms=2e-3, max_abs=0.03)
