"""GPU: the in-process tuner (the loop of rocmlir-tuning-driver.cpp:234-397)
times every kernel of a problem's tuning space, leaves the fastest applied,
and every candidate computes the same, oracle-exact result."""
import numpy as np
import pytest
import torch

from tests.gpu_util import quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu


def test_tuner_gemm_every_candidate_exact_and_best_applied(rock, oracle, gpu):
    from rocmlir_amd import tuning
    M, N, K = 384, 384, 1536   # 144 tiles of 32x32: the K-split kernel alone fills the chip, one kernel
    rng = np.random.default_rng(51)
    ra, aq = quantise(rng.integers(-3, 4, (M, K)).astype(np.float32), "f16")
    rb, bq = quantise(rng.integers(-3, 4, (N, K)).astype(np.float32), "f16")
    ref = oracle.gemm(aq, bq, 1, M, N, K, transB=True).reshape(M, N)
    A, B = to_gpu(ra, "f16", gpu), to_gpu(rb, "f16", gpu)
    out = torch.zeros(M * N, dtype=torch.float32, device=gpu)
    kern = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -out_datatype f32 -g 1 -m %d -n %d -k %d "
                           "-transB true" % (M, N, K))
    names = set()
    for perf in kern.tuning_space():
        kern.set_perf_config(perf)
        names.add(kern.kernel_name)
        out.zero_()
        kern.launch(A, B, out, None)
        torch.cuda.synchronize()
        assert np.array_equal(to_f32(out, "f32").reshape(M, N), ref), kern.kernel_name
    assert len(names) == 5
    table = tuning.TuningTable()
    results = tuning.tune(kern, A, B, out, None, table=table, warmup=3, iters=10)
    assert [r[2] for r in results] == sorted(r[2] for r in results) and results[0][2] > 0
    assert kern.perf_config == results[0][0] and kern.kernel_name == results[0][1]
    assert table.entries() == {kern.problem_key: (results[0][0], pytest.approx(results[0][2]))}
    fresh = rock.RockKernel(kern.options)
    assert table.apply(fresh) and fresh.kernel_name == results[0][1]


def test_tuner_conv_includes_the_window_resident_kernel(rock, oracle, gpu):
    from rocmlir_amd import tuning
    n, c, k, hw = 6, 64, 64, 14
    rng = np.random.default_rng(53)
    fil = rng.integers(-2, 3, (k, 3, 3, c)).astype(np.float32)       # gkyxc with g = 1
    inp = rng.integers(-2, 3, (n, hw, hw, c)).astype(np.float32)     # nhwgc
    rf, fq = quantise(fil.ravel(), "f16")
    ri, iq = quantise(inp.ravel(), "f16")
    ref, ho, wo = oracle.conv_fwd(fq, iq, "gkyxc", "nhwgc", "nhwgk", n, 1, c, k, hw, hw, 3, 3, (1, 1), (1, 1),
                                  (1, 1))
    F, I = to_gpu(rf, "f16", gpu), to_gpu(ri, "f16", gpu)
    out = torch.zeros(n * ho * wo * k, dtype=torch.float16, device=gpu)
    kern = rock.RockProgram(   # the window-resident kernel comes with a filter conversion in front of it
        "--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 --fil_layout gkyxc "
        "--in_layout nhwgc --out_layout nhwgk --batchsize %d --groupsize 1 --in_channels %d --out_channels %d "
        "--in_h %d --in_w %d --fil_h 3 --fil_w 3 --dilation_h 1 --dilation_w 1 --conv_stride_h 1 "
        "--conv_stride_w 1 --padding_h 1 --padding_w 1" % (n, c, k, hw, hw))
    results = tuning.tune(kern, F, I, out, None, warmup=3, iters=10)
    assert any(name.endswith("_direct224") for _, name, _ in results)
    for perf, name, _ in results:
        kern.set_perf_config(perf)
        out.zero_()
        kern.launch(F, I, out, None)
        torch.cuda.synchronize()
        assert np.array_equal(to_f32(out, "f16"), ref), name


def test_tuner_attention_candidates_agree_and_best_applied(rock, oracle, gpu):
    """The attention tuning space (attn:v1 strings: head-dimension tile 64 / 128,
    plain / bias-capable / element-wise kernel): every candidate passes the
    attention gate against the oracle, the fastest is left applied and goes
    into the table under the problem's key."""
    from rocmlir_amd import tuning
    from tests.gpu_util import check_float
    G, sq, sk, d = 4, 200, 333, 64
    rng = np.random.default_rng(55)
    rq, Qq = quantise(rng.standard_normal((G, sq, d)).astype(np.float32), "f16")
    rk, Kq = quantise(rng.standard_normal((G, sk, d)).astype(np.float32), "f16")
    rv, Vq = quantise(rng.standard_normal((G, sk, d)).astype(np.float32), "f16")
    scale = d ** -0.5
    ref = oracle.attention(Qq, Kq, Vq, G, sq, sk, d, d, scale=scale, transK=True)
    Q, K, V = to_gpu(rq, "f16", gpu), to_gpu(rk, "f16", gpu), to_gpu(rv, "f16", gpu)
    out = torch.zeros(G * sq * d, dtype=torch.float16, device=gpu)
    kern = rock.RockKernel("-operation attention -arch gfx950 -t f16 -g %d -seq_len_q %d -seq_len_k %d -head_dim_qk %d "
                           "-head_dim_v %d -transK true -scale %.9g" % (G, sq, sk, d, d, scale))
    space = kern.tuning_space()
    assert len(space) >= 3 and all(p.startswith("attn:v1:") for p in space)
    names = set()
    for perf in space:
        kern.set_perf_config(perf)
        names.add(kern.kernel_name)
        out.zero_()
        kern.launch(Q, K, V, None, out)
        torch.cuda.synchronize()
        check_float(to_f32(out, "f16"), ref, "f16", rms=1e-3, max_abs=0.02)
    assert len(names) == len(space) and {"rock_attention_f16_d64x64_fast", "rock_attention_f16_d128x128_fast"} <= names
    table = tuning.TuningTable()
    results = tuning.tune(kern, Q, K, V, None, out, table=table, warmup=3, iters=10)
    assert kern.perf_config == results[0][0] and kern.kernel_name == results[0][1]
    fresh = rock.RockKernel(kern.options)
    assert table.apply(fresh) and fresh.kernel_name == results[0][1]
