"""The kernels compiled for the CPU and run through whole plans, block by block, against the oracle
(tests/kernel_host/: the stand-in for the device environment and the runner).

What the model is: the kernels' own sources (csrc/gemm_conv_dlds.h and what it includes, relayout_kernels.hip)
built for x86, each thread of a block a cooperative fiber that runs until it meets an operation involving other
threads -- a barrier, a matrix instruction, a cross-lane or transposing read -- where the wave or the block
gathers and the operation is computed from every lane's operands.  LDS then holds what the GPU's LDS holds, every
address is the one the GPU thread forms, and on integer-valued data the results must equal the oracle's bit for
bit.  Buffer loads are range-checked like the hardware's, every tensor lies between canary pages and inaccessible
regions, and a 16-byte access that is not 16-byte aligned traps.  A load into LDS lands when it is issued or at
the wait that covers it, and the tests run under both.  What it is not: timing, caches, or the accumulation
order inside a matrix instruction (exact data only).

The plans come from the C ABI exactly as a caller gets them: kernel name, grid, block, parameter block and
pointer map per kernel id, tensor sizes from rockamdGetArgumentInfo.
"""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from tests.kernel_host.model import CLANG, build_model, harness_device, run_plan  # noqa: E402

pytestmark = pytest.mark.skipif(CLANG is None, reason="the host build uses clang's vector extensions")


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    """The f32, f16 and int8 kernel families and the attention kernels (a minute or two of compilation).  Every launch
    is also checked for bytes that two of its blocks change."""
    lib = build_model(str(tmp_path_factory.mktemp("kernel_host")), types=(0, 1, 3))
    lib.hm_set_owner_check(1)
    return lib


@pytest.fixture(params=["loads-land-at-issue", "loads-land-at-the-wait"])
def loads(request, model):
    """The two extremes of when a load into LDS may land: a kernel that reads a stage before its wait fails
    under the second, one that refills a stage that is still being read under the first.  The threads of a
    block take their turns in ascending order under the first and with the waves rotated from pass to pass
    under the second: no result may depend on which wave runs first."""
    late = request.param == "loads-land-at-the-wait"
    model.hm_set_late_loads(1 if late else 0)
    model.hm_set_thread_order(2 if late else 0)
    yield request.param
    model.hm_set_late_loads(0)
    model.hm_set_thread_order(0)


@pytest.fixture(scope="module")
def rock():
    import rocmlir_amd
    rocmlir_amd.load_library()
    return rocmlir_amd


_NUMPY = {"f32": np.float32, "f16": np.float16}


def _conv_problem(op, t, n, c, k, hi, wi, f, pad, layouts, stride=1, extra=""):
    fl, il, ol = layouts.split()
    return ("-operation %s -arch gfx950 -t %s -groupsize 1 -batchsize %d -in_channels %d -out_channels %d -in_h %d "
            "-in_w %d -fil_h %d -fil_w %d -padding_h %d -padding_w %d -conv_stride_h %d -conv_stride_w %d "
            "-fil_layout %s -in_layout %s -out_layout %s %s" % (op, t, n, c, k, hi, wi, f, f, pad, pad, stride, stride,
                                                               fl, il, ol, extra))


def run_conv(model, rock, oracle, op, t, n, c, k, hi, wi, f, pad, layouts, stride=1, extra="", seed=0):
    """One convolution on integer-valued data through the model; returns (kernel names, problems, result equals
    the oracle's)."""
    dt = _NUMPY[t]
    rng = np.random.default_rng(seed)
    ho, wo = (hi + 2 * pad - f) // stride + 1, (wi + 2 * pad - f) // stride + 1
    W = rng.integers(-2, 3, k * c * f * f).astype(dt)
    X = rng.integers(-2, 3, n * c * hi * wi).astype(dt)
    Y = rng.integers(-2, 3, n * k * ho * wo).astype(dt)
    opts = _conv_problem(op, t, n, c, k, hi, wi, f, pad, layouts, stride, extra)
    fl, il, ol = layouts.split()
    five = [fl.replace("k", "gk"), il.replace("c", "gc"), ol.replace("k", "gk")]
    args = five + [n, 1, c, k, hi, wi, f, f]
    kw = dict(stride=(stride, stride), pad=(pad, pad), dil=(1, 1))
    f32 = lambda a: a.astype(np.float32)
    if op == "conv":
        names, problems, out = run_plan(model, rock, opts, {0: W, 1: X})
        got, ref = out[2][:Y.nbytes], oracle.conv_fwd(f32(W), f32(X), *args, **kw)[0]
    elif op == "conv_bwd_data":
        names, problems, out = run_plan(model, rock, opts, {0: W, 2: Y})
        got, ref = out[1][:X.nbytes], oracle.conv_bwd_data(f32(W), f32(Y), *args, **kw)[0]
    else:
        names, problems, out = run_plan(model, rock, opts, {1: X, 2: Y})
        got, ref = out[0][:W.nbytes], oracle.conv_bwd_weight(f32(X), f32(Y), *args, **kw)[0]
    want = np.asarray(ref).ravel().astype(dt)
    return names, problems, np.array_equal(got.view(dt).astype(np.float64), want.astype(np.float64))


@pytest.fixture(scope="module")
def oracle():
    from oracle import rock_oracle
    return rock_oracle


def test_the_model_notices_a_short_tensor(model, rock):
    """The input gradient of a 1x1 convolution written 16 bytes short: the last store lands on the canary."""
    opts = _conv_problem("conv_bwd_data", "f32", 16, 32, 32, 14, 14, 1, 1, "kcyx nchw nkhw")
    names, problems, _ = run_plan(model, rock, opts)
    assert names[-1] == "rock_conv_f32_64x64_fast" and not problems, problems
    names, problems, _ = run_plan(model, rock, opts, shrink=(1, 16))
    assert problems and "beside argument 1" in problems[-1], problems


def test_the_model_notices_a_short_operand(model, rock):
    """A GEMM operand allocated one chunk short: the direct-to-LDS load of its last chunk is out of the tensor."""
    opts = "-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 128 -k 256"
    names, problems, _ = run_plan(model, rock, opts)
    assert names and not problems, (names, problems)
    names, problems, _ = run_plan(model, rock, opts, shrink=(0, 16))
    assert problems and "buffer load into LDS outside the tensors" in problems[0], problems


def test_the_model_notices_two_blocks_writing_one_byte(model, rock):
    """A GEMM whose result rows are given half their pitch in the parameter block: the right half of every row
    then lies on the left half of the next, which another block writes."""
    import ctypes as C
    import struct
    from tests.kernel_host.model import pointer_map
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f32 -g 1 -m 128 -n 128 -k 64 -transA false -transB true")
    assert k.kernel_name == "rock_gemm_f32_64x64_fast" and k.grid_size == 4
    model.hm_clear()
    rng = np.random.default_rng(0)
    tensors = []
    for i, nbytes in enumerate((128 * 64 * 4, 128 * 64 * 4, 128 * 128 * 4, 16)):
        at = model.hm_alloc(nbytes, b"argument %d" % i)
        np.ctypeslib.as_array((C.c_uint8 * nbytes).from_address(at))[:] = rng.integers(0, 256, nbytes, dtype=np.uint8) & 0x3F
        tensors.append(at)
    ptrs = (C.c_void_p * 8)()
    for j, (src, off) in enumerate(pointer_map(rock, k)):
        ptrs[j] = None if src < 0 else tensors[src] + off
    text = C.create_string_buffer(512)
    params = bytearray(k.params())
    assert model.hm_run(k.kernel_name.encode(), bytes(params), ptrs, 4, k.block_size, text, 512) == 0, text.value
    assert struct.unpack_from("<q", params, 56)[0] == 128   # the stride between rows of C
    struct.pack_into("<q", params, 56, 64)
    assert model.hm_run(k.kernel_name.encode(), bytes(params), ptrs, 4, k.block_size, text, 512) > 0
    assert b"which an earlier block of the launch had written" in text.value, text.value


@pytest.mark.parametrize("t", ["f16", "f32"])
@pytest.mark.parametrize("shape", [(128, 128, 256, False, False), (70, 45, 100, False, True), (96, 200, 64, True, False),
                                   (33, 17, 40, True, True), (300, 260, 72, False, True)],
                         ids=lambda s: "%dx%dx%d%s%s" % (s[0], s[1], s[2], "-tA" if s[3] else "", "-tB" if s[4] else ""))
def test_gemm_through_the_model_equals_numpy(model, rock, loads, t, shape):
    """K-contiguous and K-major operands (the transposing LDS reads), ragged tiles, operands copied into padded
    rows first: integer-valued data, every element equal to numpy's float64 product."""
    m, n, k, ta, tb = shape
    dt = _NUMPY[t]
    rng = np.random.default_rng(m + n)
    A = rng.integers(-3, 4, (k, m) if ta else (m, k)).astype(dt)
    B = rng.integers(-3, 4, (n, k) if tb else (k, n)).astype(dt)
    opts = "-operation gemm -arch gfx950 -t %s -g 1 -m %d -n %d -k %d -transA %s -transB %s" % (
        t, m, n, k, str(ta).lower(), str(tb).lower())
    names, problems, out = run_plan(model, rock, opts, {0: A, 1: B})
    assert not problems, (names, problems)
    got = out[2][:m * n * np.dtype(dt).itemsize].view(dt).reshape(m, n).astype(np.float64)
    want = (A.T if ta else A).astype(np.float64) @ (B.T if tb else B).astype(np.float64)
    assert np.array_equal(got, want), names


@pytest.mark.parametrize("tile", ["v2:256,256,8,128,16,16,1,1,1", ""], ids=["256x256", "table"])
def test_quantised_int8_gemm_through_the_model_equals_the_oracle(model, rock, oracle, loads, tile):
    """The headline configuration in small: int8 operands, int32 accumulators, f16(float(acc) * 0.01), on the
    256 x 256 tile it runs on at full size and on the tile the table picks for this size; every step is a single
    IEEE operation, so the result must equal the oracle's bit for bit."""
    from tests.gpu_util import CODE
    M, N, K = 512, 384, 256
    rng = np.random.default_rng(7)
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    B = rng.integers(-128, 128, (N, K)).astype(np.int8)
    opts = ("-operation gemm -arch gfx950 -t i8 -out_datatype f16 -g 1 -m %d -n %d -k %d -transA false -transB true "
            "-scale 0.01" % (M, N, K)) + (" -perf_config " + tile if tile else "")
    names, problems, out = run_plan(model, rock, opts, {0: A, 1: B})
    assert not problems, (names, problems)
    if tile:
        assert names == ["rock_gemm_i8_256x256_fast"], names
    acc = A.astype(np.int64) @ B.astype(np.int64).T
    want = oracle.round_through(oracle.dequantize(acc, 0.01, 0), CODE["f16"]).reshape(M, N)
    got = out[2][:M * N * 2].view(np.float16).reshape(M, N).astype(np.float32)
    assert np.array_equal(got, want.astype(np.float32)), names


# (operation, type, batch, c, k, image, filter, padding, layouts, stride, last kernel): the kinds of plan the
# reference's regression lists hold, at sizes the CPU runs in seconds
_PLANS = [
    ("conv_bwd_data", "f16", 1, 128, 64, 28, 3, 1, "kcyx nchw nkhw", 1, "rock_conv_f16_64x64_fast"),
    ("conv_bwd_data", "f16", 1, 64, 64, 28, 3, 1, "kyxc nhwc nhwk", 1, "rock_conv_f16_64x64_fast"),
    ("conv", "f16", 1, 64, 128, 28, 3, 1, "kcyx nchw nkhw", 1, "rock_conv_f16_64x64_fast"),
    ("conv", "f32", 2, 64, 64, 15, 3, 0, "kyxc nhwc nhwk", 1, "rock_conv_f32_64x64_fast"),
    ("conv", "f16", 2, 24, 40, 13, 3, 1, "kcyx nhwc nkhw", 2, None),   # channel runs that are not whole chunks
    ("conv_bwd_data", "f32", 2, 32, 32, 14, 1, 1, "kcyx nchw nkhw", 1, "rock_conv_f32_64x64_fast"),
    ("conv_bwd_data", "f16", 2, 64, 64, 56, 1, 0, "kyxc nhwc nhwk", 2, "rock_conv_f16_64x64_fast"),   # zero fill + one phase
    ("conv_bwd_data", "f32", 2, 64, 128, 17, 3, 1, "kcyx nchw nkhw", 2, "rock_conv_f32_64x64_fast"),  # four phases
    ("conv_bwd_weight", "f32", 2, 32, 32, 14, 1, 1, "kcyx nchw nkhw", 1, None),
    ("conv_bwd_weight", "f16", 2, 64, 64, 14, 3, 1, "kyxc nhwc nhwk", 1, "rock_conv_bwd_weight_f16_64x64"),
    ("conv_bwd_weight", "f32", 2, 64, 128, 17, 3, 1, "kyxc nhwc nhwk", 2, "rock_conv_bwd_weight_f32_128x128"),
    ("conv_bwd_weight", "f16", 2, 128, 128, 28, 1, 0, "kcyx nchw nkhw", 1, "rock_reduce_splits"),    # as a split GEMM
]


@pytest.mark.parametrize("plan", _PLANS, ids=lambda p: "%s-%s-%dx%d-%d-%s" % (p[0], p[1], p[5], p[5], p[6], p[8].split()[1]))
def test_convolution_plans_through_the_model_equal_the_oracle(model, rock, oracle, loads, plan):
    op, t, n, c, k, hw, f, pad, layouts, stride, last = plan
    names, problems, equal = run_conv(model, rock, oracle, op, t, n, c, k, hw, hw, f, pad, layouts, stride)
    assert not problems, (names, problems)
    assert last is None or names[-1] == last, names
    assert equal, names


_WINDOW = "-perf_config v2:224,128,8,224,32,8,1,1,1"


@pytest.mark.parametrize("case", [
    # pixels-last output: whole rows of channels
    (2, 128, 128, 28, 28, "kyxc nhwc nhwk"),
    # channel-major output, 7 x 28-pixel tiles would start inside a 16-byte vector of pixels: the planner takes
    # four rows per tile, whole vectors
    (2, 128, 128, 28, 28, "kyxc nhwc nkhw"),
    # no tile height gives whole vectors (windows of at most three rows of 14 pixels x 512 channels): the kernel
    # stores element by element
    (2, 512, 128, 16, 14, "kyxc nhwc nkhw"),
], ids=["rows", "pixel-vectors", "pixel-vectors-misaligned"])
def test_window_resident_kernel_through_the_model(model, rock, oracle, loads, case):
    """The window-resident kernel on request, its three ways of storing a tile."""
    n, c, k, hi, wi, layouts = case
    names, problems, equal = run_conv(model, rock, oracle, "conv", "f16", n, c, k, hi, wi, 3, 1, layouts, extra=_WINDOW)
    assert names == ["rock_relayout_b2", "rock_conv_f16_direct224"], names
    assert not problems, problems
    assert equal


def _attention_problem(t, G, sq, sk, dqk, dv, trans_k, scale, extra=""):
    return ("-operation attention -arch gfx950 -t %s -g %d -seq_len_q %d -seq_len_k %d -head_dim_qk %d -head_dim_v %d "
            "-transQ false -transK %s -transV false -transO false -scale %.9g %s"
            % (t, G, sq, sk, dqk, dv, "true" if trans_k else "false", scale, extra))


@pytest.mark.parametrize("case", [
    # (type, heads, seq_q, seq_k, d_qk, d_v, K stored [seq_k][d], scale tensor, bias, last kernel)
    ("f16", 2, 128, 96, 64, 64, True, False, False, "rock_attention_f16_d64x64_fast"),
    ("f16", 1, 160, 200, 128, 128, False, False, False, "rock_attention_f16_d128x128_fast_kt"),
    ("f16", 2, 128, 27, 64, 32, True, True, True, "rock_attention_f16_d64x64_fast_bias"),
    ("f16", 1, 64, 128, 256, 256, True, False, False, "rock_attention_f16_d256x256_fast_bias"),
    # three kernels around the row softmax; 45 and 77 keys are not whole 16-byte chunks: the scores lie in padded
    # rows and P's tail is written as zeros, which keeps the second GEMM on its vector path
    ("f32", 2, 70, 45, 64, 64, True, False, True, "rock_gemm_f32_64x64_fast_nn"),
    ("f16", 1, 40, 77, 320, 320, True, False, False, "rock_gemm_f16_64x64_fast_nn"),
    # head dimensions 20 and 12: copies padded with zeros around the fused kernel, the last one drops O's padding
    ("f16", 2, 50, 70, 20, 12, False, False, True, "rock_relayout_b2"),
], ids=["d64", "d128-keys-as-stored", "scale-tensor-bias-cross", "d256", "f32-three-kernels", "d320-three-kernels",
        "odd-head-dims"])
def test_attention_through_the_model_passes_the_gates(model, rock, oracle, loads, case):
    """The fused kernels (and the three-kernel form) on real-valued data through the model, under the gates of the
    GPU tests: RMS 1e-3 and maximum difference 0.02 for f16, 3e-5 and 1e-4 for f32."""
    from tests.gpu_util import check_float
    t, G, sq, sk, dqk, dv, trans_k, with_scale, with_bias, last = case
    dt = _NUMPY[t]
    rng = np.random.default_rng(sq + sk)
    Q = (rng.standard_normal((G, sq, dqk)) * 0.5).astype(dt)
    K = (rng.standard_normal((G, sk, dqk) if trans_k else (G, dqk, sk)) * 0.5).astype(dt)
    V = rng.standard_normal((G, sk, dv)).astype(dt)
    St = (rng.random((G, sq, sk)) * 0.5 + 0.75).astype(dt) if with_scale else None
    Bt = (rng.standard_normal((G, sq, sk)) * 0.5).astype(dt) if with_bias else None
    scale = 1.0 / np.sqrt(dqk)
    opts = _attention_problem(t, G, sq, sk, dqk, dv, trans_k, scale,
                              ("-with-attn-scale true " if with_scale else "") + ("-with-attn-bias true" if with_bias else ""))
    # caller list: Q, K, V, [scale tensor], bias, O, [workspace]
    inputs = {0: Q, 1: K, 2: V}
    at = 3
    if with_scale:
        inputs[at] = St
        at += 1
    if with_bias:
        inputs[at] = Bt
    names, problems, out = run_plan(model, rock, opts, inputs)
    assert not problems, (names, problems)
    assert names[-1] == last, names
    got = out[at + 1][:G * sq * dv * np.dtype(dt).itemsize].view(dt).astype(np.float32)
    f32 = lambda a: None if a is None else a.astype(np.float32)
    ref = oracle.attention(f32(Q), f32(K), f32(V), G, sq, sk, dqk, dv, scale=scale, scale_t=f32(St), bias_t=f32(Bt),
                           transK=trans_k)
    gate = {"f16": (1e-3, 0.02), "f32": (3e-5, 1e-4)}[t]
    check_float(got, ref, t, rms=gate[0], max_abs=gate[1])


# ---- the reference's end-to-end lists, by the harness of tests/test_gpu_e2e_lists.py with the model as the device ---
def _conv_macs(o):
    g = int(o.get("groupsize", 1))
    n, c, k = int(o["batchsize"]), int(o["in_channels"]) // g, int(o["out_channels"]) // g
    y, x = int(o["fil_h"]), int(o["fil_w"])
    ph, pw = int(o.get("padding_h", 0)), int(o.get("padding_w", 0))
    ho = (int(o["in_h"]) + int(o.get("padding_h_l", ph)) + int(o.get("padding_h_r", ph))
          - (y - 1) * int(o.get("dilation_h", 1)) - 1) // int(o.get("conv_stride_h", 1)) + 1
    wo = (int(o["in_w"]) + int(o.get("padding_w_l", pw)) + int(o.get("padding_w_r", pw))
          - (x - 1) * int(o.get("dilation_w", 1)) - 1) // int(o.get("conv_stride_w", 1)) + 1
    return n * g * c * k * ho * wo * y * x


def _listed(name, every, macs=1.5e7):
    """Every `every`-th problem of a list, batches capped at 2, convolutions within `macs` multiply-adds."""
    import re
    import tests.test_gpu_e2e_lists as lists
    out = []
    for i, opts in enumerate(lists._BY_LIST[name]):
        if i % every:
            continue
        opts = re.sub(r"-batchsize[= ](\d+)", lambda m: "-batchsize=%d" % min(int(m.group(1)), 2), opts)
        o = lists.parse_options(opts)
        if "conv" in o.get("operation", "") and _conv_macs(o) > macs:
            continue
        out.append((i, opts, o))
    return out


@pytest.mark.parametrize("name,every", [("conv_regression_bwd.toml", 6), ("conv_regression_fwd.toml", 15),
                                        ("PrAttentionF16.toml", 1), ("PrAttentionI8.toml", 2), ("PrAttentionF32.toml", 2),
                                        ("gemm_split_k_f16.toml", 3), ("gemm_split_k_f32.toml", 3)])
def test_reference_lists_through_the_model(model, rock, oracle, name, every):
    """Lists that have not run on a GPU (or not since the harness changed), through the same harness with the
    model as its device."""
    import torch
    import tests.test_gpu_e2e_lists as lists
    Device = harness_device(model, rock)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(1234)
    ran = 0
    for i, opts, o in _listed(name, every):
        try:
            rock.RockKernel(opts)
        except rock.RockError:
            continue   # (the twelve stated refusals: backward convolutions with unequal padding)
        op = o.get("operation", "")
        run = lists.run_gemm if op == "gemm" else lists.run_attention if op == "attention" else lists.run_conv
        run(Device, oracle, "cpu", gen, opts, o)
        ran += 1
    assert ran >= 2, ran
