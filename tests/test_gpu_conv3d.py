"""GPU parity: convolution over three spatial dimensions, forward and both
gradients, through the C ABI vs the CPU oracle.

The reference's own 3-D test (conv3d-test-from-rocmlir-gen.mlir) validates
against linalg.conv_3d on constant data and prints a pass flag, so it holds no
vectors; its case (1x1x1 channels, 8^3 input, 3^3 filter of twos and ones) is
the first case here, checked against its closed form.  Then integer-valued
data, where every partial sum is exact whatever the order, over strides,
dilations, padding (depth padding makes the zero-fill kernel run), groups,
odd channel counts, layouts and types."""
import numpy as np
import pytest
import torch

from tests.gpu_util import CODE, check_float, quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu

NCDHW = ("gkc012", "ngc012", "ngk012")      # rocmlir-gen's default spelling
NDHWC = ("gk012c", "n012gc", "n012gk")      # channels last
MIXED = ("g012ck", "n2g01c", "ngk201")      # depth first / in the middle


def _to_layout(t, canonical, layout):
    return np.ascontiguousarray(t.transpose([canonical.index(ch) for ch in layout])).ravel()


def test_conv3d_reference_case_closed_form(rock, gpu):
    # conv3d-test-from-rocmlir-gen.mlir:6-8: input 8x8x8 of ones, filter 3x3x3, output 6x6x6
    fil = torch.full((27,), 2.0, device=gpu)
    inp = torch.ones(512, device=gpu)
    info = {}
    got = rock.conv3d(fil, inp, fil_layout="gkc012", in_layout="ngc012", out_layout="ngk012", batchsize=1,
                      in_channels=1, out_channels=1, in_size=(8, 8, 8), fil_size=(3, 3, 3), info=info)
    torch.cuda.synchronize()
    assert got.cpu().tolist() == [54.0] * 216
    assert info["kernels"][-1].startswith("rock_conv_f32")


# (n g c k in(h,w,d) fil(y,x,z) stride pad dil)
CASES = [
    (2, 1, 8, 16, (6, 7, 5), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),      # the 3-D UNet / video shape
    (1, 1, 16, 8, (5, 5, 6), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),      # no padding: no zero fill
    (2, 1, 3, 8, (9, 8, 7), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),       # odd channels, stride 2
    (2, 2, 4, 6, (5, 6, 8), (2, 3, 3), (1, 2, 2), (0, 1, 2), (2, 1, 2)),       # groups, depth dilation and padding
    (3, 1, 8, 8, (4, 4, 9), (1, 1, 5), (1, 1, 3), (0, 0, 2), (1, 1, 1)),       # taps along depth only
    (2, 1, 16, 16, (4, 5, 1), (3, 3, 1), (1, 1, 1), (1, 1, 0), (1, 1, 1)),     # depth 1: a 2-D problem
    (1, 1, 32, 64, (8, 8, 8), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),     # more than one tile of channels
]


def _tensors(case, layouts, t, seed):
    n, g, c, k, ins, fs, stride, pad, dil = case
    rng = np.random.default_rng(seed)
    fil = rng.integers(-2, 3, (g, k, c) + fs).astype(np.float32)
    inp = rng.integers(-2, 3, (n, g, c) + ins).astype(np.float32)
    return quantise(_to_layout(fil, "gkc012", layouts[0]), t), quantise(_to_layout(inp, "ngc012", layouts[1]), t)


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8"])
def test_conv3d_exact(rock, oracle, gpu, case, layouts, t):
    n, g, c, k, ins, fs, stride, pad, dil = case
    (raw_f, fq), (raw_i, iq) = _tensors(case, layouts, t, 91)
    info = {}
    got = rock.conv3d(to_gpu(raw_f, t, gpu), to_gpu(raw_i, t, gpu), fil_layout=layouts[0], in_layout=layouts[1],
                      out_layout=layouts[2], batchsize=n, groupsize=g, in_channels=g * c, out_channels=g * k,
                      in_size=ins, fil_size=fs, stride=stride, padding=pad, dilation=dil, info=info)
    torch.cuda.synchronize()
    ref, outs = oracle.conv3d(fq, iq, *layouts, n, g, c, k, ins, fs, stride, pad, dil)
    if t == "i8":
        assert np.array_equal(to_f32(got, "i32"), ref)      # int32 accumulators as they are
    else:
        assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    names = info["kernels"]
    assert ("rock_fill_zero" in names) == any(
        not all(0 <= do * stride[2] + z * dil[2] - pad[2] < ins[2] for do in range(outs[2])) for z in range(fs[2]))
    assert sum(name.startswith("rock_conv_") for name in names) == 1


def test_conv3d_bias_relu_f16_output_from_int8(rock, oracle, gpu):
    case = CASES[0]
    n, g, c, k, ins, fs, stride, pad, dil = case
    (raw_f, fq), (raw_i, iq) = _tensors(case, NDHWC, "i8", 93)
    bias = np.arange(-8, 8, dtype=np.float32)
    got = rock.conv3d(to_gpu(raw_f, "i8", gpu), to_gpu(raw_i, "i8", gpu), fil_layout=NDHWC[0], in_layout=NDHWC[1],
                      out_layout=NDHWC[2], batchsize=n, in_channels=c, out_channels=k, in_size=ins, fil_size=fs,
                      stride=stride, padding=pad, dilation=dil, out_dtype="f16", scale=0.5,
                      bias=torch.tensor(bias, device=gpu), relu=True)
    torch.cuda.synchronize()
    ref, outs = oracle.conv3d(fq, iq, *NDHWC, n, g, c, k, ins, fs, stride, pad, dil)
    want = np.maximum(ref.reshape(-1, k) * np.float32(0.5) + bias, 0).ravel()
    assert np.array_equal(to_f32(got, "f16"), oracle.round_through(want, CODE["f16"]))


# ---- the gradients -----------------------------------------------------------
# Integer-valued data again: every product and partial sum is a small integer,
# exact in every type used (the sums stay far below 2^8, what bf16 holds
# exactly), so the order of the sums and the intermediate rounding of the
# unfolded gradient cannot matter and the comparison is bit for bit.
BWD_CASES = [
    (2, 1, 8, 16, (6, 7, 5), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),      # one group: filter gradient as one GEMM
    (2, 1, 3, 8, (9, 8, 7), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),       # odd channels, stride 2 everywhere
    (2, 2, 4, 6, (5, 6, 8), (2, 3, 3), (1, 2, 2), (0, 1, 2), (2, 1, 2)),       # groups, depth dilation and padding
    (3, 1, 8, 8, (4, 4, 9), (1, 1, 5), (1, 1, 3), (0, 0, 2), (1, 1, 1)),       # taps along depth only, depth stride 3
    (1, 1, 16, 8, (5, 5, 6), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),      # one image: output gradient read in place
    (2, 1, 16, 16, (4, 5, 1), (3, 3, 1), (1, 1, 1), (1, 1, 0), (1, 1, 1)),     # depth 1: a 2-D problem
    (2, 1, 3, 8, (5, 8, 6), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),       # few channels, strided: 2-D phases merged
]


def _bwd_tensors(case, layouts, t, seed):
    n, g, c, k, ins, fs, stride, pad, dil = case
    outs = tuple((ins[a] + 2 * pad[a] - (fs[a] - 1) * dil[a] - 1) // stride[a] + 1 for a in range(3))
    rng = np.random.default_rng(seed)
    fil = rng.integers(-1, 2, (g, k, c) + fs).astype(np.float32)
    inp = rng.integers(-1, 2, (n, g, c) + ins).astype(np.float32)
    dout = rng.integers(-1, 2, (n, g, k) + outs).astype(np.float32)
    return (quantise(_to_layout(fil, "gkc012", layouts[0]), t), quantise(_to_layout(inp, "ngc012", layouts[1]), t),
            quantise(_to_layout(dout, "ngk012", layouts[2]), t))


@pytest.mark.parametrize("case", BWD_CASES)
@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv3d_bwd_data_exact(rock, oracle, gpu, case, layouts, t):
    n, g, c, k, ins, fs, stride, pad, dil = case
    (raw_f, fq), _, (raw_o, oq) = _bwd_tensors(case, layouts, t, 95)
    info = {}
    print("conv3d bwd data", case, layouts, t, flush=True)
    got = rock.conv3d_bwd_data(to_gpu(raw_f, t, gpu), to_gpu(raw_o, t, gpu), fil_layout=layouts[0],
                               in_layout=layouts[1], out_layout=layouts[2], batchsize=n, groupsize=g,
                               in_channels=g * c, out_channels=g * k, in_size=ins, fil_size=fs, stride=stride,
                               padding=pad, dilation=dil, info=info)
    torch.cuda.synchronize()
    ref = oracle.conv3d_bwd_data(fq, oq, *layouts, n, g, c, k, ins, fs, stride, pad, dil)
    assert np.abs(ref).max() < 256
    assert np.array_equal(to_f32(got, t), ref)
    assert info["kernels"].count("rock_fold_depth") == 1


@pytest.mark.parametrize("case", BWD_CASES)
@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv3d_bwd_weight_exact(rock, oracle, gpu, case, layouts, t):
    n, g, c, k, ins, fs, stride, pad, dil = case
    _, (raw_i, iq), (raw_o, oq) = _bwd_tensors(case, layouts, t, 97)
    info = {}
    print("conv3d bwd weight", case, layouts, t, flush=True)
    got = rock.conv3d_bwd_weight(to_gpu(raw_i, t, gpu), to_gpu(raw_o, t, gpu), fil_layout=layouts[0],
                                 in_layout=layouts[1], out_layout=layouts[2], batchsize=n, groupsize=g,
                                 in_channels=g * c, out_channels=g * k, in_size=ins, fil_size=fs, stride=stride,
                                 padding=pad, dilation=dil, info=info)
    torch.cuda.synchronize()
    ref = oracle.conv3d_bwd_weight(iq, oq, *layouts, n, g, c, k, ins, fs, stride, pad, dil)
    assert np.abs(ref).max() < 256
    assert np.array_equal(to_f32(got, t), ref)
    # (a 1x1 window in h and w runs as a plain GEMM; one image's output gradient is read where it
    # lies, with the depth as the 2-D problem's batch, which need not be a dense pixel matrix)
    if g == 1 and fs[0] * fs[1] > 1 and n > 1:
        assert any(name.startswith("rock_conv_bwd_weight_") for name in info["kernels"])


@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv3d_gradients_real_values_unet_block(rock, oracle, gpu, t):
    """A 3-D UNet block (32 -> 64 channels at 16^3, batch 2, 3x3x3, padding 1)
    on real-valued data against the oracle under the reference's RMS gates.
    The 16-bit input gradient is rounded twice (each depth tap's 2-D gradient in
    the tensor type, then their f32 sum) where the reference rounds once: the
    gate is the measure of that, bf16 included."""
    n, g, c, k, ins, fs, stride, pad, dil = 2, 1, 32, 64, (16, 16, 16), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)
    rng = np.random.default_rng(99)
    raw_f, fq = quantise(rng.standard_normal(g * k * c * 27).astype(np.float32) * 0.1, t)
    raw_i, iq = quantise(rng.standard_normal(n * g * c * 16 ** 3).astype(np.float32), t)
    raw_o, oq = quantise(rng.standard_normal(n * g * k * 16 ** 3).astype(np.float32), t)
    kw = dict(fil_layout=NDHWC[0], in_layout=NDHWC[1], out_layout=NDHWC[2], batchsize=n, groupsize=g,
              in_channels=g * c, out_channels=g * k, in_size=ins, fil_size=fs, stride=stride, padding=pad,
              dilation=dil)
    print("conv3d gradients real values", t, flush=True)
    dx = rock.conv3d_bwd_data(to_gpu(raw_f, t, gpu), to_gpu(raw_o, t, gpu), **kw)
    dw = rock.conv3d_bwd_weight(to_gpu(raw_i, t, gpu), to_gpu(raw_o, t, gpu), **kw)
    torch.cuda.synchronize()
    check_float(to_f32(dx, t), oracle.conv3d_bwd_data(fq, oq, *NDHWC, n, g, c, k, ins, fs, stride, pad, dil), t)
    check_float(to_f32(dw, t), oracle.conv3d_bwd_weight(iq, oq, *NDHWC, n, g, c, k, ins, fs, stride, pad, dil), t)


@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16"])
def test_conv3d_residual_add_relu_exact(rock, oracle, gpu, layouts, t):
    """The element-wise tail with a second tensor (MIGraphXToTosa.cpp:1283-1295)
    behind a 3-D convolution: out = relu(conv + residual), residual laid out
    as the output; integer-valued data, bit for bit."""
    case = CASES[3]
    n, g, c, k, ins, fs, stride, pad, dil = case
    (raw_f, fq), (raw_i, iq) = _tensors(case, layouts, t, 101)
    ref, outs = oracle.conv3d(fq, iq, *layouts, n, g, c, k, ins, fs, stride, pad, dil)
    res = np.random.default_rng(102).integers(-6, 7, ref.size).astype(np.float32)
    raw_r, rq = quantise(res, t)
    info = {}
    print("conv3d residual", layouts, t, flush=True)
    got = rock.conv3d(to_gpu(raw_f, t, gpu), to_gpu(raw_i, t, gpu), fil_layout=layouts[0], in_layout=layouts[1],
                      out_layout=layouts[2], batchsize=n, groupsize=g, in_channels=g * c, out_channels=g * k,
                      in_size=ins, fil_size=fs, stride=stride, padding=pad, dilation=dil,
                      residual=to_gpu(raw_r, t, gpu), activation="relu", info=info)
    torch.cuda.synchronize()
    assert np.array_equal(to_f32(got, t), np.maximum(ref + rq, 0))
