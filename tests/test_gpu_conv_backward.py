"""GPU parity: backward-data and backward-weight convolution through the C ABI
(operations conv_bwd_data / conv_bwd_weight) vs the CPU oracle.

First the reference's own literal vectors (cpu_conv2d/*_bwd_data.mlir,
*_bwd_weight.mlir), then integer-valued data, where every partial sum is exact
in f32 whatever the order, over strides, dilations, padding, groups, layouts
and both routes (vector kernels behind the conversion kernels, element-wise
kernel on the tensors as they lie); real-valued data to the reference's RMS
gate."""
import json
import os

import numpy as np
import pytest
import torch

from tests.gpu_util import CODE, check_float, quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
NHWC = ("gkyxc", "nhwgc", "nhwgk")
NCHW = ("gkcyx", "ngchw", "ngkhw")


def _to_layout(t, canonical, layout):
    return np.ascontiguousarray(t.transpose([canonical.index(ch) for ch in layout])).ravel()


def _golden():
    with open(os.path.join(HERE, "golden", "conv_bwd_kats.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _golden(), ids=lambda c: c["source"])
@pytest.mark.parametrize("t", ["f32", "f16"])
def test_conv_backward_reference_golden_vectors(rock, oracle, gpu, case, t):
    f = case["flags"]
    n, c, k = int(f["batchsize"]), int(f["in_channels"]), int(f["out_channels"])
    hi, wi, y, x = int(f["in_h"]), int(f["in_w"]), int(f["fil_h"]), int(f["fil_w"])
    stride = (int(f["conv_stride_h"]), int(f["conv_stride_w"]))
    pad = (int(f["padding_h"]), int(f["padding_w"]))
    dil = (int(f["dilation_h"]), int(f["dilation_w"]))
    ho = oracle.conv_out_dim(hi, y, pad[0], pad[0], stride[0], dil[0])
    wo = oracle.conv_out_dim(wi, x, pad[1], pad[1], stride[1], dil[1])
    dt = {"f32": torch.float32, "f16": torch.float16}[t]
    kw = dict(fil_layout=f["fil_layout"], in_layout=f["in_layout"], out_layout=f["out_layout"], batchsize=n,
              in_channels=c, out_channels=k, in_h=hi, in_w=wi, fil_h=y, fil_w=x, stride=stride, padding=pad,
              dilation=dil)
    dy = torch.ones(n * k * ho * wo, dtype=dt, device=gpu)
    if f["operation"] == "conv_bwd_data":
        got = rock.conv2d_bwd_data(torch.ones(k * c * y * x, dtype=dt, device=gpu), dy, **kw)
    else:
        got = rock.conv2d_bwd_weight(torch.ones(n * c * hi * wi, dtype=dt, device=gpu), dy, **kw)
    assert got.cpu().double().tolist() == case["expected"]


# (n g c k hi wi y x stride pad dil)
CASES = [
    (2, 1, 16, 24, 9, 9, 3, 3, (1, 1), (1, 1), (1, 1)),
    (3, 1, 8, 16, 12, 10, 3, 3, (2, 2), (1, 1), (1, 1)),      # ResNet down-sampling 3x3
    (2, 1, 16, 8, 8, 8, 1, 1, (2, 2), (0, 0), (1, 1)),        # 1x1 stride 2: three of four phases stay zero
    (1, 1, 3, 8, 21, 21, 7, 7, (2, 2), (3, 3), (1, 1)),       # first layer, odd channel count
    (2, 2, 8, 8, 11, 13, 5, 5, (2, 3), (2, 2), (1, 2)),       # groups, mixed stride / dilation
    (2, 1, 8, 8, 10, 10, 3, 3, (2, 2), (2, 2), (2, 2)),       # stride and dilation share a factor
    (1, 1, 5, 7, 9, 9, 3, 3, (3, 3), (0, 0), (1, 1)),         # stride = filter size
    (8, 1, 16, 16, 6, 6, 3, 3, (1, 1), (1, 1), (1, 1)),       # batch large enough to split the weight reduction
    (4, 1, 16, 16, 5, 5, 2, 2, (1, 1), (0, 0), (2, 2)),
    (4, 1, 16, 24, 6, 6, 1, 1, (1, 1), (0, 0), (1, 1)),       # pointwise: the weight gradient is a split GEMM
    (3, 1, 64, 48, 8, 8, 1, 1, (1, 1), (0, 0), (1, 1)),
    (2, 1, 128, 192, 16, 16, 1, 1, (1, 1), (0, 0), (1, 1)),   # pointwise, more than one tile
    (2, 1, 64, 128, 16, 16, 1, 1, (2, 2), (0, 0), (1, 1)),    # strided pointwise: a quarter of the pixels is read
    (3, 2, 8, 8, 9, 12, 1, 1, (2, 3), (0, 0), (1, 1)),        # ... with groups, odd sizes, unequal strides
]
LAYOUTS = [NHWC, NCHW, ("gyxck", "hwcgn", "hwkgn")]


def _tensors(case, layouts, t, seed, integer=True):
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    fl, il, ol = layouts
    ho = (hi + 2 * pad[0] - (y - 1) * dil[0] - 1) // stride[0] + 1
    wo = (wi + 2 * pad[1] - (x - 1) * dil[1] - 1) // stride[1] + 1
    rng = np.random.default_rng(seed)
    if integer:
        fil = rng.integers(-2, 3, (g, k, c, y, x)).astype(np.float32)
        inp = rng.integers(-2, 3, (n, g, c, hi, wi)).astype(np.float32)
        dy = rng.integers(-2, 3, (n, g, k, ho, wo)).astype(np.float32)
    else:
        fil = (rng.standard_normal((g, k, c, y, x)) * 0.1).astype(np.float32)
        inp = (rng.standard_normal((n, g, c, hi, wi)) * 0.1).astype(np.float32)
        dy = (rng.standard_normal((n, g, k, ho, wo)) * 0.1).astype(np.float32)
    return (quantise(_to_layout(fil, "gkcyx", fl), t), quantise(_to_layout(inp, "ngchw", il), t),
            quantise(_to_layout(dy, "ngkhw", ol), t), ho, wo)


def _kw(case, layouts):
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    return dict(fil_layout=layouts[0], in_layout=layouts[1], out_layout=layouts[2], batchsize=n, groupsize=g,
                in_channels=g * c, out_channels=g * k, in_h=hi, in_w=wi, fil_h=y, fil_w=x, stride=stride,
                padding=pad, dilation=dil)


@pytest.mark.parametrize("convert", [True, False], ids=["converted", "as-is"])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("layouts", LAYOUTS, ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv_bwd_data_exact(rock, oracle, gpu, case, layouts, t, convert):
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    (raw_f, fq), _, (raw_dy, dyq), ho, wo = _tensors(case, layouts, t, 71)
    info = {}
    got = rock.conv2d_bwd_data(to_gpu(raw_f, t, gpu), to_gpu(raw_dy, t, gpu), layout_conversion=convert, info=info,
                               **_kw(case, layouts))
    torch.cuda.synchronize()
    ref, _, _ = oracle.conv_bwd_data(fq, dyq, *layouts, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    if not convert:
        assert not any(name.startswith("rock_relayout") for name in info["kernels"])
    elif (y, x, c % 64, hi % 8) == (1, 1, 0, 0) and stride == (1, 1) and layouts in (NHWC, NCHW):
        # pointwise with whole 16-byte runs: one GEMM over the tensors as they lie
        assert len(info["kernels"]) == 1 and info["kernels"][0].startswith("rock_gemm_")


@pytest.mark.parametrize("convert", [True, False], ids=["converted", "as-is"])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("layouts", LAYOUTS, ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv_bwd_weight_exact(rock, oracle, gpu, case, layouts, t, convert):
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    _, (raw_i, iq), (raw_dy, dyq), ho, wo = _tensors(case, layouts, t, 73)
    info = {}
    got = rock.conv2d_bwd_weight(to_gpu(raw_i, t, gpu), to_gpu(raw_dy, t, gpu), layout_conversion=convert,
                                 info=info, **_kw(case, layouts))
    torch.cuda.synchronize()
    ref, _, _ = oracle.conv_bwd_weight(iq, dyq, *layouts, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    if (y, x, c % 64, hi % 8) == (1, 1, 0, 0) and layouts in (NHWC, NCHW) and stride == (1, 1):
        # pointwise with whole 16-byte runs: a GEMM over the tensors as they lie, its split
        # partial sums added by the reduction kernel
        assert info["kernels"][0].startswith("rock_gemm_") and not any("relayout" in k for k in info["kernels"])
    elif (y, x, c % 64, hi % 16) == (1, 1, 0, 0) and layouts in (NHWC, NCHW) and convert:
        # strided pointwise: the pixels read are gathered first, then the same GEMM
        assert info["kernels"][0].startswith("rock_relayout") and info["kernels"][1].startswith("rock_gemm_")
    elif info["kernels"][0].startswith("rock_conv_bwd_weight_"):
        # channels-last, one group: one K-major GEMM whose second operand is the im2col matrix, no copies
        assert layouts == NHWC and g == 1 and info["kernels"][1:] in ([], ["rock_reduce_splits"])
    elif not convert and not info["kernels"][0].startswith("rock_gemm_"):
        assert len(info["kernels"]) == 1


BWD_WEIGHT_GEMM_CASES = [
    (16, 1, 128, 128, 28, 28, 3, 3, (1, 1), (1, 1), (1, 1)),   # the ResNet 3x3 layer: 9 column tiles, split pixels
    (4, 1, 64, 64, 14, 14, 3, 3, (1, 1), (1, 1), (1, 1)),      # 64x64 tiles
    (3, 1, 40, 72, 9, 11, 3, 2, (1, 1), (1, 0), (1, 1)),       # ragged rows and columns, taps straddle column tiles
    (2, 1, 16, 136, 13, 10, 5, 5, (2, 1), (2, 2), (1, 2)),     # stride, dilation, 5x5
    (5, 1, 8, 24, 7, 7, 7, 7, (1, 1), (3, 3), (1, 1)),         # filter as large as the image
    (1, 1, 256, 8, 6, 6, 1, 1, (1, 1), (0, 0), (1, 1)),        # 36 pixels: no split, gradient written directly
]


@pytest.mark.parametrize("case", BWD_WEIGHT_GEMM_CASES)
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv_bwd_weight_as_one_gemm_exact(rock, oracle, gpu, case, t):
    """The filter gradient of a channels-last problem as one K-major GEMM over
    the tensors as they lie, against the oracle and against the plan it replaces."""
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    _, (raw_i, iq), (raw_dy, dyq), ho, wo = _tensors(case, NHWC, t, 79)
    info, info_old = {}, {}
    xi, dy = to_gpu(raw_i, t, gpu), to_gpu(raw_dy, t, gpu)
    got = rock.conv2d_bwd_weight(xi, dy, info=info, **_kw(case, NHWC))
    old = rock.conv2d_bwd_weight(xi, dy, info=info_old, as_gemm=False, **_kw(case, NHWC))
    torch.cuda.synchronize()
    if (y, x) != (1, 1):
        assert info["kernels"][0] == "rock_conv_bwd_weight_%s_%s" % (t, "64x64" if k <= 64 else "128x128")
        assert not any(name.startswith("rock_conv_bwd_weight_") for name in info_old["kernels"])
    ref, _, _ = oracle.conv_bwd_weight(iq, dyq, *NHWC, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    assert torch.equal(got.view(torch.uint8), old.view(torch.uint8))


@pytest.mark.parametrize("t", ["f16", "f32"])
def test_conv_backward_resnet_block_real_values(rock, oracle, gpu, t):
    """ResNet50 3x3 128->128 @28x28 (conv-configs:5), batch 16: both gradients
    on the vector kernels (split weight reduction included), the reference's RMS gate."""
    case = (16, 1, 128, 128, 28, 28, 3, 3, (1, 1), (1, 1), (1, 1))
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    (raw_f, fq), (raw_i, iq), (raw_dy, dyq), ho, wo = _tensors(case, NHWC, t, 75, integer=False)
    info = {}
    dx = rock.conv2d_bwd_data(to_gpu(raw_f, t, gpu), to_gpu(raw_dy, t, gpu), info=info, **_kw(case, NHWC))
    assert info["kernels"][-1].endswith("_fast")
    ref, _, _ = oracle.conv_bwd_data(fq, dyq, *NHWC, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    check_float(to_f32(dx, t), ref, t)
    dw = rock.conv2d_bwd_weight(to_gpu(raw_i, t, gpu), to_gpu(raw_dy, t, gpu), info=info, **_kw(case, NHWC))
    assert info["kernels"] == ["rock_conv_bwd_weight_%s_128x128" % t, "rock_reduce_splits"]
    ref, _, _ = oracle.conv_bwd_weight(iq, dyq, *NHWC, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    check_float(to_f32(dw, t), ref, t)


@pytest.mark.parametrize("layouts", [NHWC, ("gkcyx", "nhwgc", "nhwgk")], ids=["gkyxc", "gkcyx"])
def test_conv_bwd_data_on_the_window_resident_kernel_exact(rock, oracle, gpu, layouts):
    """The unit-stride input gradient of a full-size 3x3 layer (batch 128 of
    ResNet50's 28x28 stage): the table puts it on the window-resident kernel,
    behind ONE conversion that flips, swaps and repacks the filter.  Integer
    data, bit for bit against the oracle and against the implicit-GEMM plan."""
    case = (128, 1, 128, 128, 28, 28, 3, 3, (1, 1), (1, 1), (1, 1))
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    (raw_f, fq), _, (raw_dy, dyq), ho, wo = _tensors(case, layouts, "f16", 79, integer=True)
    info = {}
    print("bwd data, window-resident", layouts, flush=True)
    dx = rock.conv2d_bwd_data(to_gpu(raw_f, "f16", gpu), to_gpu(raw_dy, "f16", gpu), info=info, **_kw(case, layouts))
    torch.cuda.synchronize()
    assert info["kernels"] == ["rock_relayout_b2", "rock_conv_f16_direct224"]
    ref, _, _ = oracle.conv_bwd_data(fq, dyq, *layouts, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(dx, "f16"), oracle.round_through(ref, CODE["f16"]))


@pytest.mark.parametrize("case,last", [
    ((128, 1, 256, 128, 28, 28, 3, 3, (1, 1), (1, 1), (1, 1)), "rock_conv_f16_128x128_fast"),
    ((64, 1, 256, 64, 56, 56, 3, 3, (1, 1), (1, 1), (1, 1)), "rock_conv_f16_direct224"),
], ids=["28x28", "56x56"])
def test_conv_bwd_data_channel_major_gradient_exact(rock, oracle, gpu, case, last):
    """The same gradients written channel-major (NCHW), as 16-byte vectors of consecutive pixels: the reference's
    backward regression list holds both layers.  Four rows of 56 pixels are whole vectors, so that layer stays on
    the window-resident kernel; seven rows of 28 pixels are not (tiles would start in the middle of a vector), and
    the table keeps the layer on the implicit-GEMM kernel, whose tiles start at multiples of 32 pixels."""
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    (raw_f, fq), _, (raw_dy, dyq), ho, wo = _tensors(case, NCHW, "f16", 83, integer=True)
    info = {}
    print("bwd data, channel-major gradient", case, flush=True)
    dx = rock.conv2d_bwd_data(to_gpu(raw_f, "f16", gpu), to_gpu(raw_dy, "f16", gpu), info=info, **_kw(case, NCHW))
    torch.cuda.synchronize()
    assert info["kernels"][-1] == last
    ref, _, _ = oracle.conv_bwd_data(fq, dyq, *NCHW, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(dx, "f16"), oracle.round_through(ref, CODE["f16"]))


NARROW_CASES = [
    (8, 1, 3, 64, 38, 38, 7, 7, (2, 2), (0, 0), (1, 1)),      # the ResNet first layer in small, pixels split
    (2, 1, 3, 16, 20, 20, 7, 7, (2, 2), (0, 0), (1, 1)),
    (3, 1, 3, 136, 15, 18, 3, 3, (2, 2), (1, 0), (1, 1)),     # rows padded at the top and bottom, 128x128 tiles
    (2, 1, 4, 24, 12, 16, 5, 3, (2, 2), (2, 0), (1, 1)),      # four channels
    (2, 1, 2, 8, 9, 16, 3, 5, (3, 4), (0, 0), (2, 1)),        # two channels, stride 4 along w, dilated rows
    (1, 1, 1, 8, 10, 24, 3, 3, (1, 8), (1, 0), (1, 1)),       # one channel
]


@pytest.mark.parametrize("case", NARROW_CASES)
@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv_bwd_weight_over_a_few_channels_exact(rock, oracle, gpu, case, layouts, t):
    """Images with a few channels: channels-last copy with the channel run padded to a fraction of a chunk,
    rows of filter taps read as one run by the K-major GEMM, padding columns left out by the reduction."""
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    _, (raw_i, iq), (raw_dy, dyq), ho, wo = _tensors(case, layouts, t, 83)
    info, info_old = {}, {}
    xi, dy = to_gpu(raw_i, t, gpu), to_gpu(raw_dy, t, gpu)
    got = rock.conv2d_bwd_weight(xi, dy, info=info, **_kw(case, layouts))
    old = rock.conv2d_bwd_weight(xi, dy, info=info_old, as_gemm=False, **_kw(case, layouts))
    torch.cuda.synchronize()
    if not (t == "f32" and c == 4):
        assert info["kernels"][-2:] == ["rock_conv_bwd_weight_%s_%s" % (t, "64x64" if k <= 64 else "128x128"),
                                        "rock_reduce_splits"]
        assert info["kernels"][0].startswith("rock_relayout_b")
    assert not any(name.startswith("rock_conv_bwd_weight_") for name in info_old["kernels"])
    ref, _, _ = oracle.conv_bwd_weight(iq, dyq, *layouts, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    assert torch.equal(got.view(torch.uint8), old.view(torch.uint8))


NARROW_K_CASES = [
    (2, 1, 320, 4, 64, 64, 3, 3, (1, 1), (1, 1), (1, 1)),     # the UNet layer that ends in 4 channels
    (2, 1, 32, 4, 12, 12, 3, 3, (1, 1), (1, 1), (1, 1)),
    (3, 1, 16, 3, 9, 11, 3, 3, (2, 2), (1, 1), (1, 1)),
    (2, 1, 64, 12, 8, 8, 5, 5, (1, 1), (2, 2), (1, 1)),
    (1, 1, 8, 1, 10, 10, 2, 2, (1, 1), (0, 0), (1, 1)),
]


@pytest.mark.parametrize("case", NARROW_K_CASES)
@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv_bwd_weight_of_a_narrow_output_gradient_exact(rock, oracle, gpu, case, layouts, t):
    """k * es not a whole chunk: the output gradient is copied with its channels padded with zeros, the
    K-major GEMM runs over the copy and the reduction leaves the padding rows out."""
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    es = 4 if t == "f32" else 2
    _, (raw_i, iq), (raw_dy, dyq), ho, wo = _tensors(case, layouts, t, 89)
    info, info_old = {}, {}
    xi, dy = to_gpu(raw_i, t, gpu), to_gpu(raw_dy, t, gpu)
    got = rock.conv2d_bwd_weight(xi, dy, info=info, **_kw(case, layouts))
    old = rock.conv2d_bwd_weight(xi, dy, info=info_old, as_gemm=False, **_kw(case, layouts))
    torch.cuda.synchronize()
    if (c * es) % 16 == 0 and (k * es) % 16 != 0:
        assert info["kernels"][-2:] == ["rock_conv_bwd_weight_%s_64x64" % t, "rock_reduce_splits"]
        assert info["kernels"][0].startswith("rock_relayout_b")
    ref, _, _ = oracle.conv_bwd_weight(iq, dyq, *layouts, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    assert torch.equal(got.view(torch.uint8), old.view(torch.uint8))


BWD_DATA_SPLIT_CASES = [
    (2, 1, 320, 640, 16, 16, 3, 3, (1, 1), (1, 1), (1, 1)),    # a UNet layer at batch 2 in small
    (2, 1, 64, 256, 8, 8, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 1, 40, 512, 6, 7, 2, 2, (1, 1), (0, 0), (1, 1)),
    (2, 1, 24, 100, 5, 5, 5, 5, (1, 1), (2, 2), (1, 1)),
    (2, 1, 128, 384, 6, 6, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 1, 72, 256, 9, 7, 3, 3, (1, 1), (1, 1), (2, 1)),       # dilated rows
]


@pytest.mark.parametrize("case", BWD_DATA_SPLIT_CASES)
@pytest.mark.parametrize("layouts", LAYOUTS, ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv_bwd_data_reduction_split_exact(rock, oracle, gpu, case, layouts, t):
    """Unit stride, few output tiles, a long reduction over (taps, k): shares of the reduction as groups,
    partial sums added by the reduction kernel into the input gradient."""
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    (raw_f, fq), _, (raw_dy, dyq), ho, wo = _tensors(case, layouts, t, 97)
    info = {}
    got = rock.conv2d_bwd_data(to_gpu(raw_f, t, gpu), to_gpu(raw_dy, t, gpu), info=info, **_kw(case, layouts))
    torch.cuda.synchronize()
    ref, _, _ = oracle.conv_bwd_data(fq, dyq, *layouts, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    es = 4 if t == "f32" else 2
    kfull = -(-k * es // 16) * 16 // es * y * x
    most = min(1024 // (-(-n * hi * wi // 64) * -(-c // 64)), kfull // 1024)
    if any(kfull % d == 0 and (kfull // d) % (128 // es) == 0 for d in range(2, most + 1)):
        assert info["kernels"][-1] == "rock_reduce_splits"


MERGED_PHASE_CASES = [
    (4, 1, 3, 64, 46, 46, 7, 7, (2, 2), (0, 0), (1, 1)),      # the first layer in small
    (2, 1, 3, 64, 32, 32, 7, 7, (2, 2), (3, 3), (1, 1)),      # padded: the phases start at different rows
    (3, 1, 4, 16, 12, 20, 3, 3, (2, 2), (1, 1), (1, 1)),
    (1, 1, 2, 24, 12, 18, 5, 5, (3, 3), (2, 2), (1, 1)),      # nine phases
    (2, 1, 16, 40, 16, 16, 3, 3, (2, 2), (1, 1), (1, 1)),     # 64 merged columns
    (2, 1, 3, 5, 12, 12, 3, 3, (2, 2), (1, 1), (1, 1)),       # k padded to whole chunks
    (2, 1, 1, 32, 16, 16, 4, 4, (2, 2), (1, 1), (1, 1)),      # one channel: runs of two elements
]


@pytest.mark.parametrize("case", MERGED_PHASE_CASES)
@pytest.mark.parametrize("layouts", LAYOUTS, ids=lambda l: l[1])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
def test_conv_bwd_data_merged_phases_exact(rock, oracle, gpu, case, layouts, t):
    """A strided layer with few input channels: every phase in one convolution with (phase, channel) output
    columns, interleaved into the input gradient by a conversion kernel."""
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    (raw_f, fq), _, (raw_dy, dyq), ho, wo = _tensors(case, layouts, t, 98)
    info = {}
    got = rock.conv2d_bwd_data(to_gpu(raw_f, t, gpu), to_gpu(raw_dy, t, gpu), info=info, **_kw(case, layouts))
    torch.cuda.synchronize()
    ref, _, _ = oracle.conv_bwd_data(fq, dyq, *layouts, n, g, c, k, hi, wi, y, x, stride, pad, dil)
    assert np.array_equal(to_f32(got, t), oracle.round_through(ref, CODE[t]))
    names = info["kernels"]
    assert sum(nm.startswith("rock_conv_") for nm in names) == 1 and "rock_fill_zero" in names, names
