"""GPU parity: forward convolution through the C ABI vs the CPU oracle and the
reference's own golden vectors."""
import json
import os

import numpy as np
import pytest
import torch

from tests.gpu_util import CODE, check_float, quantise, to_f32, to_gpu

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _to_layout(t, canonical, layout):
    perm = [canonical.index(ch) for ch in layout]
    return np.ascontiguousarray(t.transpose(perm)).ravel()


def _run(rock, oracle, gpu, t, n, g, c, k, hi, wi, y, x, stride, pad, dil, layouts, integer, seed,
         out_dtype=None, pad_r=None, **epi):
    fl, il, ol = layouts
    rng = np.random.default_rng(seed)
    if t == "i8":
        fil = rng.integers(-128, 128, (g, k, c, y, x)).astype(np.float32)
        inp = rng.integers(-128, 128, (n, g, c, hi, wi)).astype(np.float32)
    elif integer:
        fil = rng.integers(-2, 3, (g, k, c, y, x)).astype(np.float32)
        inp = rng.integers(-2, 3, (n, g, c, hi, wi)).astype(np.float32)
    else:
        fil = (rng.standard_normal((g, k, c, y, x)) * 0.1).astype(np.float32)
        inp = (rng.standard_normal((n, g, c, hi, wi)) * 0.1).astype(np.float32)
    raw_f, fq = quantise(_to_layout(fil, "gkcyx", fl), t)
    raw_i, iq = quantise(_to_layout(inp, "ngchw", il), t)
    out = rock.conv2d(to_gpu(raw_f, t, gpu), to_gpu(raw_i, t, gpu), fil_layout=fl, in_layout=il,
                      out_layout=ol, batchsize=n, in_channels=g * c, out_channels=g * k, in_h=hi,
                      in_w=wi, fil_h=y, fil_w=x, groupsize=g, stride=stride, padding=pad, dilation=dil,
                      out_dtype=out_dtype, padding_r=pad_r, **epi)
    torch.cuda.synchronize()
    if t == "i8":
        ref, ho, wo = oracle.conv_fwd(raw_f, raw_i, fl, il, ol, n, g, c, k, hi, wi, y, x, stride, pad, dil,
                                      pad_r=pad_r)
    else:
        ref, ho, wo = oracle.conv_fwd(fq, iq, fl, il, ol, n, g, c, k, hi, wi, y, x, stride, pad, dil, pad_r=pad_r)
    od = out_dtype or {"i8": "i32", "fp8": "f32", "bf8": "f32"}.get(t, t)
    assert out.numel() == ref.size
    return out, od, ref


def _golden():
    with open(os.path.join(HERE, "golden", "conv_fwd_kats.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _golden(), ids=lambda c: c["source"])
@pytest.mark.parametrize("t", ["f32", "f16", "i8"])
def test_conv_reference_golden_vectors(rock, gpu, case, t):
    """cpu_conv2d/*_fwd.mlir: all-ones data, the literal vector FileCheck expects."""
    f = case["flags"]
    n, c, k = int(f["batchsize"]), int(f["in_channels"]), int(f["out_channels"])
    hi, wi, y, x = int(f["in_h"]), int(f["in_w"]), int(f["fil_h"]), int(f["fil_w"])
    dt = {"f32": torch.float32, "f16": torch.float16, "i8": torch.int8}[t]
    fil = torch.ones(k * c * y * x, dtype=dt, device=gpu)
    inp = torch.ones(n * c * hi * wi, dtype=dt, device=gpu)
    out = rock.conv2d(fil, inp, fil_layout=f["fil_layout"], in_layout=f["in_layout"],
                      out_layout=f["out_layout"], batchsize=n, in_channels=c, out_channels=k,
                      in_h=hi, in_w=wi, fil_h=y, fil_w=x,
                      stride=(int(f["conv_stride_h"]), int(f["conv_stride_w"])),
                      padding=(int(f["padding_h"]), int(f["padding_w"])),
                      dilation=(int(f["dilation_h"]), int(f["dilation_w"])))
    assert out.cpu().double().tolist() == case["expected"]


NHWC = ("gkyxc", "nhwgc", "nhwgk")
NCHW = ("gkcyx", "ngchw", "ngkhw")
# (n g c k hi wi y x stride pad dil): PaddedGemmConfig.toml:23-48 and
# conv_regression_fwd.toml:23-227 shapes, batch trimmed
EDGE_CASES = [
    (2, 1, 7, 64, 11, 11, 3, 3, (2, 2), (1, 1), (1, 1)),
    (19, 1, 8, 16, 7, 7, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 1, 13, 11, 7, 7, 3, 3, (1, 1), (0, 0), (1, 1)),
    (1, 1, 15, 8, 5, 5, 3, 3, (2, 2), (1, 1), (1, 1)),
    (1, 1, 3, 64, 56, 56, 7, 7, (2, 2), (3, 3), (1, 1)),
    (2, 1, 3, 6, 32, 32, 7, 7, (1, 1), (0, 0), (1, 1)),
    (2, 1, 8, 8, 16, 64, 5, 5, (2, 3), (2, 2), (1, 2)),
    (1, 1, 16, 16, 14, 14, 14, 14, (1, 1), (1, 1), (1, 1)),
    (3, 1, 8, 8, 4, 4, 1, 1, (3, 3), (1, 1), (2, 2)),
    (2, 4, 64, 64, 7, 7, 1, 1, (1, 1), (0, 0), (1, 1)),
    (2, 2, 16, 24, 9, 9, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 1, 16, 24, 9, 9, 1, 1, (2, 2), (0, 0), (1, 1)),      # strided pointwise: the conversion copies the used pixels only
    (2, 1, 16, 24, 8, 10, 1, 1, (2, 3), (0, 0), (1, 1)),
    (2, 1, 8, 16, 1, 50, 1, 5, (1, 2), (0, 2), (1, 1)),      # a 1-D convolution written as 2-D with height 1
]


@pytest.mark.parametrize("case", EDGE_CASES)
@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=["nhwc", "nchw"])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8"])
def test_conv_edge_shapes_exact(rock, oracle, gpu, case, layouts, t):
    out, od, ref = _run(rock, oracle, gpu, t, *case, layouts, True, 31)
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        assert np.array_equal(to_f32(out, od), ref)


# (n g c k hi wi y x stride pad_left dil pad_right)
ASYM_PAD_CASES = [
    (2, 1, 64, 128, 14, 14, 2, 2, (1, 1), (0, 0), (1, 1), (1, 1)),   # "same" padding of an even filter
    (3, 1, 16, 32, 9, 11, 3, 3, (2, 2), (0, 1), (1, 1), (1, 2)),
    (2, 2, 8, 16, 7, 7, 3, 2, (1, 1), (2, 0), (1, 2), (0, 1)),
]


@pytest.mark.parametrize("case", ASYM_PAD_CASES)
@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=["nhwc", "nchw"])
@pytest.mark.parametrize("perf", [None, "v2:224,128,8,224,32,8,1,1,1"], ids=["table", "direct224-asked"])
def test_conv_asymmetric_padding_exact(rock, oracle, gpu, case, layouts, perf):
    """--padding_h_l / _r, --padding_w_l / _r with different values on the two
    sides.  A request for the window-resident kernel, which only knows
    symmetric padding, must fall back and still be exact."""
    *shape, pad_r = case
    info = {}
    out, od, ref = _run(rock, oracle, gpu, "f16", *shape, layouts, True, 77, pad_r=pad_r, perf_config=perf,
                        info=info)
    assert "direct224" not in info["kernel_name"]
    assert np.array_equal(to_f32(out, od), ref)


MIXED = [(f, i, o) for f in ("gkcyx", "gkyxc", "gyxck") for i, o in
         (("ngchw", "ngkhw"), ("nhwgc", "nhwgk"), ("hwcgn", "hwkgn"), ("nhwgc", "ngkhw"))]


@pytest.mark.parametrize("layouts", MIXED, ids=lambda l: "-".join(l))
def test_conv_mixed_layouts(rock, oracle, gpu, layouts):
    # MixedConvLayouts.toml:14-36: N=32, C=2, K=4, 2x2 image, 2x2 filter, p1
    out, od, ref = _run(rock, oracle, gpu, "f32", 32, 1, 2, 4, 2, 2, 2, 2, (1, 1), (1, 1), (1, 1),
                        layouts, True, 33)
    assert np.array_equal(to_f32(out, od), ref)


# 1x1 filters over NCHW images run as a batched GEMM with a K-major second
# operand (no conversion kernels).  (n c k hi wi)
POINTWISE_CASES = [(3, 64, 48, 8, 8), (2, 32, 200, 12, 12), (5, 16, 16, 16, 4), (1, 128, 300, 28, 28)]


@pytest.mark.parametrize("case", POINTWISE_CASES)
@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8"])
def test_conv_pointwise_nchw_as_gemm_exact(rock, oracle, gpu, case, t):
    n, c, k, hi, wi = case
    info = {}
    out, od, ref = _run(rock, oracle, gpu, t, n, 1, c, k, hi, wi, 1, 1, (1, 1), (0, 0), (1, 1), NCHW, True, 45,
                        info=info)
    assert info["kernels"] == [info["kernel_name"]] and info["kernel_name"].startswith("rock_gemm_")
    assert info["kernel_name"].endswith("_fast_nn")
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od]))


def test_conv_pointwise_nchw_real_values_with_epilogue(rock, oracle, gpu):
    out, od, ref = _run(rock, oracle, gpu, "f16", 4, 1, 256, 64, 56, 56, 1, 1, (1, 1), (0, 0), (1, 1), NCHW, False,
                        47, scale=0.5, relu=True)
    check_float(to_f32(out, od), np.maximum(ref * 0.5, 0.0), od)


# Channel counts whose runs are not whole 16-byte chunks: the conversion
# kernels zero-pad them (3 -> 8 f16 / 16 i8 / 4 f32 channels, 100 -> 104 f16).
# (n g c k hi wi y x stride pad dil)
PADDED_CASES = [
    (2, 1, 3, 32, 20, 300, 7, 7, (2, 2), (3, 3), (1, 1)),    # rows longer than one transposing tile
    (1, 3, 5, 16, 9, 9, 3, 3, (1, 1), (1, 1), (1, 1)),       # groups
    (1, 1, 100, 24, 6, 6, 3, 3, (1, 1), (1, 1), (1, 1)),     # several chunks a pixel, the last one partial
    (3, 2, 1, 8, 12, 12, 5, 5, (1, 1), (2, 2), (1, 1)),      # depth-wise-like single channel
]
PADDED_LAYOUTS = [NHWC, NCHW, ("gyxck", "hwcgn", "hwkgn"), ("gkcyx", "nhwgc", "ngkhw")]


@pytest.mark.parametrize("case", PADDED_CASES)
@pytest.mark.parametrize("layouts", PADDED_LAYOUTS, ids=lambda l: "-".join(l))
@pytest.mark.parametrize("t", ["f32", "f16", "i8"])
def test_conv_channel_padding_exact(rock, oracle, gpu, case, layouts, t):
    out, od, ref = _run(rock, oracle, gpu, t, *case, layouts, True, 41)
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        assert np.array_equal(to_f32(out, od), ref)


def test_conv_channel_padding_takes_the_vector_kernel(rock, oracle, gpu):
    """ResNet50's first layer (conv-configs:1, batch trimmed), real values; the
    plan's kernels are the two conversions and a vector contraction kernel."""
    info = {}
    out, od, ref = _run(rock, oracle, gpu, "f16", 4, 1, 3, 64, 230, 230, 7, 7, (2, 2), (0, 0), (1, 1),
                        NCHW, False, 43, info=info)
    assert info["kernels"] == ["rock_relayout_b2", "rock_relayout_b2", "rock_conv_f16_64x64_fast_runs"]
    check_float(to_f32(out, od), ref, od)


@pytest.mark.parametrize("t", ["f16", "bf16", "f32", "fp8"])
def test_conv_resnet_block_real_values(rock, oracle, gpu, t):
    """ResNet50 3x3 128->128 @28x28 (conv-configs:5), batch 4: the vector-load
    implicit-GEMM kernel with real-valued data, reference RMS gate."""
    out, od, ref = _run(rock, oracle, gpu, t, 4, 1, 128, 128, 28, 28, 3, 3, (1, 1), (1, 1), (1, 1),
                        NHWC, False, 35)
    check_float(to_f32(out, od), ref, od)


@pytest.mark.parametrize("tile", ["256,128", "128,128", "64,64"])
def test_conv_every_fast_tile(rock, oracle, gpu, tile):
    out, od, ref = _run(rock, oracle, gpu, "f16", 3, 2, 32, 48, 13, 11, 3, 3, (1, 2), (1, 0), (2, 1),
                        NHWC, True, 37, perf_config="v2:%s,8,64,16,8,1,1,1" % tile)
    assert np.array_equal(to_f32(out, od), ref)


# The window-resident kernel ("-perf_config v2:224,128,..."): stride 1, dilation 1.
# (n g pixel_bytes k hi wi y x pad); the channel count follows from the element size.
WINDOW_CASES = [
    (3, 1, 128, 128, 28, 28, 3, 3, (1, 1)),  # 7-row tiles: four per image
    (5, 1, 256, 96, 9, 7, 3, 3, (1, 1)),     # whole small images per tile, 96 of 128 output channels
    (4, 1, 128, 32, 30, 30, 3, 3, (0, 1)),   # 28x30 outputs, padding in one direction only
    (3, 1, 128, 64, 10, 12, 3, 3, (1, 1)),   # tiles capped at the image height of 10
    (7, 1, 128, 64, 6, 50, 3, 3, (1, 1)),    # 4-row tiles against 6-row images: tiles straddle images
    (2, 2, 128, 96, 12, 20, 3, 5, (1, 2)),   # two groups, 3x5 filter, each group padded to 128 channels
    (2, 1, 128, 160, 10, 33, 2, 2, (0, 0)),  # even filter, no padding, two tiles of output channels
    (1, 1, 512, 64, 6, 6, 5, 5, (2, 2)),     # 512-byte pixels, 5x5 filter
    (9, 1, 256, 128, 14, 14, 3, 3, (1, 1)),  # 14-wide images: 16-row budget, window-limited
    (2, 1, 1024, 32, 8, 8, 3, 3, (1, 1)),    # 1024-byte pixels: 64 chunks per pixel, eight K-steps per tap
    (3, 1, 128, 64, 12, 16, 1, 3, (0, 1)),   # one filter row: the window holds exactly the tile's rows
]


@pytest.mark.parametrize("case", WINDOW_CASES)
@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8", "fp8"])
def test_conv_window_resident_kernel_exact(rock, oracle, gpu, case, t):
    n, g, pixel_bytes, k, hi, wi, y, x, pad = case
    c = pixel_bytes // {"f32": 4, "f16": 2, "bf16": 2, "i8": 1, "fp8": 1}[t]
    info = {}
    print("window-resident conv", case, t, flush=True)
    out, od, ref = _run(rock, oracle, gpu, t, n, g, c, k, hi, wi, y, x, (1, 1), pad, (1, 1), NHWC, True, 41,
                        perf_config="v2:224,128,8,224,32,8,1,1,1", info=info)
    assert info["kernels"] == ["rock_relayout_b%d" % {"f32": 4, "f16": 2, "bf16": 2}.get(t, 1),
                               "rock_conv_%s_direct224" % t]
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        # integer data: every partial sum is exact in f32; only the final
        # narrowing rounds (sums of up to 1152 terms exceed bf16's 8 bits)
        assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od]))


def test_conv_window_resident_kernel_real_values_and_epilogue(rock, oracle, gpu):
    """Real-valued f16 data through the window-resident kernel with a ReLU and
    an f32 output, against the oracle with the reference's RMS gate."""
    info = {}
    out, od, ref = _run(rock, oracle, gpu, "f16", 4, 1, 128, 128, 28, 28, 3, 3, (1, 1), (1, 1), (1, 1),
                        NHWC, False, 43, out_dtype="f32", relu=True, perf_config="v2:224,128,8,224,32,8,1,1,1",
                        info=info)
    assert info["kernel_name"] == "rock_conv_f16_direct224"
    check_float(to_f32(out, od), np.maximum(ref, 0.0), od)


def test_conv_window_resident_request_falls_back(rock, oracle, gpu):
    """A stride-2 problem cannot use the window-resident kernel: the request
    falls back to the table (tuningFallback, AffixTuningParameters.cpp:129-141)."""
    info = {}
    out, od, ref = _run(rock, oracle, gpu, "f16", 2, 1, 64, 32, 14, 14, 3, 3, (2, 2), (1, 1), (1, 1),
                        NHWC, True, 45, perf_config="v2:224,128,8,224,32,8,1,1,1", info=info)
    assert "direct" not in info["kernel_name"]
    assert np.array_equal(to_f32(out, od), ref)


def test_conv_i8_dequantise_per_tensor(rock, oracle, gpu):
    # int8 conv 3x3 s2 p1 -> dequantize (mixr-resnet-fusion-case-1-quantization.mlir chain)
    out, od, ref = _run(rock, oracle, gpu, "i8", 2, 1, 16, 32, 14, 14, 3, 3, (2, 2), (1, 1), (1, 1),
                        NHWC, True, 39, out_dtype="f16", scale=1.2207e-4)
    want = oracle.round_through(oracle.dequantize(ref, 1.2207e-4, 0), CODE["f16"])
    assert np.array_equal(to_f32(out, "f16"), want)


# NCHW-style outputs (pixels contiguous per channel) whose pixel runs are whole
# 16-byte chunks leave the tiled kernels as 16-byte vectors of consecutive
# pixels: one- and four-byte output elements (the two-byte ones run in every
# NCHW case above), with and without the layout-conversion kernels in front.
@pytest.mark.parametrize("in_layouts", [NCHW, ("gkyxc", "nhwgc", "ngkhw")], ids=["nchw", "nhwc-in"])
@pytest.mark.parametrize("t,od", [("i8", "i8"), ("i8", "i32"), ("f16", "f32"), ("f16", "fp8")])
def test_conv_pixel_contiguous_output_vector_store_exact(rock, oracle, gpu, t, od, in_layouts):
    n, g, c, k, hi, wi = 3, 1, 32, 72, 16, 16
    if od == "i8":
        out, _, ref = _run(rock, oracle, gpu, t, n, g, c, k, hi, wi, 3, 3, (1, 1), (1, 1), (1, 1), in_layouts, True,
                           141, out_dtype="i8", scale=0.001, quant_scale=0.5, out_zero_point=-3)
        want = oracle.quantize_i8(oracle.dequantize(ref, 0.001, 0), 0.5, -3)
        assert np.array_equal(out.cpu().numpy().ravel(), want.ravel())
    elif od == "i32":
        out, _, ref = _run(rock, oracle, gpu, t, n, g, c, k, hi, wi, 3, 3, (1, 1), (1, 1), (1, 1), in_layouts, True, 142)
        assert np.array_equal(out.cpu().numpy().ravel(), ref.ravel())
    else:
        out, _, ref = _run(rock, oracle, gpu, t, n, g, c, k, hi, wi, 3, 3, (1, 1), (1, 1), (1, 1), in_layouts, True,
                           143, out_dtype=od, scale=0.25)
        want = oracle.round_through(np.asarray(ref, np.float32) * np.float32(0.25), CODE[od])
        assert np.array_equal(to_f32(out, od), want)


# (n g c k hi wi y x stride pad dil): narrow pixels, no padding or dilation along w, rows of whole chunks
TAP_ROW_CASES = [
    (4, 1, 3, 64, 38, 38, 7, 7, (2, 2), (0, 0), (1, 1)),      # the ResNet first layer in small
    (2, 1, 3, 16, 20, 20, 7, 7, (2, 2), (0, 0), (1, 1)),
    (3, 1, 3, 136, 15, 18, 3, 3, (2, 2), (1, 0), (1, 1)),     # rows padded at the top and bottom, three column tiles
    (2, 1, 2, 8, 9, 16, 3, 5, (3, 4), (0, 0), (2, 1)),        # two channels, stride 4 along w, dilated rows
    (2, 1, 4, 24, 12, 16, 4, 4, (2, 2), (2, 0), (1, 1)),      # 4 taps of 4 channels
    (1, 1, 1, 8, 10, 24, 3, 3, (1, 8), (1, 0), (1, 1)),       # one channel
    (2, 1, 3, 32, 70, 64, 5, 5, (1, 2), (2, 0), (1, 1)),      # many K-steps over the rows of taps
]


@pytest.mark.parametrize("case", TAP_ROW_CASES)
@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=["nhwc", "nchw"])
@pytest.mark.parametrize("t", ["f16", "bf16", "i8", "fp8"])
def test_conv_rows_of_taps_exact(rock, oracle, gpu, case, layouts, t):
    """Narrow pixels: both tensors copied into rows of taps, the contraction over K = y * run on the kernels
    that clear what a run holds behind its data."""
    info = {}
    out, od, ref = _run(rock, oracle, gpu, t, *case, layouts, True, 47, info=info)
    assert len(info["kernels"]) == 3 and "_64x64_fast" in info["kernels"][2]
    c, x = case[2], case[7]
    es = 2 if t in ("f16", "bf16") else 1
    cpad = max(4 // es, 1 << (c - 1).bit_length())
    while (case[8][1] * cpad * es) % 16:
        cpad *= 2
    assert info["kernels"][2].endswith("_runs") == ((x * cpad * es) % 16 != 0)
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        assert np.array_equal(to_f32(out, od), ref)


@pytest.mark.parametrize("layouts", [NHWC, NCHW], ids=["nhwc", "nchw"])
def test_conv_rows_of_taps_keep_an_infinity_in_its_own_windows(rock, oracle, gpu, layouts):
    """The pixel behind a row of taps comes along with the run's last chunk and meets zeros of the filter;
    an Inf there must not reach the sum (0 * Inf is NaN): the kernel clears it first."""
    n, g, c, k, hi, wi, y, x = 2, 1, 3, 16, 20, 20, 7, 7
    fl, il, ol = layouts
    rng = np.random.default_rng(53)
    fil = rng.integers(-2, 3, (g, k, c, y, x)).astype(np.float32)
    inp = rng.integers(-2, 3, (n, g, c, hi, wi)).astype(np.float32)
    inp[0, 0, 1, 9, 13] = np.inf     # column 13 = 2 * 3 + 7: the pixel behind the taps of output column 3
    inp[1, 0, 0, 4, 7] = -np.inf
    raw_f, fq = quantise(_to_layout(fil, "gkcyx", fl), "f16")
    raw_i, iq = quantise(_to_layout(inp, "ngchw", il), "f16")
    info = {}
    out = rock.conv2d(to_gpu(raw_f, "f16", gpu), to_gpu(raw_i, "f16", gpu), fil_layout=fl, in_layout=il,
                      out_layout=ol, batchsize=n, in_channels=c, out_channels=k, in_h=hi, in_w=wi, fil_h=y, fil_w=x,
                      groupsize=1, stride=(2, 2), padding=(0, 0), dilation=(1, 1), info=info)
    torch.cuda.synchronize()
    assert info["kernels"][2] == "rock_conv_f16_64x64_fast_runs"
    with np.errstate(invalid="ignore"):
        ref, ho, wo = oracle.conv_fwd(fq, iq, fl, il, ol, n, g, c, k, hi, wi, y, x, (2, 2), (0, 0), (1, 1))
    got = to_f32(out, "f16")
    assert np.isnan(ref).any() or np.isinf(ref).any()
    finite = np.isfinite(ref)
    assert np.array_equal(np.isfinite(got), finite) and np.array_equal(got[finite], ref[finite])
    assert np.array_equal(np.isnan(got), np.isnan(ref))


# few output tiles, a long reduction: the (taps, channels) range split over blocks
SPLIT_CASES = [
    (2, 1, 640, 320, 16, 16, 3, 3, (1, 1), (1, 1), (1, 1)),   # a UNet layer at batch 2 in small: 160 tiles, K 5760
    (2, 1, 320, 64, 8, 8, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 1, 256, 32, 6, 6, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 1, 512, 40, 5, 7, 2, 2, (1, 1), (0, 0), (1, 1)),      # ragged output channels
    (1, 1, 100, 16, 9, 12, 4, 8, (1, 1), (0, 0), (1, 1)),     # channels padded by the conversion kernels
    (2, 1, 384, 24, 6, 6, 3, 3, (2, 2), (1, 1), (1, 1)),
    (3, 1, 128, 72, 11, 9, 5, 5, (1, 2), (2, 2), (2, 1)),     # stride, dilation, 5x5
]


@pytest.mark.parametrize("case", SPLIT_CASES)
@pytest.mark.parametrize("layouts", [NHWC, NCHW, ("gyxck", "hwcgn", "hwkgn")], ids=["nhwc", "nchw", "hwcgn"])
@pytest.mark.parametrize("t", ["f32", "f16", "bf16", "i8"])
def test_conv_reduction_split_over_blocks_exact(rock, oracle, gpu, case, layouts, t):
    info = {}
    out, od, ref = _run(rock, oracle, gpu, t, *case, layouts, True, 59, info=info)
    if t == "i8":
        assert oracle.verify_int(out.cpu().numpy().ravel(), ref)[0] == 0
    else:
        # integer data: every partial sum is exact in f32; only the final narrowing rounds
        assert np.array_equal(to_f32(out, od), oracle.round_through(ref, CODE[od]))
    n, g, c, k, hi, wi, y, x, stride, pad, dil = case
    es = {"f32": 4, "i8": 1}.get(t, 2)
    ho = (hi + 2 * pad[0] - (y - 1) * dil[0] - 1) // stride[0] + 1
    wo = (wi + 2 * pad[1] - (x - 1) * dil[1] - 1) // stride[1] + 1
    kfull = -(-c * es // 16) * 16 // es * y * x
    want = min(1024 // (-(-n * ho * wo // 64) * -(-k // 64)), kfull // 1024)
    if any(kfull % d == 0 and (kfull // d) % (128 // es) == 0 for d in range(2, want + 1)):
        assert info["kernels"][-1] == "rock_reduce_splits" and info["kernels"][-2].startswith("rock_conv_")
    else:
        assert "rock_reduce_splits" not in info["kernels"]


def test_conv_reduction_split_real_values_and_declined_with_an_epilogue(rock, oracle, gpu):
    case = (2, 1, 640, 320, 16, 16, 3, 3, (1, 1), (1, 1), (1, 1))
    info = {}
    out, od, ref = _run(rock, oracle, gpu, "f16", *case, NHWC, False, 61, info=info)
    assert info["kernels"] == ["rock_conv_f16_64x64_fast", "rock_reduce_splits"]
    check_float(to_f32(out, od), ref, od)
    info = {}
    out, od, ref = _run(rock, oracle, gpu, "f16", *case, NHWC, False, 61, info=info, relu=True)
    assert len(info["kernels"]) == 1
