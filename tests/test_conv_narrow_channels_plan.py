"""Filter gradient of convolutions over images with a few channels (the
3-channel first layer of a CNN): the plan -- a channels-last copy with the
channel run padded to a fraction of a 16-byte chunk, the K-major GEMM over
rows of filter taps read as one run, the reduction that leaves the padding
columns out -- replayed kernel by kernel in numpy from the parameter blocks and
pointer maps the C ABI hands out, against the CPU oracle.  The workspace
starts as NaN, so a kernel that used a byte no earlier kernel wrote, outside
the padding columns, would show."""
import struct

import numpy as np
import pytest

from oracle import rock_oracle as orc
from tests.test_conv3d_plan import _replay_plan
from tests.test_relayout_host import conv

# (n c k hi wi y x stride pad_h) -- no padding along w, even image width
CASES = [
    (2, 3, 16, 20, 20, 7, 7, 2, 0),    # the ResNet first layer in small
    (3, 3, 64, 15, 18, 3, 3, 2, 1),    # rows padded at the top and bottom
    (2, 4, 24, 12, 16, 5, 3, 2, 2),    # four channels: no channel padding, rows of 3 taps
    (2, 2, 8, 9, 16, 3, 5, 4, 0),      # two channels (a quarter of a chunk), stride 4
    (1, 1, 8, 10, 24, 3, 3, 8, 1),     # one channel
]


def _options(case, il, fl, t):
    n, c, k, hi, wi, y, x, s, ph = case
    ho = (hi + 2 * ph - y) // s + 1
    wo = (wi - x) // s + 1
    return (conv(t, il, fl, n, c, hi, wi, k, y, x, stride=s, op="conv_bwd_weight")
            .replace("--padding_h 0", "--padding_h %d" % ph).replace("--out_h %d" % ((hi - y) // s + 1), "--out_h %d" % ho)), ho, wo


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("il,fl", [("nhwgc", "gkyxc"), ("ngchw", "gkcyx"), ("nhwgc", "gkcyx")])
@pytest.mark.parametrize("t,es", [("fp16", 2), ("f32", 4)])
def test_narrow_channel_filter_gradient_plan_replayed_on_the_cpu(rock, case, il, fl, t, es):
    n, c, k, hi, wi, y, x, s, ph = case
    if es == 4 and c == 4:
        pytest.skip("four 32-bit channels are a whole chunk: the channels-last route takes it")
    opts, ho, wo = _options(case, il, fl, t)
    ol = il.replace("c", "k")
    rng = np.random.default_rng(11)
    inp = rng.integers(-3, 4, n * c * hi * wi).astype(np.float32)
    dout = rng.integers(-3, 4, n * k * ho * wo).astype(np.float32)
    want, _, _ = orc.conv_bwd_weight(inp, dout, fl, il, ol, n, 1, c, k, hi, wi, y, x, (s, s), (ph, 0), (1, 1))
    first = rock.RockKernel(opts)
    dw = np.full(want.size, np.nan, np.float32)
    ws = np.full(first.workspace_bytes // es, np.nan, np.float32)
    tn = {"fp16": "f16"}.get(t, t)
    names = _replay_plan(rock, opts, [dw, inp, dout, None, ws], tn, es)
    assert np.array_equal(dw, want.ravel())
    copies = 1 if il == "nhwgc" else 2
    assert names == ["rock_relayout_b%d" % es] * copies + ["rock_conv_bwd_weight_%s_64x64" % tn, "rock_reduce_splits"]


FWD_CASES = [
    # (type, element size, n c k hi wi y x stride pad_h): no padding along w, rows of whole chunks
    ("fp16", 2, (2, 3, 16, 20, 20, 7, 7, 2, 0)),    # the ResNet first layer in small: 3 -> 4 channels, run of 28 in 32
    ("fp16", 2, (2, 3, 72, 15, 18, 3, 3, 2, 1)),    # run of 12 in 16; rows padded at the top and bottom
    ("fp16", 2, (2, 2, 8, 9, 16, 3, 5, 4, 0)),      # 2 channels: run of 10 in 16
    ("fp16", 2, (2, 4, 24, 12, 16, 4, 4, 2, 2)),    # 4 taps of 4 channels: whole chunks, no kernel of its own needed
    ("i8", 1, (2, 3, 16, 20, 20, 7, 7, 2, 0)),      # 8-bit: 3 -> 8 channels, run of 56 in 64
    ("i8", 1, (1, 1, 8, 10, 24, 3, 3, 4, 1)),
]


@pytest.mark.parametrize("t,es,case", FWD_CASES)
@pytest.mark.parametrize("il,fl", [("nhwgc", "gkyxc"), ("ngchw", "gkcyx")])
def test_rows_of_taps_forward_plan_replayed_on_the_cpu(rock, t, es, case, il, fl):
    n, c, k, hi, wi, y, x, s, ph = case
    opts, ho, wo = _options(case, il, fl, t)
    opts = opts.replace("--operation conv_bwd_weight", "--operation conv")
    ol = il.replace("c", "k")
    rng = np.random.default_rng(12)
    fil = rng.integers(-3, 4, k * c * y * x).astype(np.float32)
    inp = rng.integers(-3, 4, n * c * hi * wi).astype(np.float32)
    want, _, _ = orc.conv_fwd(fil, inp, fl, il, ol, n, 1, c, k, hi, wi, y, x, (s, s), (ph, 0), (1, 1))
    first = rock.RockKernel(opts)
    out = np.full(want.size, np.nan, np.float32)
    ws = np.full(first.workspace_bytes // es, np.nan, np.float32)
    tn = {"fp16": "f16"}.get(t, t)
    names = _replay_plan(rock, opts, [fil, inp, out, None, ws], tn, es)
    assert np.array_equal(out, want.ravel())
    whole = (x * max(c, 4 // es) * es) % 16 == 0 and t == "fp16"
    assert names == ["rock_relayout_b%d" % es] * 2 + ["rock_conv_%s_64x64_fast%s" % (tn, "" if whole else "_runs")]
    # the contraction reduces over rows of taps: K = y * run
    import struct
    conv_k = rock.RockKernel(opts + " --kernel_id 2")
    cc, xx = struct.unpack_from("<i", conv_k.params(), 128)[0], struct.unpack_from("<i", conv_k.params(), 148)[0]
    assert xx == 1 and (cc * es) % 16 == 0 and cc * es < x * 16


def test_narrow_channel_route_conditions(rock):
    """Padding or dilation along w, an odd image width, or a switch decline the route."""
    base, _, _ = _options(CASES[0], "nhwgc", "gkyxc", "fp16")
    names = lambda o: [rock.RockKernel(o + " --kernel_id %d" % i).kernel_name for i in range(rock.RockKernel(o).kernel_count)]
    assert names(base)[-2:] == ["rock_conv_bwd_weight_f16_64x64", "rock_reduce_splits"]
    for change in (("--padding_w 0", "--padding_w 1 --out_w 8"), ("--in_w 20 --out_h 7 --out_w 7", "--in_w 21 --out_h 7 --out_w 8"),
                   ("--dilation_w 1", "--dilation_w 2 --out_w 4")):
        assert not any(nm.startswith("rock_conv_bwd_weight_") for nm in names(base.replace(*change))), change
    assert not any(nm.startswith("rock_conv_bwd_weight_") for nm in names(base + " --bwd_weight_gemm false"))
    fwd = base.replace("--operation conv_bwd_weight", "--operation conv")
    assert names(fwd)[-1] == "rock_conv_f16_64x64_fast_runs"
    for change in (("--padding_w 0", "--padding_w 1 --out_w 8"), ("--in_w 20 --out_h 7 --out_w 7", "--in_w 21 --out_h 7 --out_w 8"),
                   ("--dilation_w 1", "--dilation_w 2 --out_w 4"), ("--conv_stride_w 2", "--conv_stride_w 1 --out_w 14"),
                   ("--padding_w 0 ", "--padding_w 0 --tap_rows false")):
        assert not names(fwd.replace(*change))[-1].endswith("_runs"), change


SPLIT_CASES = [
    # (n c k hi wi y x stride pad): few output tiles, a long reduction
    (2, 320, 64, 8, 8, 3, 3, 1, 1),      # K = 2880: halves of 1440 are whole K-steps of 32-bit elements only
    (1, 256, 32, 6, 6, 3, 3, 1, 1),      # K = 2304
    (2, 512, 40, 5, 7, 2, 2, 1, 0),      # K = 2048, ragged output channels
    (1, 100, 16, 9, 12, 4, 8, 1, 0),     # 16-bit channels padded to 104 by the conversion: K = 3328
    (2, 384, 24, 6, 6, 3, 3, 2, 1),      # K = 3456: three shares
]


@pytest.mark.parametrize("case", SPLIT_CASES)
@pytest.mark.parametrize("il,fl", [("nhwgc", "gkyxc"), ("ngchw", "gkcyx")])
@pytest.mark.parametrize("t,es", [("fp16", 2), ("f32", 4), ("i8", 1)])
def test_forward_reduction_split_plan_replayed_on_the_cpu(rock, case, il, fl, t, es):
    n, c, k, hi, wi, y, x, s, pd = case
    opts = conv(t, il, fl, n, c, hi, wi, k, y, x, stride=s, pad=pd)
    ol = il.replace("c", "k")
    rng = np.random.default_rng(13)
    fil = rng.integers(-3, 4, k * c * y * x).astype(np.float32)
    inp = rng.integers(-3, 4, n * c * hi * wi).astype(np.float32)
    want, ho, wo = orc.conv_fwd(fil, inp, fl, il, ol, n, 1, c, k, hi, wi, y, x, (s, s), (pd, pd), (1, 1))
    first = rock.RockKernel(opts)
    c_chunks = -(-c * es // 16) * 16 // es
    kfull, tiles = c_chunks * y * x, -(-n * ho * wo // 64) * -(-k // 64)
    most = min(1024 // tiles, kfull // 1024)
    splits = [d for d in range(most, 1, -1) if kfull % d == 0 and (kfull // d) % (128 // es) == 0]
    if first.kernel_count == 1:   # the tensors as they lie and no share of whole K-steps: one kernel, nothing to replay
        assert not splits
        return
    out = np.full(want.size, np.nan, np.float32)
    ws = np.full(max(first.workspace_bytes // es, 1), np.nan, np.float32)
    tn = {"fp16": "f16"}.get(t, t)
    names = _replay_plan(rock, opts, [fil, inp, out, None, ws], tn, es)
    assert np.array_equal(out, want.ravel())
    if splits:
        assert struct.unpack_from("<i", rock.RockKernel("%s --kernel_id %d" % (opts, len(names) - 2)).params(), 124)[0] == splits[0]
        assert names[-1] == "rock_reduce_splits" and names[-2].startswith("rock_conv_%s_" % tn)
        # an epilogue that does not commute with the sum, or the switch, keeps the single contraction kernel
        other = " --zero_point 3" if t == "i8" else " --relu true"
        assert rock.RockKernel(opts + other).kernel_count == first.kernel_count - 1
        assert rock.RockKernel(opts + " --split_k false").kernel_count == first.kernel_count - 1
    else:
        assert "rock_reduce_splits" not in names


# (n c k hi wi y x stride pad): an output gradient with a few channels
NARROW_K_CASES = [
    (2, 32, 4, 12, 12, 3, 3, 1, 1),      # a layer that ends in 4 channels
    (3, 16, 3, 9, 11, 3, 3, 2, 1),
    (2, 64, 12, 8, 8, 5, 5, 1, 2),       # 12 channels: one and a half chunks of 16 bits
    (1, 8, 1, 10, 10, 2, 2, 1, 0),
]


@pytest.mark.parametrize("case", NARROW_K_CASES)
@pytest.mark.parametrize("il,fl", [("nhwgc", "gkyxc"), ("ngchw", "gkcyx")])
@pytest.mark.parametrize("t,es", [("fp16", 2), ("f32", 4)])
def test_filter_gradient_of_a_narrow_output_gradient_replayed_on_the_cpu(rock, case, il, fl, t, es):
    n, c, k, hi, wi, y, x, s, pd = case
    if (c * es) % 16 or (k * es) % 16 == 0:
        pytest.skip("not this route")
    opts = conv(t, il, fl, n, c, hi, wi, k, y, x, stride=s, pad=pd, op="conv_bwd_weight")
    ol = il.replace("c", "k")
    ho, wo = (hi + 2 * pd - y) // s + 1, (wi + 2 * pd - x) // s + 1
    rng = np.random.default_rng(14)
    inp = rng.integers(-3, 4, n * c * hi * wi).astype(np.float32)
    dout = rng.integers(-3, 4, n * k * ho * wo).astype(np.float32)
    want, _, _ = orc.conv_bwd_weight(inp, dout, fl, il, ol, n, 1, c, k, hi, wi, y, x, (s, s), (pd, pd), (1, 1))
    first = rock.RockKernel(opts)
    dw = np.full(want.size, np.nan, np.float32)
    ws = np.full(first.workspace_bytes // es, np.nan, np.float32)
    tn = {"fp16": "f16"}.get(t, t)
    names = _replay_plan(rock, opts, [dw, inp, dout, None, ws], tn, es)
    assert np.array_equal(dw, want.ravel())
    assert names[0].startswith("rock_relayout_b") and names[-2:] == ["rock_conv_bwd_weight_%s_64x64" % tn, "rock_reduce_splits"]
    # a kernel_id behind the plan is an error, not another plan
    with pytest.raises(rock.RockError):
        rock.RockKernel(opts + " --kernel_id %d" % len(names))


# (n c k hi wi y x pad): unit stride, few tiles, k * taps >= 2048
BWD_DATA_SPLIT_CASES = [
    (2, 64, 256, 8, 8, 3, 3, 1),
    (1, 40, 512, 6, 7, 2, 2, 0),       # ragged channels of the input gradient
    (2, 24, 100, 5, 5, 5, 5, 2),       # 16-bit k padded to 104 by the conversion of the output gradient
    (2, 128, 384, 6, 6, 3, 3, 1),      # three shares
]


@pytest.mark.parametrize("case", BWD_DATA_SPLIT_CASES)
@pytest.mark.parametrize("il,fl", [("nhwgc", "gkyxc"), ("ngchw", "gkcyx")])
@pytest.mark.parametrize("t,es", [("fp16", 2), ("f32", 4)])
def test_backward_data_reduction_split_plan_replayed_on_the_cpu(rock, case, il, fl, t, es):
    n, c, k, hi, wi, y, x, pd = case
    opts = conv(t, il, fl, n, c, hi, wi, k, y, x, stride=1, pad=pd, op="conv_bwd_data")
    ol = il.replace("c", "k")
    ho, wo = hi + 2 * pd - y + 1, wi + 2 * pd - x + 1
    rng = np.random.default_rng(15)
    fil = rng.integers(-3, 4, k * c * y * x).astype(np.float32)
    dout = rng.integers(-3, 4, n * k * ho * wo).astype(np.float32)
    want, _, _ = orc.conv_bwd_data(fil, dout, fl, il, ol, n, 1, c, k, hi, wi, y, x, (1, 1), (pd, pd), (1, 1))
    first = rock.RockKernel(opts)
    dx = np.full(want.size, np.nan, np.float32)
    ws = np.full(first.workspace_bytes // es, np.nan, np.float32)
    tn = {"fp16": "f16"}.get(t, t)
    names = _replay_plan(rock, opts, [fil, dx, dout, None, ws], tn, es)
    assert np.array_equal(dx, want.ravel())
    kfull = -(-k * es // 16) * 16 // es * y * x
    most = min(1024 // (-(-n * hi * wi // 64) * -(-c // 64)), kfull // 1024)
    if any(kfull % d == 0 and (kfull // d) % (128 // es) == 0 for d in range(2, most + 1)):
        assert names[-1] == "rock_reduce_splits" and names[-2].startswith("rock_conv_%s_" % tn)
        assert rock.RockKernel(opts + " --split_k false").kernel_count == first.kernel_count - 1
    else:
        assert "rock_reduce_splits" not in names


def test_program_reports_its_contraction_kernel(rock):
    """A plan that ends in the reduction kernel still answers with the contraction kernel's name, perf_config
    and problem key (what the tuner records)."""
    opts = conv("fp16", "nhwgc", "gkyxc", 2, 640, 16, 16, 320, 3, 3, pad=1)
    prog = rock.RockProgram(opts)
    assert [k.kernel_name for k in prog.kernels][-1] == "rock_reduce_splits"
    assert prog.kernel_name.startswith("rock_conv_f16_") and prog.perf_config.startswith("v2:")
    assert "convfp16" in prog.problem_key and " -c 640 " in prog.problem_key


# (n, c, k, hi, wi, y, x, stride, pad)
MERGED_PHASE_CASES = [
    (2, 3, 8, 20, 16, 7, 7, 2, 0),    # the first layer's shape in small: windows of 4 and 3 taps
    (2, 3, 8, 16, 16, 7, 7, 2, 3),    # padded: the phases start at different rows
    (1, 4, 16, 12, 12, 3, 3, 2, 1),
    (1, 2, 8, 12, 18, 5, 5, 3, 2),    # nine phases
    (2, 16, 8, 8, 8, 3, 3, 2, 1),     # 64 merged columns
    (1, 3, 5, 12, 12, 3, 3, 2, 1),    # k padded to whole chunks
]


@pytest.mark.parametrize("t,es", [("fp16", 2), ("f32", 4)])
@pytest.mark.parametrize("il,fl", [("nhwgc", "gkyxc"), ("ngchw", "gkcyx")])
@pytest.mark.parametrize("case", MERGED_PHASE_CASES)
def test_backward_data_merged_phases_plan_replayed_on_the_cpu(rock, case, il, fl, t, es):
    """A strided layer with few input channels computes all its phases in one convolution with (phase, channel)
    output columns; a conversion kernel interleaves them into the input gradient."""
    n, c, k, hi, wi, y, x, st, pd = case
    ho, wo = (hi + 2 * pd - y) // st + 1, (wi + 2 * pd - x) // st + 1
    opts = conv(t, il, fl, n, c, hi, wi, k, y, x, stride=st, pad=pd, op="conv_bwd_data")
    ol = il.replace("c", "k")
    rng = np.random.default_rng(16)
    fil = rng.integers(-3, 4, k * c * y * x).astype(np.float32)
    dout = rng.integers(-3, 4, n * k * ho * wo).astype(np.float32)
    want, _, _ = orc.conv_bwd_data(fil, dout, fl, il, ol, n, 1, c, k, hi, wi, y, x, (st, st), (pd, pd), (1, 1))
    first = rock.RockKernel(opts)
    dx = np.full(want.size, np.nan, np.float32)
    ws = np.full(first.workspace_bytes // es, np.nan, np.float32)
    tn = {"fp16": "f16"}.get(t, t)
    names = _replay_plan(rock, opts, [fil, dx, dout, None, ws], tn, es)
    assert np.array_equal(dx, want.ravel())
    assert sum(nm.startswith("rock_conv_") for nm in names) == 1 and names.count("rock_fill_zero") == 1
    # switched off: one convolution per phase
    off = rock.RockKernel(opts + " --merge_phases false")
    names_off = [rock.RockKernel(opts + " --merge_phases false --kernel_id %d" % i).kernel_name
                 for i in range(off.kernel_count)]
    assert sum(nm.startswith("rock_conv_") for nm in names_off) == st * st


@pytest.mark.parametrize("extra,why", [
    (dict(c=32), "too many merged columns"),
    (dict(hi=15), "phases of different sizes"),
    (dict(dilation=2), "dilated"),
])
def test_backward_data_merged_phases_declined(rock, extra, why):
    kw = dict(c=3, hi=16, dilation=1)
    kw.update(extra)
    opts = conv("fp16", "nhwgc", "gkyxc", 2, kw["c"], kw["hi"], 16, 8, 3, 3, stride=2, pad=1, op="conv_bwd_data")
    if kw["dilation"] != 1:  # same output size: (16 + 2*2 - 5) // 2 + 1 == 8
        opts = opts.replace("--dilation_h 1 --dilation_w 1", "--dilation_h 2 --dilation_w 2").replace(
            "--padding_h 1 --padding_w 1", "--padding_h 2 --padding_w 2")
    first = rock.RockKernel(opts)
    names = [rock.RockKernel(opts + " --kernel_id %d" % i).kernel_name for i in range(first.kernel_count)]
    off = opts + " --merge_phases false"
    assert names == [rock.RockKernel(off + " --kernel_id %d" % i).kernel_name
                     for i in range(rock.RockKernel(off).kernel_count)], why
