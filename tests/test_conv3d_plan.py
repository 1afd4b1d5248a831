"""Host-side check of the 3-D convolution plan, without a GPU: every kernel of
the plan is replayed in numpy from what the C ABI reports about it (kernel
name, pointer map, parameter block) -- the zero fill and the conversion
kernels element by element, the contraction as the 2-D convolution its
parameter block describes, computed by the CPU oracle over the replayed
workspace -- and the result is compared with the oracle's 3-D convolution.
This pins the unfolding of the depth taps into the channels (which slice goes
where, which output depths a tap reaches, the strides of the 2-D view) on the
CPU; the GPU tests then only have to show that the kernels do what their
parameter blocks say."""
import ctypes as C
import struct

import numpy as np
import pytest

from oracle import rock_oracle as orc

NCDHW = ("gkc012", "ngc012", "ngk012")
NDHWC = ("gk012c", "n012gc", "n012gk")
MIXED = ("g012ck", "n2g01c", "ngk201")

CASES = [
    (2, 1, 8, 16, (6, 7, 5), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    (2, 1, 3, 8, (9, 8, 7), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),
    (2, 2, 4, 6, (5, 6, 8), (2, 3, 3), (1, 2, 2), (0, 1, 2), (2, 1, 2)),
    (3, 1, 8, 8, (4, 4, 9), (1, 1, 5), (1, 1, 3), (0, 0, 2), (1, 1, 1)),
    (1, 1, 16, 8, (5, 5, 6), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),
]


def _options(case, layouts, t):
    n, g, c, k, ins, fs, stride, pad, dil = case
    s = ("--operation conv --arch gfx950 -t %s --fil_layout %s --in_layout %s --out_layout %s --batchsize %d"
         " --groupsize %d --in_channels %d --out_channels %d" % ((t,) + layouts + (n, g, g * c, g * k)))
    for a, ax in enumerate("hwd"):
        s += (" --in_%s %d --fil_%s %d --dilation_%s %d --conv_stride_%s %d --padding_%s %d"
              % (ax, ins[a], ax, fs[a], ax, dil[a], ax, stride[a], ax, pad[a]))
    return s


def _pointer_map(rock, k):
    ncall, nk = C.c_int(), C.c_int()
    src, off = (C.c_int32 * 8)(), (C.c_int64 * 8)()
    assert rock.load_library().rockamdGetPointerMap(k._h, C.byref(ncall), C.byref(nk), src, off) == 0
    return [(src[i], off[i]) for i in range(nk.value)]


def _replay_relayout(params, src, src_off, dst, dst_off):
    ss = struct.unpack_from("<5q", params, 0)
    ds = struct.unpack_from("<5q", params, 40)
    size = struct.unpack_from("<5i", params, 80)
    src_size = struct.unpack_from("<5i", params, 100)
    idx = np.indices(size).reshape(5, -1)
    inside = np.all(idx < np.array(src_size)[:, None], axis=0)
    so = src_off + (idx * np.array(ss)[:, None]).sum(0)
    do = dst_off + (idx * np.array(ds)[:, None]).sum(0)
    assert do.min() >= 0 and do.max() < dst.size and len(np.unique(do)) == do.size
    assert so[inside].min() >= 0 and so[inside].max() < src.size
    vals = np.zeros(do.size, dst.dtype)
    vals[inside] = src[so[inside]]
    dst[do] = vals


def _replay_conv(params, fil, fil_off, inp, in_off, out, out_off):
    st = struct.unpack_from("<15q", params, 0)
    n, g, c, k, hi, wi, y, x, ho, wo, sh, sw, ph, pw, dh, dw = struct.unpack_from("<16i", params, 120)
    in_s, fil_s, out_s = st[0:5], st[5:10], st[10:15]   # n g c h w / g k c y x / n g k h w

    def gather(buf, off, sizes, strides):
        idx = np.indices(sizes).reshape(len(sizes), -1)
        o = off + (idx * np.array(strides)[:, None]).sum(0)
        assert o.min() >= 0 and o.max() < buf.size
        return o

    xin = inp[gather(inp, in_off, (n, g, c, hi, wi), in_s)]
    f = fil[gather(fil, fil_off, (g, k, c, y, x), fil_s)]
    res, ho2, wo2 = orc.conv_fwd(f, xin, "gkcyx", "ngchw", "ngkhw", n, g, c, k, hi, wi, y, x, (sh, sw), (ph, pw),
                                 (dh, dw))
    # the right-hand padding is implied by the output extent the plan states
    assert (ho2, wo2) == (ho, wo) or ho <= ho2 + 1
    res = res.reshape(n, g, k, ho2, wo2)[:, :, :, :ho, :wo].ravel()
    o = gather(out, out_off, (n, g, k, ho, wo), out_s)
    assert len(np.unique(o)) == o.size
    out[o] = res


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
@pytest.mark.parametrize("t,es", [("f32", 4), ("f16", 2)])   # f16: channel runs padded to whole 16-byte chunks
def test_conv3d_plan_replayed_on_the_cpu(rock, case, layouts, t, es):
    n, g, c, k, ins, fs, stride, pad, dil = case
    rng = np.random.default_rng(5)
    fil = rng.integers(-3, 4, g * k * c * fs[0] * fs[1] * fs[2]).astype(np.float32)
    inp = rng.integers(-3, 4, n * g * c * ins[0] * ins[1] * ins[2]).astype(np.float32)
    want, outs = orc.conv3d(fil, inp, *layouts, n, g, c, k, ins, fs, stride, pad, dil)
    opts = _options(case, layouts, t)
    first = rock.RockKernel(opts)
    count = first.kernel_count
    assert first.workspace_bytes % es == 0
    out = np.full(want.size, np.nan, np.float32)
    ws = np.full(first.workspace_bytes // es, np.nan, np.float32)
    buffers = [fil, inp, out, None, ws]
    names = []
    for i in range(count):
        kern = first if i == 0 else rock.RockKernel(opts + " --kernel_id %d" % i)
        assert (kern.kernel_count, kern.workspace_bytes, kern.caller_pointers) == (count, first.workspace_bytes, 5)
        pm = _pointer_map(rock, kern)
        names.append(kern.kernel_name)
        if kern.kernel_name == "rock_fill_zero":
            (nbytes,) = struct.unpack_from("<q", kern.params(), 0)
            (src, off), = pm
            assert off % es == 0 and off + nbytes <= buffers[src].size * es
            buffers[src][off // es:(off + nbytes) // es] = 0
        elif kern.kernel_name.startswith("rock_relayout"):
            (s_src, s_off), (d_src, d_off) = pm
            _replay_relayout(kern.params(), buffers[s_src], s_off // es, buffers[d_src], d_off // es)
        else:
            assert kern.kernel_name.startswith("rock_conv_" + t)
            (f_src, f_off), (i_src, i_off), (o_src, o_off) = pm[:3]
            assert pm[3][0] == 3 and pm[4][0] == -1
            _replay_conv(kern.params(), buffers[f_src], f_off // es, buffers[i_src], i_off // es, buffers[o_src],
                         o_off // es)
    assert np.array_equal(out, want)
    assert sum(nm.startswith("rock_conv_") for nm in names) == 1
    with pytest.raises(rock.RockError, match="kernel_id out of range"):
        rock.RockKernel(opts + " --kernel_id %d" % count)


def test_conv3d_rejects_what_it_does_not_run(rock):
    opts = _options(CASES[0], NCDHW, "f16")
    with pytest.raises(rock.RockError, match="forward direction"):
        rock.RockKernel(opts.replace("--operation conv", "--operation conv_bwd_data"))
    with pytest.raises(rock.RockError, match="residual"):
        rock.RockKernel(opts + " --residual add")
    with pytest.raises(rock.RockError, match="layout"):
        rock.RockKernel(opts.replace("ngc012", "ngc01"))
    with pytest.raises(rock.RockError, match="smaller than the filter"):
        rock.RockKernel(opts.replace("--in_d 5", "--in_d 1").replace("--padding_d 1", "--padding_d 0"))


def test_conv3d_argument_info_has_six_dimensions(rock):
    n, g, c, k, ins, fs, stride, pad, dil = CASES[2]
    kern = rock.RockKernel(_options(CASES[2], MIXED, "f16"))
    outs = [orc.conv_out_dim(ins[a], fs[a], pad[a], pad[a], stride[a], dil[a]) for a in range(3)]
    args = kern.arguments()
    # filter g012ck, input n2g01c, output ngk201, bias, workspace
    assert args[0] == (1, [g, fs[0], fs[1], fs[2], c, k])
    assert args[1] == (1, [n, ins[2], g, ins[0], ins[1], c])
    assert args[2] == (1, [n, g, k, outs[2], outs[0], outs[1]])
    assert args[3] == (0, [g * k]) and args[4] == (-1, [kern.workspace_bytes])
    keys = [rock.RockKernel(_options(CASES[2], MIXED, "f16") + " --kernel_id %d" % i).problem_key
            for i in range(kern.kernel_count)]
    # the contraction kernel carries the tuning key: the reference's 2-D fields, then the depth's
    assert sum("--in_d 8 --fil_d 3 --padding_d 2 --conv_stride_d 2 --dilation_d 2" in key for key in keys) == 1
