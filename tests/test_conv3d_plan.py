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


def _replay_split_conv(params, fil, fil_off, inp, in_off, out, out_off, es):
    """A one-group convolution whose reduction is split over its groups (k_group_stride): group s
    reduces the elements [s * K, (s + 1) * K) of the (tap, channel) index into its own f32 result."""
    st = struct.unpack_from("<15q", params, 0)
    n, S, c, k, hi, wi, y, x, ho, wo, sh, sw, ph, pw, dh, dw = struct.unpack_from("<16i", params, 120)
    (K,) = struct.unpack_from("<i", params, 192)
    (stride,) = struct.unpack_from("<i", params, 308)
    (out_dtype,) = struct.unpack_from("<i", params, 244)
    in_s, fil_s, out_s = st[0:5], st[5:10], st[10:15]
    assert stride == K and S * K == c * y * x and in_s[1] == 0 and fil_s[0] == K and out_dtype in (0, 6)  # f32, i32
    kk = np.arange(c * y * x)
    tap, ch = kk // c, kk % c
    ty, tx = tap // x, tap % x
    pix = np.arange(n * ho * wo)
    nn, oh, ow = pix // (ho * wo), (pix // wo) % ho, pix % wo
    ih = oh[:, None] * sh + ty[None, :] * dh - ph
    iw = ow[:, None] * sw + tx[None, :] * dw - pw
    ok = (ih >= 0) & (ih < hi) & (iw >= 0) & (iw < wi)
    src = in_off + nn[:, None] * in_s[0] + ih * in_s[3] + iw * in_s[4] + ch[None, :] * in_s[2]
    assert src[ok].min() >= 0 and src[ok].max() < inp.size
    a = np.where(ok, inp[np.where(ok, src, 0)], 0).astype(np.float64)
    fsrc = fil_off + np.arange(k)[:, None] * fil_s[1] + ty[None, :] * fil_s[3] + tx[None, :] * fil_s[4] + ch[None, :] * fil_s[2]
    assert fsrc.min() >= 0 and fsrc.max() < fil.size
    b = fil[fsrc].astype(np.float64)
    wide = 4 // es
    for sp in range(S):
        part = a[:, sp * K:(sp + 1) * K] @ b[:, sp * K:(sp + 1) * K].T
        assert not np.isnan(part).any()
        o = out_off + wide * (sp * out_s[1] + nn[:, None] * out_s[0] + oh[:, None] * out_s[3] + ow[:, None] * out_s[4]
                              + np.arange(k)[None, :] * out_s[2])
        assert o.min() >= 0 and o.max() + wide - 1 < out.size and len(np.unique(o)) == o.size
        out[o] = part
        for extra in range(1, wide):   # the value sits in the first of the elements it covers
            out[o + extra] = np.nan


def _replay_conv(params, fil, fil_off, inp, in_off, out, out_off, es=None):
    st = struct.unpack_from("<15q", params, 0)
    n, g, c, k, hi, wi, y, x, ho, wo, sh, sw, ph, pw, dh, dw = struct.unpack_from("<16i", params, 120)
    in_s, fil_s, out_s = st[0:5], st[5:10], st[10:15]   # n g c h w / g k c y x / n g k h w
    if struct.unpack_from("<i", params, 308)[0]:
        return _replay_split_conv(params, fil, fil_off, inp, in_off, out, out_off, es)

    def gather(buf, off, sizes, strides):
        idx = np.indices(sizes).reshape(len(sizes), -1)
        o = off + (idx * np.array(strides)[:, None]).sum(0)
        assert o.min() >= 0 and o.max() < buf.size
        return o

    xin = inp[gather(inp, in_off, (n, g, c, hi, wi), in_s)].reshape(n, g, c, hi, wi).astype(np.float64)
    (run_valid,) = struct.unpack_from("<i", params, 304)
    if run_valid:  # "_runs" kernels: what a channel run holds behind its data is cleared before it is multiplied
        xin[:, :, run_valid:] = 0
    f = fil[gather(fil, fil_off, (g, k, c, y, x), fil_s)].reshape(g, k, c, y, x).astype(np.float64)
    if (ho, wo) == (orc.conv_out_dim(hi, y, ph, ph, sh, dh), orc.conv_out_dim(wi, x, pw, pw, sw, dw)):
        # symmetric padding: the 2-D convolution of the CPU oracle
        res, _, _ = orc.conv_fwd(f.ravel(), xin.ravel(), "gkcyx", "ngchw", "ngkhw", n, g, c, k, hi, wi, y, x,
                                 (sh, sw), (ph, pw), (dh, dw))
    else:
        # any output extent (the right-hand padding is implied by it): tap by tap, zero outside the input
        acc = np.zeros((n, g, k, ho, wo))
        for ty in range(y):
            ih = np.arange(ho) * sh + ty * dh - ph
            for tx in range(x):
                iw = np.arange(wo) * sw + tx * dw - pw
                ok = ((ih >= 0) & (ih < hi))[:, None] & ((iw >= 0) & (iw < wi))[None, :]
                win = xin[:, :, :, np.clip(ih, 0, hi - 1)][:, :, :, :, np.clip(iw, 0, wi - 1)] * ok
                acc += np.einsum("ngcab,gkc->ngkab", win, f[:, :, :, ty, tx])
        res = acc.astype(np.float32).ravel()
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
            # a kernel that moves words of several elements: once per element of the word
            wide = int(kern.kernel_name[len("rock_relayout_b"):]) // es
            assert wide >= 1 and s_off % (es * wide) == 0 and d_off % (es * wide) == 0
            for part in range(wide):
                _replay_relayout(kern.params(), buffers[s_src][part::wide], s_off // (es * wide),
                                 buffers[d_src][part::wide], d_off // (es * wide))
        else:
            assert kern.kernel_name.startswith("rock_conv_" + t)
            (f_src, f_off), (i_src, i_off), (o_src, o_off) = pm[:3]
            assert pm[3][0] == 3 and pm[4][0] == -1
            _replay_conv(kern.params(), buffers[f_src], f_off // es, buffers[i_src], i_off // es, buffers[o_src],
                         o_off // es, es)
    assert np.array_equal(out, want)
    assert sum(nm.startswith("rock_conv_") for nm in names) == 1
    with pytest.raises(rock.RockError, match="kernel_id out of range"):
        rock.RockKernel(opts + " --kernel_id %d" % count)


def test_conv3d_rejects_what_it_does_not_run(rock):
    opts = _options(CASES[0], NCDHW, "f16")
    with pytest.raises(rock.RockError, match="f32, f16 or bf16"):
        rock.RockKernel(opts.replace("--operation conv", "--operation conv_bwd_data").replace("-t f16", "-t i8"))
    with pytest.raises(rock.RockError, match="symmetric padding"):
        rock.RockKernel(opts.replace("--operation conv", "--operation conv_bwd_weight") + " --padding_d_r 0")
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


# ---- the gradients -----------------------------------------------------------
def _replay_fold(params, T, t_off, dst, d_off):
    ds = struct.unpack_from("<6q", params, 0)
    (t_pix,) = struct.unpack_from("<q", params, 48)
    n, g, c, cp, hi, wi, di, d_out, Z, sd, dd, pd, dtype, _ = struct.unpack_from("<14i", params, 56)
    idx = np.indices((n, g, c, hi, wi, di)).reshape(6, -1)
    nn, gg, cc, hh, ww, dn = idx
    acc = np.zeros(idx.shape[1], np.float64)
    for z in range(Z):
        num = dn + pd - z * dd
        od = num // sd
        ok = (num >= 0) & (num % sd == 0) & (od < d_out)
        src = t_off + (((nn * d_out + od) * hi + hh) * wi + ww) * t_pix + (gg * Z + z) * cp + cc
        assert src[ok].size == 0 or (src[ok].min() >= 0 and src[ok].max() < T.size)
        vals = T[np.where(ok, src, 0)]
        assert not np.isnan(vals[ok]).any()
        acc += np.where(ok, vals, 0)
    o = d_off + (idx * np.array(ds)[:, None]).sum(0)
    assert o.min() >= 0 and o.max() < dst.size and len(np.unique(o)) == o.size
    dst[o] = acc


def _replay_plan(rock, opts, buffers, t, es):
    """Runs every kernel of the plan in numpy on `buffers` (the caller's pointer
    list, the workspace last, as flat f32 arrays of elements); returns the
    kernel names.  Skips when the plan holds a kernel this file cannot replay
    from its parameter block."""
    first = rock.RockKernel(opts)
    count = first.kernel_count
    names = []
    for i in range(count):
        kern = first if i == 0 else rock.RockKernel(opts + " --kernel_id %d" % i)
        assert (kern.kernel_count, kern.workspace_bytes, kern.caller_pointers) == (count, first.workspace_bytes, 5)
        pm = _pointer_map(rock, kern)
        name = kern.kernel_name
        names.append(name)
        if name == "rock_fill_zero":
            (nbytes,) = struct.unpack_from("<q", kern.params(), 0)
            (src, off), = pm
            assert off % es == 0 and off + nbytes <= buffers[src].size * es
            buffers[src][off // es:(off + nbytes) // es] = 0
        elif name.startswith("rock_relayout_b"):
            (s_src, s_off), (d_src, d_off) = pm
            # a kernel that moves words of several elements: once per element of the word
            wide = int(kern.kernel_name[len("rock_relayout_b"):]) // es
            assert wide >= 1 and s_off % (es * wide) == 0 and d_off % (es * wide) == 0
            for part in range(wide):
                _replay_relayout(kern.params(), buffers[s_src][part::wide], s_off // (es * wide),
                                 buffers[d_src][part::wide], d_off // (es * wide))
        elif name == "rock_fold_depth":
            (s_src, s_off), (d_src, d_off) = pm
            _replay_fold(kern.params(), buffers[s_src], s_off // es, buffers[d_src], d_off // es)
        elif name.startswith("rock_conv_" + t + "_"):
            (f_src, f_off), (i_src, i_off), (o_src, o_off) = pm[:3]
            _replay_conv(kern.params(), buffers[f_src], f_off // es, buffers[i_src], i_off // es, buffers[o_src],
                         o_off // es, es)
        elif name.startswith("rock_conv_bwd_weight_"):
            (y_src, y_off), (x_src, x_off), (w_src, w_off) = pm[:3]
            _replay_bwd_weight_gemm(kern.params(), buffers[y_src], y_off // es, buffers[x_src], x_off // es,
                                    buffers[w_src], w_off // es, es)
        elif name == "rock_reduce_splits":
            (s_src, s_off), (d_src, d_off) = pm
            _replay_reduce(kern.params(), buffers[s_src], s_off // es, buffers[d_src], d_off // es, es)
        elif name.startswith("rock_gemm_" + t + "_"):
            (a_src, a_off), (b_src, b_off), (c_src, c_off) = pm[:3]
            _replay_gemm(kern.params(), buffers[a_src], a_off // es, buffers[b_src], b_off // es, buffers[c_src],
                         c_off // es)
        else:
            pytest.skip("no numpy replay of " + name)
    return names


def _replay_gemm(params, A, a_off, B, b_off, Cm, c_off):
    """rock_gemm_*: C[g, m, n] = sum over k of A[g, m, k] * B[g, n, k] through the
    element strides of the parameter block (identity epilogue, result in the operands' type)."""
    a_gs, a_ms, a_ks, b_gs, b_ns, b_ks, c_gs, c_ms, c_ns = struct.unpack_from("<9q", params, 0)
    G, M, N, K = struct.unpack_from("<4i", params, 72)
    scale, _, _, _, has_bias, out_dtype, act, res_op = struct.unpack_from("<2f6i", params, 104)
    assert (scale, has_bias, act, res_op) == (1.0, 0, 0, 0)
    for g in range(G):
        ia = a_off + g * a_gs + np.arange(M)[:, None] * a_ms + np.arange(K)[None, :] * a_ks
        ib = b_off + g * b_gs + np.arange(N)[:, None] * b_ns + np.arange(K)[None, :] * b_ks
        assert ia.min() >= 0 and ia.max() < A.size and ib.min() >= 0 and ib.max() < B.size
        prod = A[ia].astype(np.float64) @ B[ib].astype(np.float64).T
        assert not np.isnan(prod).any()
        o = c_off + g * c_gs + np.arange(M)[:, None] * c_ms + np.arange(N)[None, :] * c_ns
        assert o.min() >= 0 and o.max() < Cm.size
        Cm[o] = prod


# f32 partial sums inside a workspace counted in 2-byte elements: the value sits in the first of
# the two elements it covers, the second holds NaN (nothing may read it)
def _replay_bwd_weight_gemm(params, dy, dy_off, xin, x_off, dst, d_off, es):
    """rock_conv_bwd_weight_*: C[s][k][(y, x, c)] = sum over the pixels of split s
    of dY[pixel][k] * X[n, ho*sh + y*dh - ph, wo*sw + x*dw - pw, c]."""
    (out_dtype,) = struct.unpack_from("<i", params, 124)
    wide = 4 // es if out_dtype == 0 else 1
    a_gs, a_ms, a_ks, _, _, _, c_gs, c_ms, c_ns = struct.unpack_from("<9q", params, 0)
    S, M, N, K = struct.unpack_from("<4i", params, 72)
    (pix_stride,) = struct.unpack_from("<q", params, 184)
    c, hi, wi, ho, wo, X, sh, sw, ph, pw, dh, dw = struct.unpack_from("<12i", params, 192)
    cols = np.arange(N)
    tap, cc = cols // c, cols % c
    ty, tx = tap // X, tap % X
    for sp in range(S):
        pix = sp * K + np.arange(K)
        nn, oh, ow = pix // (ho * wo), (pix // wo) % ho, pix % wo
        ih = oh[:, None] * sh + ty[None, :] * dh - ph
        iw = ow[:, None] * sw + tx[None, :] * dw - pw
        ok = (ih >= 0) & (ih < hi) & (iw >= 0) & (iw < wi)
        src = x_off + ((nn[:, None] * hi + ih) * wi + iw) * pix_stride + cc[None, :]
        assert src[ok].min() >= 0 and src[ok].max() < xin.size
        im2col = np.where(ok, xin[np.where(ok, src, 0)], 0).astype(np.float64)
        ysrc = dy_off + pix[:, None] * a_ks + np.arange(M)[None, :] * a_ms
        assert ysrc.min() >= 0 and ysrc.max() < dy.size
        # (columns that are padding may hold anything, NaN included: the reduction leaves them out)
        part = dy[ysrc].astype(np.float64).T @ im2col
        o = d_off + wide * (sp * c_gs + np.arange(M)[:, None] * c_ms + cols[None, :] * c_ns)
        assert o.min() >= 0 and o.max() + wide - 1 < dst.size
        dst[o] = part
        if wide > 1:
            dst[o + 1] = np.nan


def _replay_reduce(params, parts, p_off, dst, d_off, es):
    (split_stride,) = struct.unpack_from("<q", params, 0)
    ds = struct.unpack_from("<4q", params, 8)
    size = struct.unpack_from("<4i", params, 40)
    splits, _ = struct.unpack_from("<2i", params, 56)
    valid = [v or s for v, s in zip(struct.unpack_from("<4i", params, 64), size)]  # 0: the whole dimension
    total = int(np.prod(size))
    acc = np.zeros(total, np.float64)
    wide = 4 // es
    for sp in range(splits):
        acc += parts[p_off + wide * (sp * split_stride + np.arange(total))]
    idx = np.indices(size).reshape(4, -1)
    keep = np.all(idx < np.array(valid)[:, None], axis=0)
    assert not np.isnan(acc[keep]).any()
    o = d_off + (idx * np.array(ds)[:, None]).sum(0)[keep]
    assert o.min() >= 0 and o.max() < dst.size and len(np.unique(o)) == o.size
    dst[o] = acc[keep]


BWD_CASES = [
    (2, 2, 4, 6, (5, 6, 8), (2, 3, 3), (1, 2, 2), (0, 1, 2), (2, 1, 2)),
    (2, 2, 3, 8, (6, 5, 7), (3, 3, 3), (2, 1, 2), (1, 1, 1), (1, 1, 1)),
    (1, 2, 8, 8, (4, 4, 9), (1, 1, 5), (1, 1, 3), (0, 0, 2), (1, 1, 1)),
    (2, 1, 8, 16, (6, 7, 5), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),   # one group: the filter gradient as one GEMM
    (3, 1, 3, 8, (9, 8, 7), (3, 2, 3), (2, 2, 2), (1, 0, 1), (1, 1, 1)),
    (1, 1, 16, 8, (5, 5, 6), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),   # one image: the output gradient read in place
    (2, 1, 16, 16, (4, 5, 1), (3, 3, 1), (1, 1, 1), (1, 1, 0), (1, 1, 1)),  # depth 1
    (3, 1, 8, 8, (4, 4, 9), (1, 1, 5), (1, 1, 3), (0, 0, 2), (1, 1, 1)),    # depth stride 3
    (2, 1, 3, 8, (5, 8, 6), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),    # few channels, strided: the 2-D phases merged
]


@pytest.mark.parametrize("case", BWD_CASES)
@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
@pytest.mark.parametrize("t,es", [("f32", 4), ("f16", 2)])
def test_conv3d_bwd_data_plan_replayed_on_the_cpu(rock, case, layouts, t, es):
    n, g, c, k, ins, fs, stride, pad, dil = case
    rng = np.random.default_rng(7)
    outs = [orc.conv_out_dim(ins[a], fs[a], pad[a], pad[a], stride[a], dil[a]) for a in range(3)]
    fil = rng.integers(-3, 4, g * k * c * fs[0] * fs[1] * fs[2]).astype(np.float32)
    dout = rng.integers(-3, 4, n * g * k * outs[0] * outs[1] * outs[2]).astype(np.float32)
    want = orc.conv3d_bwd_data(fil, dout, *layouts, n, g, c, k, ins, fs, stride, pad, dil)
    opts = _options(case, layouts, t).replace("--operation conv", "--operation conv_bwd_data")
    ws_bytes = rock.RockKernel(opts).workspace_bytes
    dx = np.full(want.size, np.nan, np.float32)
    ws = np.full(ws_bytes // es, np.nan, np.float32)
    names = _replay_plan(rock, opts, [fil, dx, dout, None, ws], t, es)
    assert np.array_equal(dx, want)
    assert names.count("rock_fold_depth") == 1


@pytest.mark.parametrize("case", BWD_CASES)
@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
@pytest.mark.parametrize("t,es", [("f32", 4), ("f16", 2)])
def test_conv3d_bwd_weight_plan_replayed_on_the_cpu(rock, case, layouts, t, es):
    n, g, c, k, ins, fs, stride, pad, dil = case
    rng = np.random.default_rng(8)
    outs = [orc.conv_out_dim(ins[a], fs[a], pad[a], pad[a], stride[a], dil[a]) for a in range(3)]
    inp = rng.integers(-3, 4, n * g * c * ins[0] * ins[1] * ins[2]).astype(np.float32)
    dout = rng.integers(-3, 4, n * g * k * outs[0] * outs[1] * outs[2]).astype(np.float32)
    want = orc.conv3d_bwd_weight(inp, dout, *layouts, n, g, c, k, ins, fs, stride, pad, dil)
    opts = _options(case, layouts, t).replace("--operation conv", "--operation conv_bwd_weight")
    ws_bytes = rock.RockKernel(opts).workspace_bytes
    dw = np.full(want.size, np.nan, np.float32)
    ws = np.full(ws_bytes // es, np.nan, np.float32)
    _replay_plan(rock, opts, [dw, inp, dout, None, ws], t, es)
    assert np.array_equal(dw, want)


@pytest.mark.parametrize("layouts", [NCDHW, NDHWC, MIXED], ids=lambda l: l[1])
def test_conv3d_residual_plan(rock, layouts):
    """A residual tensor lies as the output does: beside an output written in
    place it is read in place (caller pointer 4), beside an output that goes
    through the workspace it is converted into the same intermediate layout."""
    case = CASES[2]
    plain = rock.RockKernel(_options(case, layouts, "f16"))
    opts = _options(case, layouts, "f16") + " --residual add"
    first = rock.RockKernel(opts)
    kerns = [first] + [rock.RockKernel(opts + " --kernel_id %d" % i) for i in range(1, first.kernel_count)]
    names = [k.kernel_name for k in kerns]
    (conv_at,) = [i for i, nm in enumerate(names) if nm.startswith("rock_conv_")]
    assert first.caller_pointers == 6 and names[conv_at].endswith("_e")
    res_src, res_off = _pointer_map(rock, kerns[conv_at])[4]
    out_src, out_off = _pointer_map(rock, kerns[conv_at])[2]
    if out_src == 2:        # written in place
        assert (res_src, res_off) == (4, 0) and first.kernel_count == plain.kernel_count
    else:
        assert out_src == 5 and res_src == 5 and res_off > out_off
        assert first.kernel_count == plain.kernel_count + 1 and first.workspace_bytes > plain.workspace_bytes
        (s_src, _), (d_src, d_off) = _pointer_map(rock, kerns[conv_at - 1])
        assert (s_src, d_src, d_off) == (4, 5, res_off)
    args = first.arguments()
    assert args[4] == args[2] and args[5][0] == -1
