"""numpy front end of the CPU oracle (librock_oracle.so).

Test infrastructure only: imported by tests/, the smoke check and the
benchmark's CPU-baseline leg.  The shipped package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librock_oracle.so")

F32, F16, BF16, I8, FP8, BF8, I32 = range(7)
TYPE_CODES = {"f32": F32, "f16": F16, "bf16": BF16, "i8": I8, "fp8": FP8,
              "bf8": BF8, "i32": I32}
_NP_STORAGE = {F32: np.float32, F16: np.uint16, BF16: np.uint16, I8: np.int8,
               FP8: np.uint8, BF8: np.uint8, I32: np.int32}


def build():
    """Compile the oracle with the Makefile next to it."""
    subprocess.run(["make", "-C", _HERE, "-s", "librock_oracle.so"], check=True)


class ConvDims(C.Structure):
    _fields_ = [(n, C.c_int64) for n in (
        "n", "g", "c", "k", "hi", "wi", "y", "x", "ho", "wo",
        "stride_h", "stride_w", "pad_h", "pad_w", "dil_h", "dil_w")]


class VerifyResult(C.Structure):
    _fields_ = [("rms", C.c_double), ("max_abs_diff", C.c_double),
                ("max_rel_diff", C.c_double), ("ave_abs_diff", C.c_double),
                ("max_mag", C.c_double), ("pass_rms", C.c_int32),
                ("pass_abs", C.c_int32), ("pass_rel", C.c_int32)]

    def passed(self):
        return bool(self.pass_rms and self.pass_abs and self.pass_rel)

    def __repr__(self):
        return ("VerifyResult(rms=%.3e, max_abs=%.3e, max_rel=%.3e, [%d %d %d])"
                % (self.rms, self.max_abs_diff, self.max_rel_diff,
                   self.pass_rms, self.pass_abs, self.pass_rel))


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        i64, i32, f32, vp = C.c_int64, C.c_int32, C.c_float, C.c_void_p
        L.orc_max_threads.restype = C.c_int
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [f32]
        L.orc_f16_to_f32.restype = f32
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [f32]
        for nm in ("orc_f32_to_e4m3fn_sat", "orc_f32_to_e4m3fn_nosat",
                   "orc_f32_to_e5m2_sat", "orc_f32_to_e5m2_nosat"):
            getattr(L, nm).restype = C.c_uint8
            getattr(L, nm).argtypes = [f32]
        for nm in ("orc_e4m3fn_to_f32", "orc_e5m2_to_f32"):
            getattr(L, nm).restype = f32
            getattr(L, nm).argtypes = [C.c_uint8]
        L.orc_widen.argtypes = [vp, C.c_int, i64, vp]
        L.orc_narrow.argtypes = [vp, C.c_int, i64, vp]
        L.orc_round_through.argtypes = [vp, C.c_int, i64]
        gemm_args = [vp, vp, vp, i64, i64, i64, i64, C.c_int, C.c_int, C.c_int,
                     i64, i64, C.c_int]
        L.orc_gemm_f32.argtypes = gemm_args
        L.orc_gemm_i8.argtypes = gemm_args
        conv_args = [vp, vp, vp, C.c_char_p, C.c_char_p, C.c_char_p,
                     C.POINTER(ConvDims), i64, i64, C.c_int]
        L.orc_conv_fwd_f32.argtypes = conv_args
        L.orc_conv_fwd_f32.restype = C.c_int
        L.orc_conv_fwd_i8.argtypes = conv_args
        L.orc_conv_fwd_i8.restype = C.c_int
        bwd_args = [vp, vp, vp, C.c_char_p, C.c_char_p, C.c_char_p,
                    C.POINTER(ConvDims), C.c_int]
        for nm in ("orc_conv_bwd_data_f32", "orc_conv_bwd_weight_f32"):
            getattr(L, nm).argtypes = bwd_args
            getattr(L, nm).restype = C.c_int
        L.orc_attention_f32.argtypes = [vp, vp, vp, vp, vp, f32, vp, i64, i64,
                                        i64, i64, i64, C.c_int, C.c_int,
                                        C.c_int, C.c_int, i64, i64, C.c_int]
        L.orc_attention_where_f32.argtypes = [vp, vp, vp, vp, vp, vp, vp, f32, vp, i64, i64,
                                              i64, i64, i64, C.c_int, C.c_int,
                                              C.c_int, C.c_int, i64, i64, C.c_int]
        L.orc_softmax_f32.argtypes = [vp, vp, i64, i64]
        L.orc_dequantize_i64.argtypes = [vp, i64, f32, i32, vp]
        L.orc_quantize_i8.argtypes = [vp, i64, f32, i32, vp]
        L.orc_dequantize_i64_per_channel.argtypes = [vp, i64, i64, vp, vp, vp]
        L.orc_quantize_i8_per_channel.argtypes = [vp, i64, i64, vp, vp, vp]
        L.orc_scale_bias_f32.argtypes = [vp, i64, i64, f32, vp]
        L.orc_verify_float.argtypes = [vp, vp, i64, f32, f32, f32,
                                       C.POINTER(VerifyResult)]
        L.orc_verify_int32_int64.argtypes = [vp, vp, i64, C.POINTER(i64),
                                             C.POINTER(i64)]
        L.orc_verify_int32_int64.restype = i64
        L.orc_fill_fixed.argtypes = [vp, i64, C.c_int]
        L.orc_seed.argtypes = [C.c_uint32]
        L.orc_fill_rand.argtypes = [vp, i64, C.c_int, C.c_int, C.c_int]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def max_threads():
    return lib().orc_max_threads()


# ---- codecs -----------------------------------------------------------
def widen(raw, type_code):
    """Raw storage array (uint16 / uint8 / int8 / float32) -> float32."""
    raw = _c(raw, _NP_STORAGE[type_code])
    out = np.empty(raw.shape, np.float32)
    lib().orc_widen(_p(raw), type_code, raw.size, _p(out))
    return out


def narrow(x, type_code):
    """float32 -> raw storage array of the given type (RNE; fp8 saturates)."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, _NP_STORAGE[type_code])
    lib().orc_narrow(_p(x), type_code, x.size, _p(out))
    return out


def round_through(x, type_code):
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    lib().orc_round_through(_p(x), type_code, x.size)
    return x


# ---- GEMM -------------------------------------------------------------
def gemm(A, B, G, M, N, K, transA=False, transB=False, transC=False,
         rows=None, threads=0):
    """A, B: flat (or any-shape) arrays in the reference's storage order.
    float32 inputs -> float32 C; int8 inputs -> int64 C.  Returns a flat C of
    G*M*N elements (rows outside `rows` are zero)."""
    r0, r1 = rows if rows is not None else (0, M)
    if A.dtype == np.int8:
        A, B = _c(A, np.int8), _c(B, np.int8)
        Cm = np.zeros(G * M * N, np.int64)
        fn = lib().orc_gemm_i8
    else:
        A, B = _c(A, np.float32), _c(B, np.float32)
        Cm = np.zeros(G * M * N, np.float32)
        fn = lib().orc_gemm_f32
    assert A.size == G * M * K and B.size == G * K * N
    fn(_p(A), _p(B), _p(Cm), G, M, N, K, int(transA), int(transB), int(transC),
       r0, r1, threads)
    return Cm


# ---- convolution --------------------------------------------------------
def conv_out_dim(in_len, fil_len, pad_l, pad_r, stride, dil):
    """Output extent, ConvGenerator.h:101-108."""
    return (in_len + pad_l + pad_r - (fil_len - 1) * dil - 1) // stride + 1


def conv_fwd(fil, inp, fil_layout, in_layout, out_layout, n, g, c, k, hi, wi,
             y, x, stride=(1, 1), pad=(0, 0), dil=(1, 1), out_range=None,
             threads=0, pad_r=None):
    """c and k are PER-GROUP channel counts.  Layout strings: permutations of
    'gkcyx' / 'ngchw' / 'ngkhw'.  `pad` is the top / left padding and, unless
    `pad_r` gives the bottom / right one, that one too.  Returns (flat output,
    ho, wo)."""
    pad_r = pad if pad_r is None else pad_r
    ho = conv_out_dim(hi, y, pad[0], pad_r[0], stride[0], dil[0])
    wo = conv_out_dim(wi, x, pad[1], pad_r[1], stride[1], dil[1])
    d = ConvDims(n, g, c, k, hi, wi, y, x, ho, wo, stride[0], stride[1],
                 pad[0], pad[1], dil[0], dil[1])
    total = n * g * k * ho * wo
    b, e = out_range if out_range is not None else (0, total)
    if fil.dtype == np.int8:
        fil, inp = _c(fil, np.int8), _c(inp, np.int8)
        out = np.zeros(total, np.int64)
        fn = lib().orc_conv_fwd_i8
    else:
        fil, inp = _c(fil, np.float32), _c(inp, np.float32)
        out = np.zeros(total, np.float32)
        fn = lib().orc_conv_fwd_f32
    assert fil.size == g * k * c * y * x and inp.size == n * g * c * hi * wi
    rc = fn(_p(fil), _p(inp), _p(out), fil_layout.encode(), in_layout.encode(),
            out_layout.encode(), C.byref(d), b, e, threads)
    if rc != 0:
        raise ValueError("bad layout string")
    return out, ho, wo


def conv_bwd_data(fil, out, fil_layout, in_layout, out_layout, n, g, c, k, hi,
                  wi, y, x, stride=(1, 1), pad=(0, 0), dil=(1, 1), threads=0, pad_r=None):
    """Gradient with respect to the input: (flat input-shaped array, ho, wo)."""
    pad_r = pad if pad_r is None else pad_r   # bottom / right padding: it only sets the output's extent
    ho = conv_out_dim(hi, y, pad[0], pad_r[0], stride[0], dil[0])
    wo = conv_out_dim(wi, x, pad[1], pad_r[1], stride[1], dil[1])
    d = ConvDims(n, g, c, k, hi, wi, y, x, ho, wo, stride[0], stride[1],
                 pad[0], pad[1], dil[0], dil[1])
    fil, out = _c(fil, np.float32), _c(out, np.float32)
    assert fil.size == g * k * c * y * x and out.size == n * g * k * ho * wo
    inp = np.zeros(n * g * c * hi * wi, np.float32)
    rc = lib().orc_conv_bwd_data_f32(_p(fil), _p(inp), _p(out), fil_layout.encode(), in_layout.encode(),
                                     out_layout.encode(), C.byref(d), threads)
    if rc != 0:
        raise ValueError("bad layout string")
    return inp, ho, wo


def conv_bwd_weight(inp, out, fil_layout, in_layout, out_layout, n, g, c, k, hi,
                    wi, y, x, stride=(1, 1), pad=(0, 0), dil=(1, 1), threads=0, pad_r=None):
    """Gradient with respect to the filter: (flat filter-shaped array, ho, wo)."""
    pad_r = pad if pad_r is None else pad_r
    ho = conv_out_dim(hi, y, pad[0], pad_r[0], stride[0], dil[0])
    wo = conv_out_dim(wi, x, pad[1], pad_r[1], stride[1], dil[1])
    d = ConvDims(n, g, c, k, hi, wi, y, x, ho, wo, stride[0], stride[1],
                 pad[0], pad[1], dil[0], dil[1])
    inp, out = _c(inp, np.float32), _c(out, np.float32)
    assert inp.size == n * g * c * hi * wi and out.size == n * g * k * ho * wo
    fil = np.zeros(g * k * c * y * x, np.float32)
    rc = lib().orc_conv_bwd_weight_f32(_p(fil), _p(inp), _p(out), fil_layout.encode(), in_layout.encode(),
                                       out_layout.encode(), C.byref(d), threads)
    if rc != 0:
        raise ValueError("bad layout string")
    return fil, ho, wo


def conv3d(fil, inp, fil_layout, in_layout, out_layout, n, g, c, k, in_size, fil_size,
           stride=(1, 1, 1), pad=(0, 0, 0), dil=(1, 1, 1)):
    """Forward convolution over three spatial dimensions, the arithmetic the
    reference checks its 3-D rock.conv against (linalg.conv_3d in
    mlir/test/Dialect/Rock/integration/conv3d-test-from-rocmlir-gen.mlir:12-20,
    grouped and strided as rocmlir-gen.cpp:171-294 parameterises it).  Flat
    arrays laid out as six-letter strings over g k c 0 1 2 / n g c 0 1 2 /
    n g k 0 1 2 say; numpy, one slice product per filter tap, sums in f64 (tests
    use integer-valued data where the order of the sum cannot matter, and a
    tolerance otherwise).  Returns (flat output, output sizes)."""
    outs = tuple(conv_out_dim(in_size[a], fil_size[a], pad[a], pad[a], stride[a], dil[a]) for a in range(3))

    def canon(flat, layout, letters, sizes):
        shape = [sizes[letters.index(ch)] for ch in layout]
        arr = np.asarray(flat, np.float64).reshape(shape)
        return arr.transpose([layout.index(ch) for ch in letters])

    f = canon(fil, fil_layout, "gkc012", (g, k, c) + tuple(fil_size))
    x = canon(inp, in_layout, "ngc012", (n, g, c) + tuple(in_size))
    xp = np.zeros((n, g, c) + tuple(in_size[a] + 2 * pad[a] for a in range(3)))
    xp[:, :, :, pad[0]:pad[0] + in_size[0], pad[1]:pad[1] + in_size[1], pad[2]:pad[2] + in_size[2]] = x
    out = np.zeros((n, g, k) + outs)
    for t0 in range(fil_size[0]):
        for t1 in range(fil_size[1]):
            for t2 in range(fil_size[2]):
                win = xp[:, :, :,
                         t0 * dil[0]:t0 * dil[0] + (outs[0] - 1) * stride[0] + 1:stride[0],
                         t1 * dil[1]:t1 * dil[1] + (outs[1] - 1) * stride[1] + 1:stride[1],
                         t2 * dil[2]:t2 * dil[2] + (outs[2] - 1) * stride[2] + 1:stride[2]]
                out += np.einsum("ngcabd,gkc->ngkabd", win, f[:, :, :, t0, t1, t2])
    flat = out.transpose(["ngk012".index(ch) for ch in out_layout]).astype(np.float32).ravel()
    return flat, outs


def _conv3d_canon(flat, layout, letters, sizes):
    shape = [sizes[letters.index(ch)] for ch in layout]
    arr = np.asarray(flat, np.float64).reshape(shape)
    return arr.transpose([layout.index(ch) for ch in letters])


def _conv3d_windows(in_size, fil_size, outs, stride, pad, dil):
    """For every filter tap the slices of the padded input its products touch
    (one input position per output position)."""
    for t0 in range(fil_size[0]):
        for t1 in range(fil_size[1]):
            for t2 in range(fil_size[2]):
                yield (t0, t1, t2), tuple(
                    slice(t * dil[a], t * dil[a] + (outs[a] - 1) * stride[a] + 1, stride[a])
                    for a, t in enumerate((t0, t1, t2)))


def conv3d_bwd_data(fil, dout, fil_layout, in_layout, out_layout, n, g, c, k, in_size, fil_size,
                    stride=(1, 1, 1), pad=(0, 0, 0), dil=(1, 1, 1)):
    """Input gradient of the 3-D convolution: the reference's CPU validator
    is one loop nest for every direction and any number of spatial dimensions
    (createCPUConvWithMLIR, rocmlir-gen.cpp:1715-1997); for this direction the
    result tensor is the input (:1731-1733), the output position follows from
    out_tmp = in + pad - t*dilation, out = out_tmp / stride where that divides
    (:1895-1904) and in[n,g,c,i] += fil[g,k,c,t] * out[n,g,k,o] (:1938-1945,
    1951-1966).  numpy, one slice update
    per filter tap, sums in f64.  Returns the flat input-shaped gradient."""
    outs = tuple(conv_out_dim(in_size[a], fil_size[a], pad[a], pad[a], stride[a], dil[a]) for a in range(3))
    f = _conv3d_canon(fil, fil_layout, "gkc012", (g, k, c) + tuple(fil_size))
    dy = _conv3d_canon(dout, out_layout, "ngk012", (n, g, k) + outs)
    dxp = np.zeros((n, g, c) + tuple(in_size[a] + 2 * pad[a] for a in range(3)))
    for (t0, t1, t2), win in _conv3d_windows(in_size, fil_size, outs, stride, pad, dil):
        dxp[(slice(None),) * 3 + win] += np.einsum("ngkabd,gkc->ngcabd", dy, f[:, :, :, t0, t1, t2])
    dx = dxp[:, :, :, pad[0]:pad[0] + in_size[0], pad[1]:pad[1] + in_size[1], pad[2]:pad[2] + in_size[2]]
    return dx.transpose(["ngc012".index(ch) for ch in in_layout]).astype(np.float32).ravel()


def conv3d_bwd_weight(inp, dout, fil_layout, in_layout, out_layout, n, g, c, k, in_size, fil_size,
                      stride=(1, 1, 1), pad=(0, 0, 0), dil=(1, 1, 1)):
    """Filter gradient of the 3-D convolution, the same loop nest
    (rocmlir-gen.cpp:1715-1997) with the filter as the result tensor
    (:1734-1736): fil[g,k,c,t] += out[n,g,k,o] * in[n,g,c,i] with
    i = o*stride + t*dilation - pad, wherever i lies inside the input
    (:1905-1911, 1930-1937).
    numpy, one product per filter tap, sums in f64.  Returns the flat
    filter-shaped gradient."""
    outs = tuple(conv_out_dim(in_size[a], fil_size[a], pad[a], pad[a], stride[a], dil[a]) for a in range(3))
    x = _conv3d_canon(inp, in_layout, "ngc012", (n, g, c) + tuple(in_size))
    dy = _conv3d_canon(dout, out_layout, "ngk012", (n, g, k) + outs)
    xp = np.zeros((n, g, c) + tuple(in_size[a] + 2 * pad[a] for a in range(3)))
    xp[:, :, :, pad[0]:pad[0] + in_size[0], pad[1]:pad[1] + in_size[1], pad[2]:pad[2] + in_size[2]] = x
    df = np.zeros((g, k, c) + tuple(fil_size))
    for (t0, t1, t2), win in _conv3d_windows(in_size, fil_size, outs, stride, pad, dil):
        df[:, :, :, t0, t1, t2] = np.einsum("ngcabd,ngkabd->gkc", xp[(slice(None),) * 3 + win], dy)
    return df.transpose(["gkc012".index(ch) for ch in fil_layout]).astype(np.float32).ravel()


# ---- attention ------------------------------------------------------------
def attention(Q, K, V, G, sq, sk, dqk, dv, scale=1.0, scale_t=None,
              bias_t=None, transQ=False, transK=False, transV=False,
              transO=False, q_rows=None, threads=0, mask=None, other=None):
    """mask (int8 [G,sq,sk]) and other (f32 [G,sq,sk]): where mask is zero the
    score is replaced by other before the softmax (migraphx.where)."""
    Q, K, V = _c(Q, np.float32), _c(K, np.float32), _c(V, np.float32)
    assert Q.size == G * sq * dqk and K.size == G * sk * dqk
    assert V.size == G * sk * dv
    st = _c(scale_t, np.float32) if scale_t is not None else None
    bt = _c(bias_t, np.float32) if bias_t is not None else None
    O = np.zeros(G * sq * dv, np.float32)
    q0, q1 = q_rows if q_rows is not None else (0, sq)
    if mask is not None:
        mk, ot = _c(mask, np.int8), _c(other, np.float32)
        assert mk.size == G * sq * sk and ot.size == G * sq * sk
        lib().orc_attention_where_f32(_p(Q), _p(K), _p(V), _p(st), _p(bt), _p(mk), _p(ot),
                                      np.float32(scale), _p(O), G, sq, sk, dqk, dv,
                                      int(transQ), int(transK), int(transV), int(transO),
                                      q0, q1, threads)
        return O
    lib().orc_attention_f32(_p(Q), _p(K), _p(V), _p(st), _p(bt),
                            np.float32(scale), _p(O), G, sq, sk, dqk, dv,
                            int(transQ), int(transK), int(transV), int(transO),
                            q0, q1, threads)
    return O


def run_attention_program(program, x, inputs):
    """The pre-softmax region of rock.attention (RockOps.td:208-254) as postfix
    code over float32 arrays: x = the scores, t<i> = inputs[i], c:<number>,
    add sub mul div max min, exp neg tanh sigmoid relu abs erf, where
    (c a b -> c != 0 ? a : b).  Plain numpy, one float32 operation per token."""
    import math
    f32 = np.float32
    stack = []
    binary = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide,
              "max": np.maximum, "min": np.minimum}
    unary = {"exp": np.exp, "neg": np.negative, "tanh": np.tanh,
             "sigmoid": lambda a: (f32(1) / (f32(1) + np.exp(-a))).astype(f32),
             "relu": lambda a: np.maximum(a, f32(0)), "abs": np.abs,
             "erf": lambda a: np.vectorize(math.erf)(a.astype(np.float64)).astype(f32)}
    for tok in program.replace(" ", "").split(","):
        if tok == "x":
            stack.append(np.asarray(x, f32))
        elif tok[0] == "t" and tok[1:].isdigit():
            stack.append(np.asarray(inputs[int(tok[1:])], f32).reshape(np.shape(x)))
        elif tok.startswith("c:"):
            stack.append(np.full(np.shape(x), f32(float(tok[2:])), f32))
        elif tok in binary:
            b, a = stack.pop(), stack.pop()
            stack.append(binary[tok](a, b).astype(f32))
        elif tok in unary:
            stack.append(np.asarray(unary[tok](stack.pop()), f32))
        elif tok == "where":
            b, a, c = stack.pop(), stack.pop(), stack.pop()
            stack.append(np.where(c != 0, a, b).astype(f32))
        else:
            raise ValueError("unknown token %r" % tok)
    assert len(stack) == 1
    return stack[0]


def attention_program(Q, K, V, G, sq, sk, dqk, dv, program, inputs=(), transK=False):
    """Attention with a pre-softmax program: O = softmax(program(Q K, inputs)) V,
    float32 throughout in the validator's order of steps (rocmlir-gen.cpp:
    2565-2620: the first GEMM, the element-wise region, softmax over the keys,
    the second GEMM); numpy, for sizes a test finishes in seconds.  Q [G,sq,d],
    K [G,d,sk] ([G,sk,d] with transK), V [G,sk,dv]."""
    Q = _c(Q, np.float32).reshape(G, sq, dqk)
    K = _c(K, np.float32).reshape((G, sk, dqk) if transK else (G, dqk, sk))
    V = _c(V, np.float32).reshape(G, sk, dv)
    Kt = K.transpose(0, 2, 1) if transK else K
    S = np.matmul(Q, Kt).astype(np.float32)
    X = run_attention_program(program, S, inputs)
    return np.matmul(softmax(X).reshape(G, sq, sk), V).astype(np.float32).ravel()


def softmax(x):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    lib().orc_softmax_f32(_p(x), _p(y), x.size // x.shape[-1], x.shape[-1])
    return y


# ---- quantisation epilogue ----------------------------------------------------
def dequantize(acc_i64, scale, zero_point=0):
    acc = _c(acc_i64, np.int64)
    y = np.empty(acc.shape, np.float32)
    lib().orc_dequantize_i64(_p(acc), acc.size, np.float32(scale), zero_point,
                             _p(y))
    return y


def quantize_i8(x, scale, zero_point=0):
    x = _c(x, np.float32)
    q = np.empty(x.shape, np.int8)
    lib().orc_quantize_i8(_p(x), x.size, np.float32(scale), zero_point, _p(q))
    return q


def dequantize_per_channel(acc_i64, scale, zero_point=None):
    """acc [..., channels]; scale f32[channels], zero_point int32[channels] or None."""
    acc = _c(acc_i64, np.int64)
    ch = acc.shape[-1]
    sc = _c(scale, np.float32)
    zp = _c(zero_point, np.int32) if zero_point is not None else None
    assert sc.size == ch and (zp is None or zp.size == ch)
    y = np.empty(acc.shape, np.float32)
    lib().orc_dequantize_i64_per_channel(_p(acc), acc.size // ch, ch, _p(sc), _p(zp), _p(y))
    return y


def quantize_i8_per_channel(x, scale, zero_point=None):
    """x [..., channels]; scale f32[channels], zero_point int32[channels] or None."""
    x = _c(x, np.float32)
    ch = x.shape[-1]
    sc = _c(scale, np.float32)
    zp = _c(zero_point, np.int32) if zero_point is not None else None
    assert sc.size == ch and (zp is None or zp.size == ch)
    q = np.empty(x.shape, np.int8)
    lib().orc_quantize_i8_per_channel(_p(x), x.size // ch, ch, _p(sc), _p(zp), _p(q))
    return q


def scale_bias(x, rows, cols, scale, bias=None):
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    b = _c(bias, np.float32) if bias is not None else None
    lib().orc_scale_bias_f32(_p(x), rows, cols, np.float32(scale), _p(b))
    return x


# ---- verifier -------------------------------------------------------------------
def verify_float(gpu, val, thr_rms=3e-5, thr_abs=100.0, thr_rel=100.0):
    gpu, val = _c(gpu, np.float32).ravel(), _c(val, np.float32).ravel()
    assert gpu.size == val.size
    res = VerifyResult()
    lib().orc_verify_float(_p(gpu), _p(val), gpu.size, thr_rms, thr_abs,
                           thr_rel, C.byref(res))
    return res


def verify_int(gpu_i32, val_i64):
    gpu, val = _c(gpu_i32, np.int32).ravel(), _c(val_i64, np.int64).ravel()
    assert gpu.size == val.size
    ovf, mad = C.c_int64(0), C.c_int64(0)
    fails = lib().orc_verify_int32_int64(_p(gpu), _p(val), gpu.size,
                                         C.byref(ovf), C.byref(mad))
    return fails, ovf.value, mad.value


# ---- data fill ----------------------------------------------------------------------
def fill_fixed(n, is_int=False):
    x = np.empty(n, np.float32)
    lib().orc_fill_fixed(_p(x), n, int(is_int))
    return x


def seed(s):
    lib().orc_seed(s)


def fill_rand(n, lo, hi, as_float):
    x = np.empty(n, np.float32)
    lib().orc_fill_rand(_p(x), n, lo, hi, int(as_float))
    return x
