/*
 * rock_oracle.c -- CPU restatement of the reference's validator for the
 * Rock-dialect contraction path (GEMM, forward convolution, attention,
 * quantisation epilogue), plus its verifier metrics and data fill.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the GPU kernels
 * are compared with; it is never linked into, loaded by or called from the
 * shipped library.  Only tests, the smoke check and the benchmark's CPU
 * baseline leg may use it.
 *
 * Every routine follows the loop nest that `rocmlir-gen -pv` generates
 * (citations are relative to the reference tree):
 *   GEMM       mlir/tools/rocmlir-gen/rocmlir-gen.cpp:2401-2493
 *   conv fwd   mlir/tools/rocmlir-gen/rocmlir-gen.cpp:1715-1997
 *   attention  mlir/tools/rocmlir-gen/rocmlir-gen.cpp:2507-2638
 *   verifier   mlir/lib/ExecutionEngine/conv-validation-wrappers.cpp:104-285
 *   data fill  mlir/tools/rocmlir-gen/rocmlir-gen.cpp:1325-1486 and
 *              mlir/lib/ExecutionEngine/conv-validation-wrappers.cpp:27-50
 *   quant math mlir/lib/Conversion/MIGraphXToTosa/MIGraphXToTosa.cpp:874-982
 *
 * Arithmetic rules kept from the reference: small floats are widened to f32
 * before any arithmetic (rocmlir-gen.cpp:1692-1704), every product is one
 * IEEE multiply followed by one IEEE add into a zero-initialised output
 * (no fused multiply-add: build with -ffp-contract=off), reductions run in
 * ascending index order, int8 operands accumulate in int64.
 *
 * Two deliberate deviations, both documented where they occur:
 *   - the int8 convolution widens before multiplying (the reference multiplies
 *     in i8 first, rocmlir-gen.cpp:1955-1960, which only agrees on data in
 *     [-11,11]);
 *   - attention computes scores, softmax and P*V in f32 and leaves rounding
 *     to the caller (the reference's f16 validator does each TOSA op in f16).
 *
 * The `threads` argument splits independent output elements over OpenMP
 * threads; the reduction order inside one output element never changes, so
 * results are bit-identical for any thread count.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_EXPORT __attribute__((visibility("default")))

/* element type codes used by the widen / narrow helpers */
enum {
  ORC_F32 = 0,
  ORC_F16 = 1,
  ORC_BF16 = 2,
  ORC_I8 = 3,
  ORC_FP8_E4M3FN = 4,
  ORC_BF8_E5M2 = 5,
  ORC_I32 = 6
};

static int orc_threads(int threads) {
#ifdef _OPENMP
  if (threads <= 0)
    return omp_get_max_threads();
  return threads;
#else
  (void)threads;
  return 1;
#endif
}

ORC_EXPORT int orc_max_threads(void) { return orc_threads(0); }

/* ------------------------------------------------------------------ */
/* scalar codecs                                                       */
/* ------------------------------------------------------------------ */

static uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Generic IEEE-style narrowing with round-to-nearest-even.
 * ebits/mbits describe the target; bias = 2^(ebits-1)-1.
 * ieee_inf: target has inf/nan in the top exponent (f16, e5m2);
 * otherwise the target is "fn": top exponent is finite except the
 * all-ones mantissa pattern which is NaN (e4m3fn).
 * saturate: finite overflow (and +-inf) clamp to the largest finite value
 * (the GPU lowering's behaviour, Pipelines.cpp:238); otherwise overflow
 * gives inf (ieee) or NaN (fn). */
static uint32_t narrow_rne(float f, int ebits, int mbits, int ieee_inf,
                           int saturate) {
  uint32_t u = f32_bits(f);
  uint32_t sign = u >> 31;
  uint32_t absu = u & 0x7fffffffu;
  int bias = (1 << (ebits - 1)) - 1;
  uint32_t exp_all = (1u << ebits) - 1;
  uint32_t max_finite_bits =
      ieee_inf ? (((exp_all - 1) << mbits) | ((1u << mbits) - 1))
               : ((exp_all << mbits) | ((1u << mbits) - 2));
  uint32_t nan_bits = ieee_inf ? ((exp_all << mbits) | (1u << (mbits - 1)))
                               : ((exp_all << mbits) | ((1u << mbits) - 1));
  uint32_t inf_bits = ieee_inf ? (exp_all << mbits) : nan_bits;
  uint32_t out;
  if (absu > 0x7f800000u) { /* NaN */
    out = nan_bits;
  } else if (absu == 0x7f800000u) { /* inf */
    out = saturate ? max_finite_bits : inf_bits;
  } else if (absu == 0) {
    out = 0;
  } else {
    int e = (int)(absu >> 23) - 127; /* unbiased exponent (f32 normal) */
    uint32_t man = absu & 0x7fffffu;
    if ((absu >> 23) == 0) { /* f32 subnormal: far below any target range */
      e = -126;
    } else {
      man |= 0x800000u;
    }
    /* value = man * 2^(e-23).  Target quantum exponent: */
    int emin = 1 - bias; /* smallest normal exponent */
    int qexp = (e < emin ? emin : e) - mbits; /* exponent of one ulp */
    int shift = (e - 23) - qexp;              /* man * 2^shift ulps */
    uint64_t q;
    if (shift >= 0) {
      q = (uint64_t)man << shift;
    } else {
      int s = -shift;
      if (s > 40) {
        q = 0;
      } else {
        uint64_t m64 = man;
        uint64_t floor_q = m64 >> s;
        uint64_t rem = m64 & ((1ull << s) - 1);
        uint64_t half = 1ull << (s - 1);
        if (rem > half || (rem == half && (floor_q & 1)))
          floor_q++;
        q = floor_q;
      }
    }
    /* q counts ulps of 2^qexp; rebuild exponent/mantissa */
    int te = (e < emin ? emin : e);
    if (q >= (2ull << mbits)) { /* rounding carried into next binade */
      q >>= 1;
      te++;
    }
    if (q < (1ull << mbits)) { /* subnormal (or zero) in target */
      out = (uint32_t)q;
    } else {
      out = ((uint32_t)(te + bias) << mbits) | (uint32_t)(q & ((1ull << mbits) - 1));
    }
    if (out > max_finite_bits)
      out = saturate ? max_finite_bits : inf_bits;
  }
  return (sign << (ebits + mbits)) | out;
}

static float widen_small(uint32_t v, int ebits, int mbits, int ieee_inf) {
  uint32_t sign = (v >> (ebits + mbits)) & 1;
  uint32_t e = (v >> mbits) & ((1u << ebits) - 1);
  uint32_t m = v & ((1u << mbits) - 1);
  int bias = (1 << (ebits - 1)) - 1;
  uint32_t exp_all = (1u << ebits) - 1;
  float r;
  if (e == exp_all && ieee_inf) {
    r = m ? NAN : INFINITY;
  } else if (e == exp_all && !ieee_inf && m == ((1u << mbits) - 1)) {
    r = NAN;
  } else if (e == 0) {
    r = ldexpf((float)m, 1 - bias - mbits);
  } else {
    r = ldexpf((float)(m | (1u << mbits)), (int)e - bias - mbits);
  }
  return sign ? -r : r;
}

ORC_EXPORT uint16_t orc_f32_to_f16(float f) {
  return (uint16_t)narrow_rne(f, 5, 10, 1, 0);
}
ORC_EXPORT float orc_f16_to_f32(uint16_t h) { return widen_small(h, 5, 10, 1); }

ORC_EXPORT uint16_t orc_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return (uint16_t)((u >> 16) | 0x40);
  uint32_t lsb = (u >> 16) & 1;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}
ORC_EXPORT float orc_bf16_to_f32(uint16_t h) {
  return bits_f32((uint32_t)h << 16);
}

/* OCP e4m3fn: max 448, no inf, NaN = S.1111.111.  Saturating narrow. */
ORC_EXPORT uint8_t orc_f32_to_e4m3fn_sat(float f) {
  return (uint8_t)narrow_rne(f, 4, 3, 0, 1);
}
/* Non-saturating variant = the reference's host-side software truncation
 * (EmulateFp8ExtTrunc.cpp:384-629): finite overflow becomes NaN. */
ORC_EXPORT uint8_t orc_f32_to_e4m3fn_nosat(float f) {
  return (uint8_t)narrow_rne(f, 4, 3, 0, 0);
}
ORC_EXPORT float orc_e4m3fn_to_f32(uint8_t v) { return widen_small(v, 4, 3, 0); }

/* OCP e5m2: IEEE-like, max 57344. */
ORC_EXPORT uint8_t orc_f32_to_e5m2_sat(float f) {
  return (uint8_t)narrow_rne(f, 5, 2, 1, 1);
}
ORC_EXPORT uint8_t orc_f32_to_e5m2_nosat(float f) {
  return (uint8_t)narrow_rne(f, 5, 2, 1, 0);
}
ORC_EXPORT float orc_e5m2_to_f32(uint8_t v) { return widen_small(v, 5, 2, 1); }

/* TOSA float -> int cast: round half to even, then saturate
 * (TosaToLinalg.cpp:497-530 in the vendored MLIR). */
static int64_t round_even_sat(float x, int64_t lo, int64_t hi) {
  if (isnan(x))
    return 0;
  float r = nearbyintf(x); /* default rounding mode = ties to even */
  if (r <= (float)lo)
    return lo;
  if (r >= (float)hi)
    return hi;
  return (int64_t)r;
}

ORC_EXPORT void orc_widen(const void *src, int type, int64_t n, float *dst) {
  int64_t i;
  switch (type) {
  case ORC_F32:
    memcpy(dst, src, (size_t)n * 4);
    break;
  case ORC_F16:
    for (i = 0; i < n; ++i)
      dst[i] = orc_f16_to_f32(((const uint16_t *)src)[i]);
    break;
  case ORC_BF16:
    for (i = 0; i < n; ++i)
      dst[i] = orc_bf16_to_f32(((const uint16_t *)src)[i]);
    break;
  case ORC_I8:
    for (i = 0; i < n; ++i)
      dst[i] = (float)((const int8_t *)src)[i];
    break;
  case ORC_FP8_E4M3FN:
    for (i = 0; i < n; ++i)
      dst[i] = orc_e4m3fn_to_f32(((const uint8_t *)src)[i]);
    break;
  case ORC_BF8_E5M2:
    for (i = 0; i < n; ++i)
      dst[i] = orc_e5m2_to_f32(((const uint8_t *)src)[i]);
    break;
  case ORC_I32:
    for (i = 0; i < n; ++i)
      dst[i] = (float)((const int32_t *)src)[i];
    break;
  }
}

/* f32 -> type with round-to-nearest-even (arith.truncf); fp8 saturates as
 * the GPU path does; integers use the TOSA cast (round-even + saturate). */
ORC_EXPORT void orc_narrow(const float *src, int type, int64_t n, void *dst) {
  int64_t i;
  switch (type) {
  case ORC_F32:
    memcpy(dst, src, (size_t)n * 4);
    break;
  case ORC_F16:
    for (i = 0; i < n; ++i)
      ((uint16_t *)dst)[i] = orc_f32_to_f16(src[i]);
    break;
  case ORC_BF16:
    for (i = 0; i < n; ++i)
      ((uint16_t *)dst)[i] = orc_f32_to_bf16(src[i]);
    break;
  case ORC_I8:
    for (i = 0; i < n; ++i)
      ((int8_t *)dst)[i] = (int8_t)round_even_sat(src[i], -128, 127);
    break;
  case ORC_FP8_E4M3FN:
    for (i = 0; i < n; ++i)
      ((uint8_t *)dst)[i] = orc_f32_to_e4m3fn_sat(src[i]);
    break;
  case ORC_BF8_E5M2:
    for (i = 0; i < n; ++i)
      ((uint8_t *)dst)[i] = orc_f32_to_e5m2_sat(src[i]);
    break;
  case ORC_I32:
    for (i = 0; i < n; ++i)
      ((int32_t *)dst)[i] =
          (int32_t)round_even_sat(src[i], INT32_MIN, INT32_MAX);
    break;
  }
}

/* Round an f32 array through `type` and back: what the verifier does to the
 * CPU result before comparing (rocmlir-gen.cpp:2828-2840). */
ORC_EXPORT void orc_round_through(float *x, int type, int64_t n) {
  int64_t i;
  if (type == ORC_F16)
    for (i = 0; i < n; ++i)
      x[i] = orc_f16_to_f32(orc_f32_to_f16(x[i]));
  else if (type == ORC_BF16)
    for (i = 0; i < n; ++i)
      x[i] = orc_bf16_to_f32(orc_f32_to_bf16(x[i]));
  else if (type == ORC_FP8_E4M3FN)
    for (i = 0; i < n; ++i)
      x[i] = orc_e4m3fn_to_f32(orc_f32_to_e4m3fn_sat(x[i]));
  else if (type == ORC_BF8_E5M2)
    for (i = 0; i < n; ++i)
      x[i] = orc_e5m2_to_f32(orc_f32_to_e5m2_sat(x[i]));
}

/* ------------------------------------------------------------------ */
/* GEMM  (rocmlir-gen.cpp:2401-2493)                                   */
/* ------------------------------------------------------------------ */
/* Storage shapes (rocmlir-gen.cpp:2058-2080):
 *   A is [G,M,K], or [G,K,M] when transA;
 *   B is [G,K,N], or [G,N,K] when transB;
 *   C is [G,M,N], or [G,N,M] when transC.
 * C is zero-initialised, then for k ascending: C += A*B (mul, then add).
 * row_begin/row_end restrict the computed m range (a bounded sample for
 * timing); rows outside are left untouched. */
ORC_EXPORT void orc_gemm_f32(const float *A, const float *B, float *C,
                             int64_t G, int64_t M, int64_t N, int64_t K,
                             int transA, int transB, int transC,
                             int64_t row_begin, int64_t row_end, int threads) {
  int64_t a_ms = transA ? 1 : K, a_ks = transA ? M : 1;
  int64_t b_ks = transB ? 1 : N, b_ns = transB ? K : 1;
  int64_t c_ms = transC ? 1 : N, c_ns = transC ? M : 1;
  int nt = orc_threads(threads);
  int64_t rows = row_end - row_begin;
  (void)nt;
#pragma omp parallel for collapse(2) num_threads(nt) schedule(static)
  for (int64_t g = 0; g < G; ++g) {
    for (int64_t mi = 0; mi < rows; ++mi) {
      int64_t m = row_begin + mi;
      const float *a = A + g * M * K + m * a_ms;
      const float *b = B + g * K * N;
      float *c = C + g * M * N + m * c_ms;
      for (int64_t n = 0; n < N; ++n) {
        float acc = 0.0f;
        const float *bn = b + n * b_ns;
        for (int64_t k = 0; k < K; ++k) {
          float prod = a[k * a_ks] * bn[k * b_ks];
          acc = prod + acc;
        }
        c[n * c_ns] = acc;
      }
    }
  }
}

/* int8 operands, int64 accumulation (rocmlir-gen.cpp:2061-2065,3225-3228):
 * both operands are sign-extended to the accumulator type before the
 * multiply (rocmlir-gen.cpp:2467-2471). */
ORC_EXPORT void orc_gemm_i8(const int8_t *A, const int8_t *B, int64_t *C,
                            int64_t G, int64_t M, int64_t N, int64_t K,
                            int transA, int transB, int transC,
                            int64_t row_begin, int64_t row_end, int threads) {
  int64_t a_ms = transA ? 1 : K, a_ks = transA ? M : 1;
  int64_t b_ks = transB ? 1 : N, b_ns = transB ? K : 1;
  int64_t c_ms = transC ? 1 : N, c_ns = transC ? M : 1;
  int nt = orc_threads(threads);
  int64_t rows = row_end - row_begin;
  (void)nt;
#pragma omp parallel for collapse(2) num_threads(nt) schedule(static)
  for (int64_t g = 0; g < G; ++g) {
    for (int64_t mi = 0; mi < rows; ++mi) {
      int64_t m = row_begin + mi;
      const int8_t *a = A + g * M * K + m * a_ms;
      const int8_t *b = B + g * K * N;
      int64_t *c = C + g * M * N + m * c_ms;
      for (int64_t n = 0; n < N; ++n) {
        int64_t acc = 0;
        const int8_t *bn = b + n * b_ns;
        for (int64_t k = 0; k < K; ++k)
          acc += (int64_t)a[k * a_ks] * (int64_t)bn[k * b_ks];
        c[n * c_ns] = acc;
      }
    }
  }
}

/* ------------------------------------------------------------------ */
/* forward convolution (rocmlir-gen.cpp:1715-1997)                     */
/* ------------------------------------------------------------------ */
/* Layout strings are 5 lowercase letters, a permutation of
 *   filter "gkcyx", input "ngchw", output "ngkhw"
 * giving the storage order, slowest dimension first.  Loop nest: the five
 * output dimensions in output-layout order, then c, then y, then x
 * (rocmlir-gen.cpp:1806-1816); the tap contributes only when the computed
 * input coordinate is in bounds (rocmlir-gen.cpp:1869-1905). */
typedef struct {
  int64_t n, g, c, k, hi, wi, y, x, ho, wo;
  int64_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
} orc_conv_dims;

static int layout_strides(const char *layout, const char *letters,
                          const int64_t *sizes, int64_t *strides) {
  /* letters[i] has extent sizes[i]; returns strides[i] for letters[i] */
  int64_t run = 1;
  int found = 0;
  for (int pos = 4; pos >= 0; --pos) {
    const char *p = strchr(letters, layout[pos]);
    if (!p)
      return -1;
    int idx = (int)(p - letters);
    strides[idx] = run;
    run *= sizes[idx];
    found |= 1 << idx;
  }
  return found == 31 ? 0 : -1;
}

#define CONV_BODY(ACC_T, IN_T, WIDEN)                                          \
  int64_t fs[5], is[5], os[5];                                                 \
  int64_t fsz[5] = {d->g, d->k, d->c, d->y, d->x};                             \
  int64_t isz[5] = {d->n, d->g, d->c, d->hi, d->wi};                           \
  int64_t osz[5] = {d->n, d->g, d->k, d->ho, d->wo};                           \
  if (layout_strides(fil_layout, "gkcyx", fsz, fs) ||                          \
      layout_strides(in_layout, "ngchw", isz, is) ||                           \
      layout_strides(out_layout, "ngkhw", osz, os))                            \
    return -1;                                                                 \
  /* output loop order = output layout order */                                \
  int ord[5];                                                                  \
  int64_t ext[5];                                                              \
  for (int p = 0; p < 5; ++p) {                                                \
    ord[p] = (int)(strchr("ngkhw", out_layout[p]) - "ngkhw");                  \
    ext[p] = osz[ord[p]];                                                      \
  }                                                                            \
  int64_t total = ext[0] * ext[1] * ext[2] * ext[3] * ext[4];                  \
  if (out_end > total)                                                         \
    out_end = total;                                                           \
  int nt = orc_threads(threads);                                               \
  (void)nt;                                                                    \
  _Pragma("omp parallel for num_threads(nt) schedule(static)")                 \
  for (int64_t flat = out_begin; flat < out_end; ++flat) {                     \
    int64_t idx[5]; /* n g k h w */                                            \
    int64_t rem = flat;                                                        \
    for (int p = 4; p >= 0; --p) {                                             \
      idx[ord[p]] = rem % ext[p];                                              \
      rem /= ext[p];                                                           \
    }                                                                          \
    int64_t n = idx[0], g = idx[1], k = idx[2], ho = idx[3], wo = idx[4];      \
    ACC_T acc = 0;                                                             \
    for (int64_t c = 0; c < d->c; ++c)                                         \
      for (int64_t y = 0; y < d->y; ++y)                                       \
        for (int64_t x = 0; x < d->x; ++x) {                                   \
          int64_t hi = ho * d->stride_h + y * d->dil_h - d->pad_h;             \
          int64_t wi = wo * d->stride_w + x * d->dil_w - d->pad_w;             \
          if (hi < 0 || hi >= d->hi || wi < 0 || wi >= d->wi)                  \
            continue;                                                          \
          IN_T fv = fil[g * fs[0] + k * fs[1] + c * fs[2] + y * fs[3] +        \
                        x * fs[4]];                                            \
          IN_T iv = in[n * is[0] + g * is[1] + c * is[2] + hi * is[3] +        \
                       wi * is[4]];                                            \
          ACC_T prod = WIDEN(fv) * WIDEN(iv);                                  \
          acc = acc + prod;                                                    \
        }                                                                      \
    out[n * os[0] + g * os[1] + k * os[2] + ho * os[3] + wo * os[4]] = acc;    \
  }                                                                            \
  return 0;

#define WIDEN_F(v) (v)
#define WIDEN_I(v) ((int64_t)(v))

/* out_begin/out_end: range of flattened output positions (in output-layout
 * order) to compute -- a bounded sample for timing; pass 0 and INT64_MAX
 * for everything. */
ORC_EXPORT int orc_conv_fwd_f32(const float *fil, const float *in, float *out,
                                const char *fil_layout, const char *in_layout,
                                const char *out_layout, const orc_conv_dims *d,
                                int64_t out_begin, int64_t out_end,
                                int threads) {
  CONV_BODY(float, float, WIDEN_F)
}

/* int8: widened to int64 BEFORE the multiply (deviation from
 * rocmlir-gen.cpp:1955-1960, which multiplies in i8). */
ORC_EXPORT int orc_conv_fwd_i8(const int8_t *fil, const int8_t *in,
                               int64_t *out, const char *fil_layout,
                               const char *in_layout, const char *out_layout,
                               const orc_conv_dims *d, int64_t out_begin,
                               int64_t out_end, int threads) {
  CONV_BODY(int64_t, int8_t, WIDEN_I)
}

/* ------------------------------------------------------------------ */
/* backward convolutions (same generator, rocmlir-gen.cpp:1715-1997)   */
/* ------------------------------------------------------------------ */
/* Backward data: loop nest = the five INPUT dimensions in input-layout order,
 * then k, then y, x (rocmlir-gen.cpp:1817-1821);
 *   out_tmp = in_idx + pad - fil_idx * dilation          (:1895-1897)
 * contributes only when out_tmp % stride == 0 and out_tmp / stride lies in
 * [0, out extent) (:1786-1804); in += filter * out (:1938-1945, :1965-1969). */
ORC_EXPORT int orc_conv_bwd_data_f32(const float *fil, float *in, const float *out, const char *fil_layout,
                                     const char *in_layout, const char *out_layout, const orc_conv_dims *d,
                                     int threads) {
  int64_t fs[5], is[5], os[5];
  int64_t fsz[5] = {d->g, d->k, d->c, d->y, d->x};
  int64_t isz[5] = {d->n, d->g, d->c, d->hi, d->wi};
  int64_t osz[5] = {d->n, d->g, d->k, d->ho, d->wo};
  if (layout_strides(fil_layout, "gkcyx", fsz, fs) || layout_strides(in_layout, "ngchw", isz, is) ||
      layout_strides(out_layout, "ngkhw", osz, os))
    return -1;
  int ord[5];
  int64_t ext[5];
  for (int p = 0; p < 5; ++p) {
    ord[p] = (int)(strchr("ngchw", in_layout[p]) - "ngchw");
    ext[p] = isz[ord[p]];
  }
  int64_t total = ext[0] * ext[1] * ext[2] * ext[3] * ext[4];
  int nt = orc_threads(threads);
  (void)nt;
  _Pragma("omp parallel for num_threads(nt) schedule(static)")
  for (int64_t flat = 0; flat < total; ++flat) {
    int64_t idx[5]; /* n g c h w */
    int64_t rem = flat;
    for (int p = 4; p >= 0; --p) {
      idx[ord[p]] = rem % ext[p];
      rem /= ext[p];
    }
    int64_t n = idx[0], g = idx[1], c = idx[2], hi = idx[3], wi = idx[4];
    float acc = 0.0f;
    for (int64_t k = 0; k < d->k; ++k)
      for (int64_t y = 0; y < d->y; ++y)
        for (int64_t x = 0; x < d->x; ++x) {
          int64_t th = hi + d->pad_h - y * d->dil_h, tw = wi + d->pad_w - x * d->dil_w;
          if (th < 0 || tw < 0 || th % d->stride_h != 0 || tw % d->stride_w != 0)
            continue;
          int64_t ho = th / d->stride_h, wo = tw / d->stride_w;
          if (ho >= d->ho || wo >= d->wo)
            continue;
          float fv = fil[g * fs[0] + k * fs[1] + c * fs[2] + y * fs[3] + x * fs[4]];
          float ov = out[n * os[0] + g * os[1] + k * os[2] + ho * os[3] + wo * os[4]];
          float prod = fv * ov;
          acc = acc + prod;
        }
    in[n * is[0] + g * is[1] + c * is[2] + hi * is[3] + wi * is[4]] = acc;
  }
  return 0;
}

/* Backward weight: loop nest = the five FILTER dimensions in filter-layout
 * order, then n, then ho, wo (rocmlir-gen.cpp:1822-1826);
 *   in_idx = out_idx * stride + fil_idx * dilation - pad  (:1905-1910)
 * in bounds (:1786-1804); filter += out * in (:1930-1937, :1965-1969). */
ORC_EXPORT int orc_conv_bwd_weight_f32(float *fil, const float *in, const float *out, const char *fil_layout,
                                       const char *in_layout, const char *out_layout, const orc_conv_dims *d,
                                       int threads) {
  int64_t fs[5], is[5], os[5];
  int64_t fsz[5] = {d->g, d->k, d->c, d->y, d->x};
  int64_t isz[5] = {d->n, d->g, d->c, d->hi, d->wi};
  int64_t osz[5] = {d->n, d->g, d->k, d->ho, d->wo};
  if (layout_strides(fil_layout, "gkcyx", fsz, fs) || layout_strides(in_layout, "ngchw", isz, is) ||
      layout_strides(out_layout, "ngkhw", osz, os))
    return -1;
  int ord[5];
  int64_t ext[5];
  for (int p = 0; p < 5; ++p) {
    ord[p] = (int)(strchr("gkcyx", fil_layout[p]) - "gkcyx");
    ext[p] = fsz[ord[p]];
  }
  int64_t total = ext[0] * ext[1] * ext[2] * ext[3] * ext[4];
  int nt = orc_threads(threads);
  (void)nt;
  _Pragma("omp parallel for num_threads(nt) schedule(static)")
  for (int64_t flat = 0; flat < total; ++flat) {
    int64_t idx[5]; /* g k c y x */
    int64_t rem = flat;
    for (int p = 4; p >= 0; --p) {
      idx[ord[p]] = rem % ext[p];
      rem /= ext[p];
    }
    int64_t g = idx[0], k = idx[1], c = idx[2], y = idx[3], x = idx[4];
    float acc = 0.0f;
    for (int64_t n = 0; n < d->n; ++n)
      for (int64_t ho = 0; ho < d->ho; ++ho)
        for (int64_t wo = 0; wo < d->wo; ++wo) {
          int64_t hi = ho * d->stride_h + y * d->dil_h - d->pad_h;
          int64_t wi = wo * d->stride_w + x * d->dil_w - d->pad_w;
          if (hi < 0 || hi >= d->hi || wi < 0 || wi >= d->wi)
            continue;
          float ov = out[n * os[0] + g * os[1] + k * os[2] + ho * os[3] + wo * os[4]];
          float iv = in[n * is[0] + g * is[1] + c * is[2] + hi * is[3] + wi * is[4]];
          float prod = ov * iv;
          acc = acc + prod;
        }
    fil[g * fs[0] + k * fs[1] + c * fs[2] + y * fs[3] + x * fs[4]] = acc;
  }
  return 0;
}

/* ------------------------------------------------------------------ */
/* attention (rocmlir-gen.cpp:2507-2638)                               */
/* ------------------------------------------------------------------ */
/* Storage shapes (rocmlir-gen.cpp:2149-2200):
 *   Q [G,seq_q,d_qk]  (transQ: [G,d_qk,seq_q])
 *   K [G,d_qk,seq_k]  (transK: [G,seq_k,d_qk])
 *   V [G,seq_k,d_v]   (transV: [G,d_v,seq_k])
 *   O [G,seq_q,d_v]   (transO: [G,d_v,seq_q])
 *   scale_t, bias_t: optional [G,seq_q,seq_k] tensors (may be NULL).
 * Op order: S = Q*K ; S *= scale_t ; S *= scale ; S += bias_t ;
 * m = rowmax ; e = exp(S - m) ; l = rowsum ; P = e * (1/l) ; O = P*V.
 * `scale` is the scalar form of the pre-softmax multiply (a splat constant
 * in the reference's MIGraphX tests); pass 1.0f for none.
 * All arithmetic in f32 (deviation noted in the file header).
 * q_begin/q_end restrict the computed query rows per g. */
static void attention_f32(const float *Q, const float *K,
                          const float *V, const float *scale_t,
                          const float *bias_t, const int8_t *mask, const float *other, float scale, float *O,
                          int64_t G, int64_t sq, int64_t sk,
                          int64_t dqk, int64_t dv, int transQ,
                          int transK, int transV, int transO,
                          int64_t q_begin, int64_t q_end, int threads) {
  int64_t q_rs = transQ ? 1 : dqk, q_ds = transQ ? sq : 1;
  int64_t k_ds = transK ? 1 : sk, k_js = transK ? dqk : 1;
  int64_t v_js = transV ? 1 : dv, v_es = transV ? sk : 1;
  int64_t o_rs = transO ? 1 : dv, o_es = transO ? sq : 1;
  int nt = orc_threads(threads);
  int64_t rows = q_end - q_begin;
  (void)nt;
#pragma omp parallel num_threads(nt)
  {
    float *s = (float *)malloc((size_t)sk * sizeof(float));
#pragma omp for collapse(2) schedule(static)
    for (int64_t g = 0; g < G; ++g) {
      for (int64_t ri = 0; ri < rows; ++ri) {
        int64_t i = q_begin + ri;
        const float *q = Q + g * sq * dqk + i * q_rs;
        const float *kk = K + g * sk * dqk;
        const float *vv = V + g * sk * dv;
        float *o = O + g * sq * dv + i * o_rs;
        for (int64_t j = 0; j < sk; ++j) {
          float acc = 0.0f;
          for (int64_t dd = 0; dd < dqk; ++dd) {
            float prod = q[dd * q_ds] * kk[dd * k_ds + j * k_js];
            acc = acc + prod;
          }
          if (scale_t)
            acc = acc * scale_t[(g * sq + i) * sk + j];
          if (scale != 1.0f)
            acc = acc * scale;
          if (bias_t)
            acc = acc + bias_t[(g * sq + i) * sk + j];
          /* migraphx.where(mask, scores, other) in front of the softmax
           * (mlir/test/fusion/pr-e2e/attention/mixr-attn-where.mlir:11): a select, not an addition */
          if (mask && !mask[(g * sq + i) * sk + j])
            acc = other[(g * sq + i) * sk + j];
          s[j] = acc;
        }
        float m = s[0];
        for (int64_t j = 1; j < sk; ++j)
          m = s[j] > m ? s[j] : m;
        float l = 0.0f;
        for (int64_t j = 0; j < sk; ++j) {
          s[j] = expf(s[j] - m);
          l = l + s[j];
        }
        float inv = 1.0f / l;
        for (int64_t j = 0; j < sk; ++j)
          s[j] = s[j] * inv;
        for (int64_t e = 0; e < dv; ++e) {
          float acc = 0.0f;
          for (int64_t j = 0; j < sk; ++j) {
            float prod = s[j] * vv[j * v_js + e * v_es];
            acc = acc + prod;
          }
          o[e * o_es] = acc;
        }
      }
    }
    free(s);
  }
}

ORC_EXPORT void orc_attention_f32(const float *Q, const float *K,
                                  const float *V, const float *scale_t,
                                  const float *bias_t, float scale, float *O,
                                  int64_t G, int64_t sq, int64_t sk,
                                  int64_t dqk, int64_t dv, int transQ,
                                  int transK, int transV, int transO,
                                  int64_t q_begin, int64_t q_end, int threads) {
  attention_f32(Q, K, V, scale_t, bias_t, NULL, NULL, scale, O, G, sq, sk, dqk, dv, transQ, transK, transV, transO,
                q_begin, q_end, threads);
}

/* The same with a pre-softmax select: where mask[g,i,j] is zero the score is
 * replaced by other[g,i,j] (after the scale tensor, the scale and the bias). */
ORC_EXPORT void orc_attention_where_f32(const float *Q, const float *K, const float *V, const float *scale_t,
                                        const float *bias_t, const int8_t *mask, const float *other, float scale,
                                        float *O, int64_t G, int64_t sq, int64_t sk, int64_t dqk, int64_t dv,
                                        int transQ, int transK, int transV, int transO, int64_t q_begin,
                                        int64_t q_end, int threads) {
  attention_f32(Q, K, V, scale_t, bias_t, mask, other, scale, O, G, sq, sk, dqk, dv, transQ, transK, transV, transO,
                q_begin, q_end, threads);
}

/* softmax over the last axis, the decomposition of
 * MIGraphXToTosa.cpp:1020-1044 (max, sub, exp, sum, reciprocal, mul). */
ORC_EXPORT void orc_softmax_f32(const float *x, float *y, int64_t rows,
                                int64_t cols) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * cols;
    float *yr = y + r * cols;
    float m = xr[0];
    for (int64_t j = 1; j < cols; ++j)
      m = xr[j] > m ? xr[j] : m;
    float l = 0.0f;
    for (int64_t j = 0; j < cols; ++j) {
      yr[j] = expf(xr[j] - m);
      l = l + yr[j];
    }
    float inv = 1.0f / l;
    for (int64_t j = 0; j < cols; ++j)
      yr[j] = yr[j] * inv;
  }
}

/* ------------------------------------------------------------------ */
/* quantisation epilogue (MIGraphXToTosa.cpp:874-982)                  */
/* ------------------------------------------------------------------ */
/* dequantizelinear: y = (float(acc) - float(zp)) * scale. */
ORC_EXPORT void orc_dequantize_i64(const int64_t *acc, int64_t n, float scale,
                                   int32_t zero_point, float *y) {
  for (int64_t i = 0; i < n; ++i) {
    float a = (float)(int32_t)acc[i]; /* i32 accumulator -> f32, RNE */
    float z = (float)zero_point;
    y[i] = (a - z) * scale;
  }
}

/* quantizelinear: q = clamp(cast_i32(x * (1/scale)) + zp, -128, 127), the
 * cast being round-half-even with saturation. */
ORC_EXPORT void orc_quantize_i8(const float *x, int64_t n, float scale,
                                int32_t zero_point, int8_t *q) {
  float inv = 1.0f / scale;
  for (int64_t i = 0; i < n; ++i) {
    float scaled = x[i] * inv;
    int64_t r = round_even_sat(scaled, INT32_MIN, INT32_MAX);
    r += zero_point;
    if (r < -128)
      r = -128;
    if (r > 127)
      r = 127;
    q[i] = (int8_t)r;
  }
}

/* The same two with one scale and one zero point per output channel: the
 * reference broadcasts scale and zero-point tensors shaped like one value per
 * channel through the same element-wise chain (MIGraphXToTosa.cpp:874-982;
 * mlir/test/fusion/resnet50-e2e/mixr-resnet-fusion-case-1-quantization.mlir:8-9
 * passes a <1x128x1x1xf32> scale to both).  x is [rows][channels]; a NULL
 * zero-point vector means zero. */
ORC_EXPORT void orc_dequantize_i64_per_channel(const int64_t *acc, int64_t rows, int64_t channels,
                                               const float *scale, const int32_t *zero_point, float *y) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < channels; ++c) {
      float a = (float)(int32_t)acc[r * channels + c];
      float z = (float)(zero_point ? zero_point[c] : 0);
      y[r * channels + c] = (a - z) * scale[c];
    }
}

ORC_EXPORT void orc_quantize_i8_per_channel(const float *x, int64_t rows, int64_t channels, const float *scale,
                                            const int32_t *zero_point, int8_t *q) {
  for (int64_t c = 0; c < channels; ++c) {
    float inv = 1.0f / scale[c]; /* tosa.reciprocal, then the multiplication */
    for (int64_t r = 0; r < rows; ++r) {
      float scaled = x[r * channels + c] * inv;
      int64_t v = round_even_sat(scaled, INT32_MIN, INT32_MAX);
      v += zero_point ? zero_point[c] : 0;
      if (v < -128)
        v = -128;
      if (v > 127)
        v = 127;
      q[r * channels + c] = (int8_t)v;
    }
  }
}

/* y = x * scale (+ bias[col]) : the float epilogue (rescale by the product
 * of per-tensor scales, optional per-column bias). */
ORC_EXPORT void orc_scale_bias_f32(float *x, int64_t rows, int64_t cols,
                                   float scale, const float *bias) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      float v = x[r * cols + c] * scale;
      if (bias)
        v = v + bias[c];
      x[r * cols + c] = v;
    }
}

/* ------------------------------------------------------------------ */
/* verifier (conv-validation-wrappers.cpp:104-285)                     */
/* ------------------------------------------------------------------ */
typedef struct {
  double rms;          /* sqrt(sum d^2) / (maxMag * sqrt(N)) */
  double max_abs_diff; /* max |val - gpu| */
  double max_rel_diff; /* max |val - gpu| / |val| over val != 0 */
  double ave_abs_diff;
  double max_mag;
  int32_t pass_rms, pass_abs, pass_rel;
} orc_verify_result;

ORC_EXPORT void orc_verify_float(const float *gpu, const float *val, int64_t n,
                                 float thr_rms, float thr_abs, float thr_rel,
                                 orc_verify_result *res) {
  float maxAbsDiff = 0.0f, maxMag = 0.0f;
  double sumAbsDiff = 0.0, maxRelDiff = 0.0, sumDiffSq = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    float valNum = val[i], gpuNum = gpu[i];
    float maxNum = fmaxf(fabsf(valNum), fabsf(gpuNum));
    maxMag = fmaxf(maxMag, maxNum);
    if (valNum == gpuNum)
      continue;
    if (isinf(valNum))
      valNum = valNum > 0 ? 65504.0f : -65504.0f;
    float absDiff = fabsf(valNum - gpuNum);
    if (absDiff > maxAbsDiff)
      maxAbsDiff = absDiff;
    sumAbsDiff += (double)absDiff;
    if (valNum != 0.0f) {
      double relDiff = (double)absDiff / (double)fabsf(valNum);
      if (relDiff > maxRelDiff)
        maxRelDiff = relDiff;
    }
    sumDiffSq += (double)absDiff * (double)absDiff;
  }
  double rms = sqrt(sumDiffSq) / ((double)maxMag * sqrt((double)n));
  res->rms = rms;
  res->max_abs_diff = maxAbsDiff;
  res->max_rel_diff = maxRelDiff;
  res->ave_abs_diff = sumAbsDiff / (double)n;
  res->max_mag = maxMag;
  res->pass_rms = rms <= thr_rms;
  res->pass_abs = maxAbsDiff <= thr_abs;
  res->pass_rel = maxRelDiff <= thr_rel;
}

/* returns the number of mismatching elements; *overflow counts validation
 * values that do not fit in int32 (conv-validation-wrappers.cpp:232-285). */
ORC_EXPORT int64_t orc_verify_int32_int64(const int32_t *gpu,
                                          const int64_t *val, int64_t n,
                                          int64_t *overflow,
                                          int64_t *max_abs_diff) {
  int64_t fail = 0, ovf = 0, mad = 0;
  for (int64_t i = 0; i < n; ++i) {
    int64_t v = val[i];
    if (v > INT32_MAX || v < INT32_MIN)
      ovf++;
    if ((int64_t)gpu[i] != v) {
      fail++;
      int64_t dabs = llabs(v - (int64_t)gpu[i]);
      if (dabs > mad)
        mad = dabs;
    }
  }
  if (overflow)
    *overflow = ovf;
  if (max_abs_diff)
    *max_abs_diff = mad;
  return fail;
}

/* ------------------------------------------------------------------ */
/* data fill (rocmlir-gen.cpp:1325-1486; wrappers.cpp:27-50)           */
/* ------------------------------------------------------------------ */
/* "-rand fixed": pattern cycled by flat index mod 3. */
ORC_EXPORT void orc_fill_fixed(float *x, int64_t n, int is_int) {
  static const float fpat[3] = {0.5f, -1.0f, 0.75f};
  static const float ipat[3] = {1.0f, -1.0f, 2.0f};
  for (int64_t i = 0; i < n; ++i)
    x[i] = is_int ? ipat[i % 3] : fpat[i % 3];
}

ORC_EXPORT void orc_seed(uint32_t seed) { srand(seed); }

/* "-rand N": integers in [min,max) or floats min + (max-min)*rand()/RAND_MAX,
 * drawn element by element from libc rand(). */
ORC_EXPORT void orc_fill_rand(float *x, int64_t n, int min, int max,
                              int as_float) {
  for (int64_t i = 0; i < n; ++i) {
    if (min == max) {
      x[i] = as_float ? (float)min * 0.1f : (float)min;
    } else if (as_float) {
      x[i] = (float)((max - min) * (double)rand() / (double)RAND_MAX) +
             (float)min;
    } else {
      int16_t r = (int16_t)((rand() % (max - min)) + min);
      x[i] = (float)r;
    }
  }
}
