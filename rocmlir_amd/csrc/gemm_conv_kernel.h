// Tiled MFMA contraction kernel for gfx950, general-layout body: GEMM and
// implicit-GEMM forward convolution share one main loop and differ only in
// how a tile row is addressed in global memory.  This body gathers operands
// element by element, so it takes ANY strides (all transposes, NCHW, odd K,
// unaligned rows); operands made of K-contiguous 16-byte chunks take the
// direct-to-LDS body in gemm_conv_dlds.h instead, which shares the tile
// decode, the MFMA mapping and the epilogue defined here.
//
// Behaviour replaced: the reference's gridwise GEMM schedule
// (mlir/lib/Dialect/Rock/Transforms/GridwiseGemmToBlockwise.cpp:2409-2811)
// and its conv->GEMM views (mlir/lib/Dialect/Rock/Transforms/ConvToGemm.cpp:
// 1190-1393).  Nothing of that code is reused; the design is:
//
//   * block tile BM x BN, K advanced 128 BYTES per iteration for every
//     element type (128 int8/fp8, 64 f16/bf16, 32 f32 elements);
//   * global -> registers -> LDS, two LDS stages, one barrier per iteration;
//   * LDS tile = rows of 8 sixteen-byte chunks, chunk index XOR-swizzled with
//     the row so that the 32 rows an MFMA operand reads at one chunk index
//     hit distinct 16-byte bank groups;
//   * the problem's B rows feed the MFMA row operand and its A rows the
//     column operand, so every lane ends up with 4 CONSECUTIVE n of one m and
//     the C tile is written with 4/8/16-byte stores;
//   * out-of-range rows and the K tail are zero-filled on load, never read
//     past the tensor; the epilogue (scale, zero point, bias, cast) runs on
//     the accumulators in registers.
#pragma once
#include <type_traits>
#include "mfma_gfx950.h"

namespace rk {

enum LoaderKind : int {
  LD_ROWS_FAST = 0,     // K-contiguous rows, 16-byte aligned chunks (direct-to-LDS body)
  LD_ROWS_GENERIC = 1,  // arbitrary element strides, element-wise
  LD_CONV_IN_FAST = 2,  // convolution input, channel-contiguous, C*ES % 16 == 0 (direct-to-LDS body)
  LD_CONV_IN_GENERIC = 3,
  LD_CONV_FIL_GENERIC = 4,
  LD_COLS_FAST = 5,     // GEMM operand stored K-major (its M or N index contiguous), 16-byte aligned chunks
  LD_CONV_COLS = 6,     // forward im2col matrix as a K-major operand (reduction over pixels): filter gradient
  LD_CONV_IN_RUNS = 7   // as LD_CONV_IN_FAST over channel runs whose last chunk holds bytes that are not data
};

constexpr int kChunk = 16;       // bytes
constexpr int kRowBytes = 128;   // K bytes per tile row
constexpr int kChunksPerRow = 8;

__device__ __forceinline__ int swizzle(int row, int chunk) {
  return chunk ^ ((row >> 1) & 7);
}

// ---------------------------------------------------------------------------
// Work-item decode: 1-D grid -> (g, tile_m, tile_n) with the XCD round-robin
// undone and tile rows walked in groups so that co-resident blocks share
// operand tiles in one XCD's L2 (the reference has the same idea at
// mlir/lib/Dialect/Rock/Transforms/GridLayoutEmitter.cpp:38-109).
// ---------------------------------------------------------------------------
__device__ __forceinline__ void decode_block(int tiles_m, int tiles_n, int G,
                                             int group_m, int xcd_remap,
                                             int &g, int &tm, int &tn) {
  int bid = blockIdx.x;
  const int tiles = tiles_m * tiles_n;
  const int total = tiles * G;
  if (xcd_remap) {
    const int per = total >> 3;
    if (bid < (per << 3))
      bid = (bid & 7) * per + (bid >> 3);
  }
  g = bid / tiles;
  const int t = bid - g * tiles;
  const int group_sz = group_m * tiles_n;
  const int grp = t / group_sz;
  const int first_m = grp * group_m;
  const int rows_here = min(tiles_m - first_m, group_m);
  const int in_grp = t - grp * group_sz;
  tm = first_m + in_grp % rows_here;
  tn = in_grp / rows_here;
}

// ---------------------------------------------------------------------------
// Row loaders.  Each thread owns NCH chunks of the tile: chunk column
// c = tid & 7 (fixed), rows (tid >> 3) + i * (NT / 8).
// ---------------------------------------------------------------------------
template <int DT, int ROWS, int NT> struct TileGeom {
  static constexpr int ES = MmaTraits<DT>::ES;
  static constexpr int EPC = kChunk / ES; // elements per chunk
  static constexpr int BKE = kRowBytes / ES; // K elements per tile
  static constexpr int TOTAL = ROWS * kChunksPerRow;
  static constexpr int NCH = (TOTAL + NT - 1) / NT;
  static constexpr int ROW_STEP = NT / kChunksPerRow;
  static_assert(NT % kChunksPerRow == 0, "thread count must be a multiple of 8");
};

// Assemble one chunk element by element through a caller-supplied fetch.
template <int DT, typename F>
__device__ __forceinline__ v4i gather_chunk(F fetch) {
  constexpr int ES = MmaTraits<DT>::ES;
  v4i out = {0, 0, 0, 0};
  if constexpr (ES == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      out[e] = (int)fetch(e);
  } else if constexpr (ES == 2) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      out[e >> 1] |= (int)(fetch(e) & 0xffffu) << (16 * (e & 1));
  } else {
#pragma unroll
    for (int e = 0; e < 16; ++e)
      out[e >> 2] |= (int)(fetch(e) & 0xffu) << (8 * (e & 3));
  }
  return out;
}

template <int ES>
__device__ __forceinline__ uint32_t load_elem(const void *base, int64_t idx) {
  if constexpr (ES == 4)
    return ((const uint32_t *)base)[idx];
  else if constexpr (ES == 2)
    return ((const uint16_t *)base)[idx];
  else
    return ((const uint8_t *)base)[idx];
}

// Arbitrary strides: element (row, k) at base[row*rs + k*ks].
template <int DT, int ROWS, int NT> struct RowsGeneric {
  using Gm = TileGeom<DT, ROWS, NT>;
  const void *base;
  int64_t rs, ks;
  int row0, rows_total, K, tid;

  __device__ __forceinline__ void init(const void *b, int64_t row_stride,
                                       int64_t k_stride, int r0, int rt, int k,
                                       int t) {
    base = b; rs = row_stride; ks = k_stride; row0 = r0; rows_total = rt; K = k; tid = t;
  }
  __device__ __forceinline__ void load(int kt, v4i (&regs)[Gm::NCH]) const {
    const int c = tid & 7;
#pragma unroll
    for (int i = 0; i < Gm::NCH; ++i) {
      int r = (tid >> 3) + i * Gm::ROW_STEP;
      int gr = row0 + r;
      bool rok = (r < ROWS) && (gr < rows_total);
      int k0 = kt * Gm::BKE + c * Gm::EPC;
      regs[i] = gather_chunk<DT>([&](int e) -> uint32_t {
        int k = k0 + e;
        return (rok && k < K) ? load_elem<Gm::ES>(base, (int64_t)gr * rs + (int64_t)k * ks) : 0u;
      });
    }
  }
};

// Decompose the reduction index for the generic convolution loaders.
__device__ __forceinline__ void conv_split_k(const RockConvParams &p, int k,
                                             int &c, int &y, int &x) {
  if (p.k_order_yxc) {
    int tap = k / p.c;
    c = k - tap * p.c;
    y = tap / p.x;
    x = tap - y * p.x;
  } else {
    int yx = p.y * p.x;
    c = k / yx;
    int tap = k - c * yx;
    y = tap / p.x;
    x = tap - y * p.x;
  }
}

template <int DT, int ROWS, int NT> struct ConvInGeneric {
  using Gm = TileGeom<DT, ROWS, NT>;
  const void *in;
  const RockConvParams *p;
  int g, row0, tid;
  __device__ __forceinline__ void init(const void *i, const RockConvParams &cp,
                                       int gg, int r0, int t) {
    in = i; p = &cp; g = gg; row0 = r0; tid = t;
  }
  __device__ __forceinline__ void load(int kt, v4i (&regs)[Gm::NCH]) const {
    const int cidx = tid & 7;
#pragma unroll
    for (int i = 0; i < Gm::NCH; ++i) {
      int r = (tid >> 3) + i * Gm::ROW_STEP;
      int m = row0 + r;
      bool rok = (r < ROWS) && (m < p->M);
      int mm = min(m, p->M - 1);
      int n = mm / (p->ho * p->wo);
      int rem = mm - n * (p->ho * p->wo);
      int ho = rem / p->wo, wo = rem - (rem / p->wo) * p->wo;
      int k0 = kt * Gm::BKE + cidx * Gm::EPC;
      regs[i] = gather_chunk<DT>([&](int e) -> uint32_t {
        int k = k0 + e;
        if (!rok || k >= p->K) return 0u;
        int c, y, x;
        conv_split_k(*p, k, c, y, x);
        int hi = ho * p->stride_h + y * p->dil_h - p->pad_h;
        int wi = wo * p->stride_w + x * p->dil_w - p->pad_w;
        if (hi < 0 || hi >= p->hi || wi < 0 || wi >= p->wi) return 0u;
        int64_t idx = (int64_t)n * p->in_ns + (int64_t)g * p->in_gs + (int64_t)c * p->in_cs +
                      (int64_t)hi * p->in_hs + (int64_t)wi * p->in_ws;
        return load_elem<Gm::ES>(in, idx);
      });
    }
  }
};

template <int DT, int ROWS, int NT> struct ConvFilGeneric {
  using Gm = TileGeom<DT, ROWS, NT>;
  const void *fil;
  const RockConvParams *p;
  int g, row0, tid;
  __device__ __forceinline__ void init(const void *f, const RockConvParams &cp,
                                       int gg, int r0, int t) {
    fil = f; p = &cp; g = gg; row0 = r0; tid = t;
  }
  __device__ __forceinline__ void load(int kt, v4i (&regs)[Gm::NCH]) const {
    const int cidx = tid & 7;
#pragma unroll
    for (int i = 0; i < Gm::NCH; ++i) {
      int r = (tid >> 3) + i * Gm::ROW_STEP;
      int ko = row0 + r;
      bool rok = (r < ROWS) && (ko < p->N);
      int k0 = kt * Gm::BKE + cidx * Gm::EPC;
      regs[i] = gather_chunk<DT>([&](int e) -> uint32_t {
        int k = k0 + e;
        if (!rok || k >= p->K) return 0u;
        int c, y, x;
        conv_split_k(*p, k, c, y, x);
        int64_t idx = (int64_t)g * p->fil_gs + (int64_t)ko * p->fil_ks + (int64_t)c * p->fil_cs +
                      (int64_t)y * p->fil_ys + (int64_t)x * p->fil_xs;
        return load_elem<Gm::ES>(fil, idx);
      });
    }
  }
};

// ---------------------------------------------------------------------------
// LDS tile store / fragment read
// ---------------------------------------------------------------------------
template <int DT, int ROWS, int NT>
__device__ __forceinline__ void store_tile(char *lds, const v4i (&regs)[TileGeom<DT, ROWS, NT>::NCH], int tid) {
  using Gm = TileGeom<DT, ROWS, NT>;
  const int c = tid & 7;
#pragma unroll
  for (int i = 0; i < Gm::NCH; ++i) {
    int r = (tid >> 3) + i * Gm::ROW_STEP;
    if (Gm::TOTAL % NT == 0 || r < ROWS)
      *(v4i *)(lds + r * kRowBytes + swizzle(r, c) * kChunk) = regs[i];
  }
}

// Fragment of one 32-row block: lane (row = lane % 32, half = lane / 32)
// takes chunk  step*2*CHUNKS + 2*c + half  for c in [0, CHUNKS).
template <int DT>
__device__ __forceinline__ Frag<DT> read_frag(const char *lds, int row, int step, int half) {
  Frag<DT> f;
  constexpr int CH = MmaTraits<DT>::CHUNKS;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    int chunk = step * 2 * CH + 2 * c + half;
    f.c[c] = *(const v4i *)(lds + row * kRowBytes + swizzle(row, chunk) * kChunk);
  }
  return f;
}

// ---------------------------------------------------------------------------
// Epilogue: convert 4 consecutive output channels of one row, pack them in
// the output type, store them.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int out_elem_size(int od) {
  return (od == ROCK_F32 || od == ROCK_I32) ? 4 : (od == ROCK_F16 || od == ROCK_BF16) ? 2 : 1;
}

// relu and clip cost an instruction or two and are applied where the
// accumulators sit.  The transcendental activations are long routines; a
// copy per accumulator element of an unrolled epilogue would dominate the code
// object, so the tiled kernels run them in a rolled loop over values parked in
// LDS (dl_epilogue) and the element-wise kernels call them out of line.
__device__ __forceinline__ bool activation_is_slow(const RockEpilogue &e) { return e.activation > ROCK_ACT_CLIP; }

// relu and clip are one clamp: the host resolves the bounds (relu: [0, +inf))
__device__ __forceinline__ float activation_fast(float v, const RockEpilogue &e) {
  return fminf(fmaxf(v, e.act_lo), e.act_hi);
}

__device__ __forceinline__ float activation_slow(float v, int activation) {
  switch (activation) { // uniform
  case ROCK_ACT_SIGMOID: return __frcp_rn(1.0f + __expf(-v)); // hardware exp2 and reciprocal: ~1e-7 relative
  case ROCK_ACT_TANH: return tanhf(v);
  case ROCK_ACT_ERF: return erff(v);
  case ROCK_ACT_GELU: return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
  case ROCK_ACT_EXP: return expf(v);
  default: return v;
  }
}
__device__ __attribute__((noinline)) float activation_slow_call(float v, int activation) {
  return activation_slow(v, activation);
}

// One element of a tensor of the output type, widened.
template <int OD> __device__ __forceinline__ float load_out_elem(const void *base, int64_t idx) {
  if constexpr (OD == ROCK_F32)
    return ((const float *)base)[idx];
  else if constexpr (OD == ROCK_F16)
    return (float)((const _Float16 *)base)[idx];
  else if constexpr (OD == ROCK_BF16)
    return __builtin_bit_cast(float, (uint32_t)((const uint16_t *)base)[idx] << 16);
  else if constexpr (OD == ROCK_I8)
    return (float)((const int8_t *)base)[idx];
  else if constexpr (OD == ROCK_FP8)
    return e4m3fn_to_f32(((const uint8_t *)base)[idx]);
  else if constexpr (OD == ROCK_BF8)
    return e5m2_to_f32(((const uint8_t *)base)[idx]);
  else
    return (float)((const int *)base)[idx];
}

// The same with the type as a run-time value (uniform across the block).
__device__ __forceinline__ float load_out_elem_rt(const void *base, int64_t idx, int od) {
  switch (od) {
  case ROCK_F32: return load_out_elem<ROCK_F32>(base, idx);
  case ROCK_F16: return load_out_elem<ROCK_F16>(base, idx);
  case ROCK_BF16: return load_out_elem<ROCK_BF16>(base, idx);
  case ROCK_I8: return load_out_elem<ROCK_I8>(base, idx);
  case ROCK_FP8: return load_out_elem<ROCK_FP8>(base, idx);
  case ROCK_BF8: return load_out_elem<ROCK_BF8>(base, idx);
  default: return load_out_elem<ROCK_I32>(base, idx);
  }
}

template <int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// Steps 1-3 of the epilogue for 4 consecutive output channels of one row:
// acc[r] belongs to channel n0 + r.  `res` is the residual tensor and res_off
// the element offset of (row, n0) in it, channels res_ns apart; null when the
// epilogue names no residual operation or the row is out of range.
// element n of a per-channel zero-point vector of int32 or int8 elements
__device__ __forceinline__ float chan_zero_point(const void *vec, int n, bool is_i8) {
  return is_i8 ? (float)((const int8_t *)vec)[n] : (float)((const int *)vec)[n];
}

// CHAN: the per-channel vectors of RockEpilogue::chan_flags are honoured (the
// kernels with the rolled epilogue and the element-wise kernels); the plain
// tiled kernels are compiled without them.
template <bool INT_ACC, int OD, bool CHAN = false, typename Acc4>
__device__ __forceinline__ void epilogue_affine4(const Acc4 &acc, const RockEpilogue &e, const void *aux,
                                                 int n0, int n_limit, const void *res, int64_t res_off,
                                                 int64_t res_ns, float (&v)[4]) {
  // the four bias values as one 16-byte load where the group is whole (n0 is a
  // multiple of 4 and the vector starts on a 16-byte boundary like its tensor)
  float b4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (e.has_bias) {
    if (n0 + 3 < n_limit) {
      const v4f b = *(const v4f *)((const float *)aux + n0);
      b4[0] = b[0]; b4[1] = b[1]; b4[2] = b[2]; b4[3] = b[3];
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n0 + r < n_limit)
          b4[r] = ((const float *)aux)[n0 + r];
    }
  }
  float s4[4] = {e.scale, e.scale, e.scale, e.scale};
  float z4[4] = {(float)e.zero_point, (float)e.zero_point, (float)e.zero_point, (float)e.zero_point};
  if constexpr (CHAN) {
    if (e.chan_flags & (ROCK_CHAN_SCALE | ROCK_CHAN_ZP)) { // uniform
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n0 + r < n_limit) {
          if (e.chan_flags & ROCK_CHAN_SCALE)
            s4[r] = e.scale_vec[n0 + r];
          if (e.chan_flags & ROCK_CHAN_ZP)
            z4[r] = chan_zero_point(e.zero_point_vec, n0 + r, (e.chan_flags & ROCK_CHAN_ZP_I8) != 0);
        }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float f;
    if constexpr (INT_ACC)
      f = ((float)(int)acc[r] - z4[r]) * s4[r];
    else
      f = (float)acc[r] * s4[r];
    if (e.has_bias)
      f = f + b4[r];
    if (res && n0 + r < n_limit) {
      const float rv = load_out_elem<OD>(res, res_off + r * res_ns);
      f = e.residual_op == ROCK_RES_ADD ? f + rv : f * rv;
    }
    v[r] = f;
  }
}

// Step 5: 4 values narrowed to the output type and packed back to back in the
// low 4*elem_size bytes.
// n0 / n_limit: the channels the four values belong to (read only for a
// per-channel requantisation, CHAN)
template <int OD, bool CHAN = false>
__device__ __forceinline__ v4i epilogue_pack4(const float (&v)[4], const RockEpilogue &e, int n0 = 0, int n_limit = 0) {
  v4i out = {0, 0, 0, 0};
  if constexpr (OD == ROCK_F32 || OD == ROCK_I32) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      out[r] = __builtin_bit_cast(int, v[r]);
  } else if constexpr (OD == ROCK_F16) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      _Float16 hv = (_Float16)v[r];
      out[r >> 1] |= (int)__builtin_bit_cast(uint16_t, hv) << (16 * (r & 1));
    }
  } else if constexpr (OD == ROCK_BF16) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      __bf16 hv = (__bf16)v[r];
      out[r >> 1] |= (int)__builtin_bit_cast(uint16_t, hv) << (16 * (r & 1));
    }
  } else if constexpr (OD == ROCK_I8) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float inv = e.inv_quant_scale, zp = (float)e.out_zero_point;
      if constexpr (CHAN) {
        if ((e.chan_flags & (ROCK_CHAN_QUANT_SCALE | ROCK_CHAN_OUT_ZP)) && n0 + r < n_limit) { // uniform flags
          if (e.chan_flags & ROCK_CHAN_QUANT_SCALE)
            inv = 1.0f / e.quant_scale_vec[n0 + r]; // tosa.reciprocal, then the multiplication (MIGraphXToTosa.cpp:917-921)
          if (e.chan_flags & ROCK_CHAN_OUT_ZP)
            zp = chan_zero_point(e.out_zero_point_vec, n0 + r, (e.chan_flags & ROCK_CHAN_OUT_ZP_I8) != 0);
        }
      }
      float q = __builtin_rintf(v[r] * inv) + zp;
      out[0] |= ((int)f32_to_i8_sat(q) & 0xff) << (8 * r);
    }
  } else if constexpr (OD == ROCK_FP8) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      out[0] |= (int)f32_to_e4m3fn_sat(v[r]) << (8 * r);
  } else if constexpr (OD == ROCK_BF8) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      out[0] |= (int)f32_to_e5m2_sat(v[r]) << (8 * r);
  }
  return out;
}

__device__ __forceinline__ v4i epilogue_pack4_rt(const float (&v)[4], int od, const RockEpilogue &e, int n0, int n_limit) {
  switch (od) {
  case ROCK_F32: return epilogue_pack4<ROCK_F32>(v, e);
  case ROCK_F16: return epilogue_pack4<ROCK_F16>(v, e);
  case ROCK_BF16: return epilogue_pack4<ROCK_BF16>(v, e);
  case ROCK_I8: return epilogue_pack4<ROCK_I8, true>(v, e, n0, n_limit);
  case ROCK_FP8: return epilogue_pack4<ROCK_FP8>(v, e);
  default: return epilogue_pack4<ROCK_BF8>(v, e);
  }
}

// The whole epilogue for 4 channels.  OD (the output type) is a compile-time
// constant so that the unrolled epilogue is straight-line code.  SLOW_CALL:
// transcendental activations are applied here through an out-of-line call
// (element-wise kernels); otherwise the caller has dealt with them.
template <bool INT_ACC, int OD, bool SLOW_CALL = false, bool CHAN = false, typename Acc4>
__device__ __forceinline__ v4i epilogue_convert4(const Acc4 &acc, const RockEpilogue &e,
                                                 const void *aux, int n0, int n_limit,
                                                 const void *res = nullptr, int64_t res_off = 0,
                                                 int64_t res_ns = 1) {
  if constexpr (INT_ACC && OD == ROCK_I32) { // exact accumulators, optional int32 bias and residual
    v4i v;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = (int)acc[r];
      if (e.has_bias && n0 + r < n_limit)
        v[r] += ((const int *)aux)[n0 + r];
      if (res && n0 + r < n_limit) {
        const int rv = ((const int *)res)[res_off + r * res_ns];
        v[r] = e.residual_op == ROCK_RES_ADD ? v[r] + rv : v[r] * rv;
      }
    }
    return v;
  } else {
    float v[4];
    epilogue_affine4<INT_ACC, OD, CHAN>(acc, e, aux, n0, n_limit, res, res_off, res_ns, v);
    if (SLOW_CALL && activation_is_slow(e)) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        v[r] = activation_slow_call(v[r], e.activation);
    } else if (e.activation) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        v[r] = activation_fast(v[r], e);
    }
    return epilogue_pack4<OD, CHAN>(v, e, n0, n_limit);
  }
}

// Calls f(std::integral_constant<int, OD>) for the run-time output type.
template <bool INT_ACC, typename F>
__device__ __forceinline__ void dispatch_out_dtype(int od, F &&f) {
  switch (od) {
  case ROCK_F32: f(std::integral_constant<int, ROCK_F32>{}); break;
  case ROCK_F16: f(std::integral_constant<int, ROCK_F16>{}); break;
  case ROCK_BF16: f(std::integral_constant<int, ROCK_BF16>{}); break;
  case ROCK_I8: f(std::integral_constant<int, ROCK_I8>{}); break;
  case ROCK_FP8: f(std::integral_constant<int, ROCK_FP8>{}); break;
  case ROCK_BF8: f(std::integral_constant<int, ROCK_BF8>{}); break;
  case ROCK_I32:
    if constexpr (INT_ACC)
      f(std::integral_constant<int, ROCK_I32>{});
    break; // float accumulators written as int32 are not a legal problem
  }
}

template <int OD> struct OutElemSize {
  static constexpr int value = (OD == ROCK_F32 || OD == ROCK_I32) ? 4 : (OD == ROCK_F16 || OD == ROCK_BF16) ? 2 : 1;
};

// `off` is the element offset of channel n0 of this row.
__device__ __forceinline__ void store_packed4(const v4i &raw, int es, void *out_base, int64_t off,
                                              int64_t n_stride, int n0, int n_limit, bool vec_ok) {
  char *o = (char *)out_base;
  if (vec_ok && n0 + 3 < n_limit) {
    if (es == 4)
      *(v4i *)(o + off * 4) = raw;
    else if (es == 2)
      *(v2i *)(o + off * 2) = v2i{raw[0], raw[1]};
    else
      *(int *)(o + off) = raw[0];
    return;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (n0 + r >= n_limit)
      continue;
    int64_t idx = off + r * n_stride;
    if (es == 4)
      ((int *)o)[idx] = raw[r];
    else if (es == 2)
      ((uint16_t *)o)[idx] = (uint16_t)((uint32_t)raw[r >> 1] >> (16 * (r & 1)));
    else
      ((uint8_t *)o)[idx] = (uint8_t)((uint32_t)raw[0] >> (8 * r));
  }
}

// ---- parameter-block adapters ------------------------------------------------
__device__ __forceinline__ int p_batch(const RockGemmParams &p) { return p.G; }
__device__ __forceinline__ int p_batch(const RockConvParams &p) { return p.g; }

// The per-channel values of the epilogue (bias, quantisation vectors) belong to
// output channel g * K + k of a convolution, to column n of a GEMM whatever the
// batch entry: a convolution block of group g moves the pointers on by g * K
// channels before its epilogue indexes them with the channel inside the group.
// (The shares of a split reduction, which run as groups, take no such values.)
__device__ __forceinline__ void group_channel_pointers(RockGemmParams &, const void *&, int) {}
__device__ __forceinline__ void group_channel_pointers(RockConvParams &p, const void *&aux, int g) {
  const int base = g * p.N;
  if (base == 0)
    return;
  RockEpilogue &e = p.epi;
  if (e.has_bias)
    aux = (const char *)aux + (int64_t)base * 4; // f32, or int32 beside int32 results
  if (e.chan_flags & ROCK_CHAN_SCALE)
    e.scale_vec += base;
  if (e.chan_flags & ROCK_CHAN_ZP)
    e.zero_point_vec = (const char *)e.zero_point_vec + (int64_t)base * ((e.chan_flags & ROCK_CHAN_ZP_I8) ? 1 : 4);
  if (e.chan_flags & ROCK_CHAN_QUANT_SCALE)
    e.quant_scale_vec += base;
  if (e.chan_flags & ROCK_CHAN_OUT_ZP)
    e.out_zero_point_vec =
        (const char *)e.out_zero_point_vec + (int64_t)base * ((e.chan_flags & ROCK_CHAN_OUT_ZP_I8) ? 1 : 4);
}

__device__ __forceinline__ bool aligned_for_vec(const void *base, int64_t row_off, int out_dtype) {
  // 4 consecutive outputs stored as one 4/8/16-byte access need that alignment
  int es = out_elem_size(out_dtype);
  return ((((uintptr_t)base) + (uintptr_t)row_off * es) & (uintptr_t)(4 * es - 1)) == 0;
}

__device__ __forceinline__ void out_row_addr(const RockGemmParams &p, int g, int m, const void *base,
                                             int64_t &row_off, int64_t &n_stride, bool &vec_ok) {
  row_off = (int64_t)g * p.c_gs + (int64_t)m * p.c_ms;
  n_stride = p.c_ns;
  vec_ok = (p.c_ns == 1) && aligned_for_vec(base, row_off, p.epi.out_dtype);
}

__device__ __forceinline__ void out_row_addr(const RockConvParams &p, int g, int m, const void *base,
                                             int64_t &row_off, int64_t &n_stride, bool &vec_ok) {
  if (p.out_hs == (int64_t)p.wo * p.out_ws && p.out_ns == (int64_t)p.ho * p.out_hs) {
    // pixels of one group are equally spaced in memory (NHWC-like outputs):
    // the pixel index addresses the row directly, no division
    row_off = (int64_t)g * p.out_gs + (int64_t)m * p.out_ws;
  } else {
    int n = m / (p.ho * p.wo);
    int rem = m - n * (p.ho * p.wo);
    int ho = rem / p.wo;
    int wo = rem - ho * p.wo;
    row_off = (int64_t)n * p.out_ns + (int64_t)g * p.out_gs + (int64_t)ho * p.out_hs + (int64_t)wo * p.out_ws;
  }
  n_stride = p.out_ks;
  vec_ok = (p.out_ks == 1) && aligned_for_vec(base, row_off, p.epi.out_dtype);
}

// Every output row starts on a 16-byte boundary, rows are n-contiguous and a
// row is a whole number of 16-byte pieces: the staged epilogue may write 16
// bytes per lane.
__device__ __forceinline__ bool out_rows_chunk_aligned(const RockGemmParams &p, const void *base, int es) {
  return p.c_ns == 1 && (((uintptr_t)base | (uintptr_t)(p.c_ms * es) | (uintptr_t)(p.c_gs * es) |
                          (uintptr_t)((int64_t)p.N * es)) & 15) == 0;
}
__device__ __forceinline__ bool out_rows_chunk_aligned(const RockConvParams &p, const void *base, int es) {
  return p.out_ks == 1 &&
         (((uintptr_t)base | (uintptr_t)(p.out_ns * es) | (uintptr_t)(p.out_gs * es) |
           (uintptr_t)(p.out_hs * es) | (uintptr_t)(p.out_ws * es) | (uintptr_t)((int64_t)p.N * es)) & 15) == 0;
}

// The output is contiguous along m (rows of the implicit GEMM), not along n:
// a transposed C, or an NCHW-style convolution output whose pixels are
// contiguous per channel.  16 bytes' worth of consecutive m must start on a
// 16-byte boundary and stay inside one image.
__device__ __forceinline__ bool out_cols_chunk_aligned(const RockGemmParams &p, const void *base, int es) {
  return p.c_ms == 1 && (((uintptr_t)base | (uintptr_t)(p.c_ns * es) | (uintptr_t)(p.c_gs * es) |
                          (uintptr_t)((int64_t)p.M * es)) & 15) == 0;
}
__device__ __forceinline__ bool out_cols_chunk_aligned(const RockConvParams &p, const void *base, int es) {
  return p.out_ws == 1 && p.out_hs == (int64_t)p.wo &&
         (((uintptr_t)base | (uintptr_t)(p.out_ns * es) | (uintptr_t)(p.out_gs * es) | (uintptr_t)(p.out_ks * es) |
           (uintptr_t)((int64_t)p.ho * p.wo * es)) & 15) == 0;
}
// element offset of output (g, m, n = 0) and the stride between channels, for m-contiguous outputs
__device__ __forceinline__ void out_col_addr(const RockGemmParams &p, int g, int m, int64_t &off, int64_t &n_stride) {
  off = (int64_t)g * p.c_gs + m;
  n_stride = p.c_ns;
}
__device__ __forceinline__ void out_col_addr(const RockConvParams &p, int g, int m, int64_t &off, int64_t &n_stride) {
  const int img = m / (p.ho * p.wo);
  off = (int64_t)img * p.out_ns + (int64_t)g * p.out_gs + (m - img * (p.ho * p.wo));
  n_stride = p.out_ks;
}

template <int DT, int ROWS, int NT, int KIND>
__device__ __forceinline__ auto make_loader_a(const void *A, const RockGemmParams &p, int g, int m0, int tid) {
  static_assert(KIND == LD_ROWS_GENERIC, "K-contiguous operands take the direct-to-LDS body");
  RowsGeneric<DT, ROWS, NT> l;
  l.init((const char *)A + (int64_t)g * p.a_gs * MmaTraits<DT>::ES, p.a_ms, p.a_ks, m0, p.M, p.K, tid);
  return l;
}
template <int DT, int ROWS, int NT, int KIND>
__device__ __forceinline__ auto make_loader_b(const void *B, const RockGemmParams &p, int g, int n0, int tid) {
  static_assert(KIND == LD_ROWS_GENERIC, "K-contiguous operands take the direct-to-LDS body");
  RowsGeneric<DT, ROWS, NT> l;
  l.init((const char *)B + (int64_t)g * p.b_gs * MmaTraits<DT>::ES, p.b_ns, p.b_ks, n0, p.N, p.K, tid);
  return l;
}
// convolution: "A" is the input image (implicit rows), "B" the filter
template <int DT, int ROWS, int NT, int KIND>
__device__ __forceinline__ auto make_loader_a(const void *in, const RockConvParams &p, int g, int m0, int tid) {
  static_assert(KIND == LD_CONV_IN_GENERIC, "channel-contiguous input takes the direct-to-LDS body");
  ConvInGeneric<DT, ROWS, NT> l;
  l.init(in, p, g, m0, tid);
  return l;
}
template <int DT, int ROWS, int NT, int KIND>
__device__ __forceinline__ auto make_loader_b(const void *fil, const RockConvParams &p, int g, int n0, int tid) {
  static_assert(KIND == LD_CONV_FIL_GENERIC, "K-contiguous filters take the direct-to-LDS body");
  ConvFilGeneric<DT, ROWS, NT> l;
  l.init(fil, p, g, n0, tid);
  return l;
}

// Epilogue straight from the accumulator layout: the lane owns rows
// m_lane + 32*i and channels n_lane + 32*j + 8*q + {0..3}.
template <bool INT_ACC, int OD, int MI, int NI, typename Acc4, bool SLOW_CALL = true, typename AccArr, typename Params>
__device__ __forceinline__ void direct_epilogue(const AccArr &acc, const Params &p, int g, void *Cptr,
                                                const void *aux, const void *res, int m_lane, int n_lane) {
  constexpr int ES = OutElemSize<OD>::value;
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m_lane + i * 32;
    if (m >= p.M)
      continue;
    int64_t row_off, n_stride;
    bool vec_ok;
    out_row_addr(p, g, m, Cptr, row_off, n_stride, vec_ok);
#pragma unroll
    for (int j = 0; j < NI; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n_lane + j * 32 + q * 8;
        if (n >= p.N)
          continue;
        Acc4 a4 = {acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                   acc[i][j][4 * q + 3]};
        // (the callers that take every epilogue -- SLOW_CALL -- also take the per-channel vectors)
        v4i raw = epilogue_convert4<INT_ACC, OD, SLOW_CALL, SLOW_CALL>(a4, p.epi, aux, n, p.N, p.epi.residual_op ? res : nullptr,
                                                 row_off + (int64_t)n * n_stride, n_stride);
        store_packed4(raw, ES, Cptr, row_off + (int64_t)n * n_stride, n_stride, n, p.N, vec_ok);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The kernel body.  IS_CONV selects the parameter block type.
// ---------------------------------------------------------------------------
template <int DT, int BM, int BN, int WAVES_M, int WAVES_N, int LDA, int LDB, typename Params>
__device__ __forceinline__ void contraction_body(const void *Aptr, const void *Bptr, void *Cptr,
                                                 const void *aux, const void *res, const Params &p) {
  using Tr = MmaTraits<DT>;
  using Acc = typename Tr::Acc;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N; // wave tile
  constexpr int MI = WTM / 32, NI = WTN / 32;
  constexpr int STEPS = kChunksPerRow / (2 * Tr::CHUNKS); // MFMA K steps per 128-byte tile row
  constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32");

  __shared__ __attribute__((aligned(16))) char lds[2 * (A_BYTES + B_BYTES)];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  const int lrow = lane & 31, lgrp = lane >> 5;

  int g, tm, tn;
  decode_block(p.tiles_m, p.tiles_n, p_batch(p), p.group_m, p.xcd_remap, g, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // ---- loaders
  using GA = TileGeom<DT, BM, NT>;
  using GB = TileGeom<DT, BN, NT>;
  auto la = make_loader_a<DT, BM, NT, LDA>(Aptr, p, g, m0, tid);
  auto lb = make_loader_b<DT, BN, NT, LDB>(Bptr, p, g, n0, tid);
  v4i ra[GA::NCH], rb[GB::NCH];

  Acc acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        acc[i][j][v] = 0;

  const int K = p.K;
  const int nk = (K + GA::BKE - 1) / GA::BKE;

  la.load(0, ra);
  lb.load(0, rb);
  store_tile<DT, BM, NT>(lds, ra, tid);
  store_tile<DT, BN, NT>(lds + A_BYTES, rb, tid);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const char *sa = lds + cur * (A_BYTES + B_BYTES);
    const char *sb = sa + A_BYTES;
    const bool more = kt + 1 < nk;
    if (more) {
      la.load(kt + 1, ra);
      lb.load(kt + 1, rb);
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      Frag<DT> fb[NI];
#pragma unroll
      for (int j = 0; j < NI; ++j)
        fb[j] = read_frag<DT>(sb, wn * WTN + j * 32 + lrow, s, lgrp);
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        Frag<DT> fa = read_frag<DT>(sa, wm * WTM + i * 32 + lrow, s, lgrp);
#pragma unroll
        for (int j = 0; j < NI; ++j)
          mma32x32<DT>(fb[j], fa, acc[i][j]);
      }
    }
    if (more) {
      char *da = lds + (cur ^ 1) * (A_BYTES + B_BYTES);
      store_tile<DT, BM, NT>(da, ra, tid);
      store_tile<DT, BN, NT>(da + A_BYTES, rb, tid);
    }
    __syncthreads();
  }

  // ---- epilogue: lane holds m = .. + lrow, n = .. + 8*q + 4*lgrp + {0..3}
  Params pg = p;
  const void *aux_g = aux;
  group_channel_pointers(pg, aux_g, g);
  const RockEpilogue &e = pg.epi;
  using Acc4 = decltype(__builtin_shufflevector(acc[0][0], acc[0][0], 0, 1, 2, 3));
  dispatch_out_dtype<Tr::INT_ACC>(e.out_dtype, [&](auto od_const) __attribute__((always_inline)) {
    constexpr int OD = decltype(od_const)::value;
    direct_epilogue<Tr::INT_ACC, OD, MI, NI, Acc4>(acc, pg, g, Cptr, aux_g, res, m0 + wm * WTM + lrow,
                                                  n0 + wn * WTN + lgrp * 4);
  });
}

} // namespace rk
