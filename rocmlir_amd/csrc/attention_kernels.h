// Fused attention for gfx950: O = softmax(scale * Q K^T + bias) V, one pass,
// scores never leave the compute unit.
//
// Behaviour replaced: rock.attention lowered by
// mlir/lib/Dialect/Rock/Transforms/GridwiseGemmToBlockwise.cpp:1607-2403
// (online softmax over seq_k blocks, exp2 with the log2(e) factor folded into
// the scale, -inf for padded keys, final division by the row sum).  The
// reference reduces rows through LDS and runs the softmax in the element type;
// this kernel is organised so that no cross-lane reduction beyond one
// half-wave swap is needed and the statistics stay in f32:
//
//   * a wave owns 32 query rows; S^T = K_tile * Q^T is computed with the
//     32x32x16 MFMA, whose result layout gives every lane ONE query column and
//     16 of the 32 keys of the tile (the other 16 sit in lane ^ 32);
//   * row max / row sum are therefore per-lane loops plus one exchange with
//     lane ^ 32; the running max, sum and the rescale factor are
//     per-lane scalars that apply directly to the O^T accumulators, which use
//     the same "lane = query column" layout (O^T = V^T * P^T);
//   * P^T is packed to 16-bit floats in registers and used as the MFMA column
//     operand as is: the key order inside a K-slice is a fixed permutation,
//     and V^T is stored to LDS with the same permutation applied;
//   * K is staged row-major (row pitch padded by 16 bytes), V is transposed
//     while it is written to LDS (pitch 144 bytes) so that both MFMA row
//     operands are single conflict-free 16-byte reads;
//   * next K/V tiles are fetched into registers while the current ones are
//     being multiplied; two LDS stages, one barrier per tile.
#pragma once
#include <type_traits>
#include "mfma_gfx950.h"

namespace rk {

constexpr int kBQ = 128;  // query rows per block (4 waves x 32)
constexpr int kBKV = 64;  // keys per tile
constexpr int kAttnThreads = 256;
constexpr int kVPitch = kBKV * 2 + 16; // bytes per V^T row in LDS

// value of x held by lane ^ 32.  (v_permlane32_swap would do, but the
// compiler folds its two tied operands into one register when both are the
// same value, which turns the swap into a copy; the LDS crossbar permute has
// no such trap and costs two instructions per K/V tile.)
__device__ __forceinline__ float other_half(float x) {
  const int lane = (int)(threadIdx.x & 63);
  int v = __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, x));
  return __builtin_bit_cast(float, v);
}
// Both halves of the wave through one v_permlane32_swap: with a = b = x in two
// different registers the instruction leaves a = [x.lo, x.lo] and
// b = [x.hi, x.hi].  Written as assembly: the compiler builtin folds the two
// equal operands into one register and then drops the combine that follows.
// The s_nop pair covers the wait states the instruction needs after a VALU
// write of its operands and before a VALU read of its results, which the
// compiler's hazard pass cannot see inside an asm block.
__device__ __forceinline__ void both_halves(float x, float &lo, float &hi) {
#ifdef __AMDGCN__
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  lo = a;
  hi = b;
#else // (the CPU build of the kernels that the tests run: the same two values through the cross-lane read)
  const int lane = (int)(threadIdx.x & 63);
  lo = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane & 31) << 2, __builtin_bit_cast(int, x)));
  hi = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane | 32) << 2, __builtin_bit_cast(int, x)));
#endif
}
__device__ __forceinline__ float half_swap_max_fast(float x) {
  float lo, hi;
  both_halves(x, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float half_swap_max(float x) { return fmaxf(x, other_half(x)); }
__device__ __forceinline__ float half_swap_sum(float x) { return x + other_half(x); }

template <int DT>
__device__ __forceinline__ v16f mma32(const v4i &rows, const v4i &cols, const v16f &acc) {
  if constexpr (DT == MM_F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, rows),
                                                  __builtin_bit_cast(v8h, cols), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, rows),
                                                   __builtin_bit_cast(v8bf, cols), acc, 0, 0, 0);
}

template <int DT> __device__ __forceinline__ uint32_t pack2(float a, float b) {
  if constexpr (DT == MM_F16) {
    _Float16 ha = (_Float16)a, hb = (_Float16)b;
    return (uint32_t)__builtin_bit_cast(uint16_t, ha) | ((uint32_t)__builtin_bit_cast(uint16_t, hb) << 16);
  } else {
    __bf16 ha = (__bf16)a, hb = (__bf16)b;
    return (uint32_t)__builtin_bit_cast(uint16_t, ha) | ((uint32_t)__builtin_bit_cast(uint16_t, hb) << 16);
  }
}

template <int DT> __device__ __forceinline__ float elem_to_f32(uint16_t raw) {
  if constexpr (DT == MM_F16)
    return (float)__builtin_bit_cast(_Float16, raw);
  else
    return __builtin_bit_cast(float, (uint32_t)raw << 16);
}

// 8 consecutive 16-bit elements starting at (row, col0) of a strided matrix;
// zero outside [0,rows) x [0,cols).  FAST: unit column stride, col0 % 8 == 0,
// cols % 8 == 0 and 16-byte aligned rows.
template <bool FAST>
__device__ __forceinline__ v4i load8(const uint16_t *base, int64_t rs, int64_t cs, int row, int col0,
                                     int rows, int cols) {
  v4i out = {0, 0, 0, 0};
  if (row >= rows || col0 >= cols)
    return out;
  if constexpr (FAST) {
    out = *(const v4i *)(base + (int64_t)row * rs + col0);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      uint32_t v = (col0 + e < cols) ? base[(int64_t)row * rs + (int64_t)(col0 + e) * cs] : 0u;
      out[e >> 1] |= (int)(v << (16 * (e & 1)));
    }
  }
  return out;
}

template <int DT, int DQK, int DV, bool FAST>
__device__ __forceinline__ void attention_body(const void *Qv, const void *Kv, const void *Vv,
                                               const void *scalev, const void *biasv, const void *maskv,
                                               const void *otherv, void *Ov, const RockAttentionParams &p) {
  constexpr int KCH = DQK / 8;              // 16-byte chunks per K row
  constexpr int KPITCH = DQK * 2 + 16;      // bytes
  constexpr int K_BYTES = kBKV * KPITCH;
  constexpr int V_BYTES = DV * kVPitch;
  constexpr int STAGE = K_BYTES + V_BYTES;
  constexpr int KSTEPS = DQK / 16;          // MFMA K steps of the first GEMM
  constexpr int DTILES = DV / 32;           // 32-row tiles of O^T
  constexpr int K_NCH = (kBKV * KCH) / kAttnThreads;   // K chunks per thread
  constexpr int V_UNITS = 16 * (DV / 8);    // (key quad, dv chunk) units per tile
  constexpr int V_NU = (V_UNITS + kAttnThreads - 1) / kAttnThreads;
  static_assert((kBKV * KCH) % kAttnThreads == 0, "K tile must divide over the block");

  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lq = lane & 31, h = lane >> 5;

  // block -> (g, query block), undoing the round-robin block->XCD dispatch so
  // that the query blocks of one g (which share K and V) run on one XCD
  int bid = blockIdx.x;
  {
    const int total = p.G * p.q_blocks;
    const int per = total >> 3;
    if (p.xcd_remap && bid < (per << 3))
      bid = (bid & 7) * per + (bid >> 3);
  }
  const int g = bid / p.q_blocks;
  const int qb = bid - g * p.q_blocks;
  const int q_row = qb * kBQ + wave * 32 + lq; // this lane's query row

  const uint16_t *Q = (const uint16_t *)Qv + (int64_t)g * p.q_gs;
  const uint16_t *K = (const uint16_t *)Kv + (int64_t)g * p.k_gs;
  const uint16_t *V = (const uint16_t *)Vv + (int64_t)g * p.v_gs;
  uint16_t *O = (uint16_t *)Ov + (int64_t)g * p.o_gs;
  const uint16_t *bias = p.has_bias ? (const uint16_t *)biasv + (int64_t)g * p.bias_gs : nullptr;
  const uint16_t *scale_t = p.has_scale_tensor ? (const uint16_t *)scalev + (int64_t)g * p.bias_gs : nullptr;
  const int8_t *mask = p.has_mask ? (const int8_t *)maskv + (int64_t)g * p.bias_gs : nullptr;
  const uint16_t *other = p.has_mask ? (const uint16_t *)otherv + (int64_t)g * p.bias_gs : nullptr;

  // ---- Q^T fragments: column operand, lane = query row, 8 d per K step
  v4i qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks)
    qf[ks] = load8<FAST>(Q, p.q_is, p.q_ds, q_row, ks * 16 + h * 8, p.seq_q, p.d_qk);

  v16f o[DTILES];
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      o[dt][v] = 0.0f;
  float m_run = -INFINITY; // running max of scaled scores (log2 domain)
  float l_run = 0.0f;      // this lane's share of the running row sum

  const float c_scale = p.scale * 1.44269504088896340736f;
  const int nkv = (p.seq_k + kBKV - 1) / kBKV;

  v4i kreg[K_NCH];
  v4i vreg[V_NU][4];

  auto fetch = [&](int t) {
    const int key0 = t * kBKV;
#pragma unroll
    for (int i = 0; i < K_NCH; ++i) {
      int id = tid + i * kAttnThreads;
      int row = id / KCH, c = id - row * KCH;
      kreg[i] = load8<FAST>(K, p.k_js, p.k_ds, key0 + row, c * 8, p.seq_k, p.d_qk);
    }
#pragma unroll
    for (int i = 0; i < V_NU; ++i) {
      int u = tid + i * kAttnThreads;
      int kq = u & 15, dvc = u >> 4;
#pragma unroll
      for (int b = 0; b < 4; ++b)
        vreg[i][b] = (u < V_UNITS)
                         ? load8<FAST>(V, p.v_js, p.v_es, key0 + kq * 4 + b, dvc * 8, p.seq_k, p.d_v)
                         : v4i{0, 0, 0, 0};
    }
  };
  auto stash = [&](int stage) {
    char *sk = lds + stage * STAGE;
    char *sv = sk + K_BYTES;
#pragma unroll
    for (int i = 0; i < K_NCH; ++i) {
      int id = tid + i * kAttnThreads;
      int row = id / KCH, c = id - row * KCH;
      *(v4i *)(sk + row * KPITCH + c * 16) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < V_NU; ++i) {
      int u = tid + i * kAttnThreads;
      if (u < V_UNITS) {
        int kq = u & 15, dvc = u >> 4;
        // position of key 4*kq inside the tile after the in-slice permutation
        int pos0 = 16 * (kq >> 2) + 8 * (kq & 1) + 4 * ((kq & 3) >> 1);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          // element e of each of the 4 key rows -> 4 consecutive positions of V^T row dv
          uint32_t w[4];
#pragma unroll
          for (int b = 0; b < 4; ++b)
            w[b] = ((uint32_t)vreg[i][b][e >> 1] >> (16 * (e & 1))) & 0xffffu;
          v2i pk = {(int)(w[0] | (w[1] << 16)), (int)(w[2] | (w[3] << 16))};
          *(v2i *)(sv + (dvc * 8 + e) * kVPitch + pos0 * 2) = pk;
        }
      }
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();

  for (int t = 0; t < nkv; ++t) {
    const int cur = t & 1;
    const char *sk = lds + cur * STAGE;
    const char *sv = sk + K_BYTES;
    const bool more = t + 1 < nkv;
    if (more)
      fetch(t + 1);

    // ---- S^T tiles: rows = keys, cols = queries
    v16f s[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
      for (int v = 0; v < 16; ++v)
        s[st][v] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        v4i kf = *(const v4i *)(sk + (st * 32 + lq) * KPITCH + (ks * 2 + h) * 16);
        s[st] = mma32<DT>(kf, qf[ks], s[st]);
      }
    }

    // ---- online softmax on this lane's 32 scores of row q_row
    const int key_base = t * kBKV + 4 * h;
    float mloc = -INFINITY;
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int key = key_base + st * 32 + 8 * (v >> 2) + (v & 3);
        float x = s[st][v];
        // op order of the reference: * scale tensor, * scale, + bias (rocmlir-gen.cpp:2565-2590)
        if (scale_t != nullptr && key < p.seq_k && q_row < p.seq_q)
          x = x * elem_to_f32<DT>(scale_t[(int64_t)q_row * p.bias_is + (int64_t)key * p.bias_js]);
        x = x * c_scale;
        if (bias != nullptr && key < p.seq_k && q_row < p.seq_q)
          x = x + elem_to_f32<DT>(bias[(int64_t)q_row * p.bias_is + (int64_t)key * p.bias_js]) *
                      1.44269504088896340736f;
        // where(mask, x, other): a select behind the element-wise chain (mixr-attn-where.mlir:11)
        if (mask != nullptr && key < p.seq_k && q_row < p.seq_q &&
            mask[(int64_t)q_row * p.bias_is + (int64_t)key * p.bias_js] == 0)
          x = elem_to_f32<DT>(other[(int64_t)q_row * p.bias_is + (int64_t)key * p.bias_js]) * 1.44269504088896340736f;
        x = key < p.seq_k ? x : -INFINITY;
        s[st][v] = x;
        mloc = fmaxf(mloc, x);
      }
    const float mt = half_swap_max(mloc);
    const float m_new = fmaxf(m_run, mt);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    m_run = m_new;
    float psum = 0.0f;
    uint32_t pp[2][8]; // packed P^T: two 16-bit values per register
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int v = 0; v < 16; v += 2) {
        float p0 = __builtin_amdgcn_exp2f(s[st][v] - m_use);
        float p1 = __builtin_amdgcn_exp2f(s[st][v + 1] - m_use);
        psum += p0 + p1;
        pp[st][v >> 1] = pack2<DT>(p0, p1);
      }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        o[dt][v] *= alpha;

    // ---- O^T += V^T * P^T ; K step (st,u) covers keys 32*st + 16*u + [0,16)
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        v4i pf = {(int)pp[st][4 * u + 0], (int)pp[st][4 * u + 1], (int)pp[st][4 * u + 2],
                  (int)pp[st][4 * u + 3]};
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) {
          v4i vf = *(const v4i *)(sv + (dt * 32 + lq) * kVPitch + (st * 32 + u * 16 + h * 8) * 2);
          o[dt] = mma32<DT>(vf, pf, o[dt]);
        }
      }

    if (more)
      stash(cur ^ 1);
    __syncthreads();
  }

  // ---- normalise and store: lane holds O[q_row][32*dt + 8*(v/4) + 4*h + v%4]
  const float l_tot = half_swap_sum(l_run);
  const float inv = 1.0f / l_tot;
  if (q_row < p.seq_q) {
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const int e0 = dt * 32 + 8 * vq + 4 * h;
        if (e0 >= p.d_v)
          continue;
        float r0 = o[dt][4 * vq + 0] * inv, r1 = o[dt][4 * vq + 1] * inv;
        float r2 = o[dt][4 * vq + 2] * inv, r3 = o[dt][4 * vq + 3] * inv;
        uint16_t *dst = O + (int64_t)q_row * p.o_is + (int64_t)e0 * p.o_es;
        if (FAST) {
          v2i pk = {(int)pack2<DT>(r0, r1), (int)pack2<DT>(r2, r3)};
          *(v2i *)dst = pk;
        } else {
          float r[4] = {r0, r1, r2, r3};
#pragma unroll
          for (int b = 0; b < 4; ++b)
            if (e0 + b < p.d_v)
              dst[(int64_t)b * p.o_es] = (uint16_t)(pack2<DT>(r[b], 0.0f) & 0xffffu);
        }
      }
  }
}

__device__ __forceinline__ void wait_vmcnt_attn0() {
  __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0); expcnt and lgkmcnt left alone
}
// Before the barrier that hands an LDS tile back to the loaders: this wave's
// loads have landed AND its LDS reads have returned.  Without the second part
// a read issued just before the barrier can still sit in the LDS queue when
// another wave's refill of that tile lands.
__device__ __forceinline__ void wait_loads_and_lds_reads() {
  __builtin_amdgcn_s_waitcnt(0x0070); // vmcnt(0) lgkmcnt(0); expcnt left alone
}

} // namespace rk

#include "attention_dlds.h"

// pointer order follows the reference: Q, K, V, the pre-softmax inputs (scale tensor, bias, where-mask and its
// "other" tensor; NULL when the problem has none), O
#define RK_ATTN(DTNAME, DT, DQK, DV, FASTNAME, FAST)                                          \
  extern "C" __global__ __launch_bounds__(rk::kAttnThreads) void                              \
      rock_attention_##DTNAME##_d##DQK##x##DV##_##FASTNAME(const void *Q, const void *K,      \
                                                           const void *V, const void *scale,  \
                                                           const void *bias, const void *mask, const void *other, void *O, \
                                                           RockAttentionParams p) {           \
    rk::attention_body<DT, DQK, DV, FAST>(Q, K, V, scale, bias, mask, other, O, p);           \
  }

// fast variants: two blocks per compute unit (register budget 256 per lane).
// The build (rocmlir_amd/_build.py holds the list) compiles every kernel into a
// code object of its own from a small source that includes this file and
// invokes one of the two macros.
// Head dimensions above 128: one block per compute unit (its K and V slots
// fill 128 KiB of LDS and its O accumulators half a wave's registers), simple
// order "scores, softmax, PV" per tile, with or without the pre-softmax tensors.
#define RK_ATTN_DL_WIDE(DTNAME, DT, D)                                                        \
  extern "C" __global__ __launch_bounds__(rk::kAttnThreads, 1) void                           \
      rock_attention_##DTNAME##_d##D##x##D##_fast_bias(const void *Q, const void *K,          \
                                                       const void *V, const void *scale,      \
                                                       const void *bias, const void *mask, const void *other, void *O, \
                                                       RockAttentionParams p) {               \
    rk::attention_body_dl<DT, D, false>(Q, K, V, scale, bias, mask, other, O, p);             \
  }
// int8 Q and K, f16 V / bias / O
#define RK_ATTN_DL_I8(D, SUFFIX, PLAIN)                                                       \
  extern "C" __global__ __launch_bounds__(rk::kAttnThreads, 2) void                           \
      rock_attention_i8_d##D##x##D##_##SUFFIX(const void *Q, const void *K, const void *V,    \
                                              const void *scale, const void *bias, const void *mask, const void *other, void *O, \
                                              RockAttentionParams p) {                        \
    rk::attention_body_dl<MM_F16, D, PLAIN, true>(Q, K, V, scale, bias, mask, other, O, p);   \
  }
// K stored [d][seq_k] (the reference's default layout)
#define RK_ATTN_DL_KT(DTNAME, DT, D, SUFFIX, PLAIN, OCC)                                      \
  extern "C" __global__ __launch_bounds__(rk::kAttnThreads, OCC) void                         \
      rock_attention_##DTNAME##_d##D##x##D##_##SUFFIX(const void *Q, const void *K,           \
                                                      const void *V, const void *scale,       \
                                                      const void *bias, const void *mask, const void *other, void *O, \
                                                      RockAttentionParams p) {                \
    rk::attention_body_dl<DT, D, PLAIN, false, true>(Q, K, V, scale, bias, mask, other, O, p); \
  }
#define RK_ATTN_DL(DTNAME, DT, D, SUFFIX, PLAIN)                                              \
  extern "C" __global__ __launch_bounds__(rk::kAttnThreads, 2) void                           \
      rock_attention_##DTNAME##_d##D##x##D##_##SUFFIX(const void *Q, const void *K,           \
                                                      const void *V, const void *scale,       \
                                                      const void *bias, const void *mask, const void *other, void *O, \
                                                      RockAttentionParams p) {                \
    rk::attention_body_dl<DT, D, PLAIN>(Q, K, V, scale, bias, mask, other, O, p);             \
  }
