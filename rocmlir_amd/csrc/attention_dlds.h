// Fast path of the fused attention kernel (unit-stride head dimension, head
// dims multiples of 8): K and V tiles stream global -> LDS without passing
// through registers, V is transposed by the LDS read itself, and two blocks
// share a compute unit so that one wave's softmax overlaps another's MFMAs.
//
// Included by attention_kernels.hip after the helpers it uses.  Algorithm and
// accumulator layouts are the ones described at the top of that file; what
// changes relative to the register-staged body there:
//
//   * K and V tiles (64 keys x D) are stored row-major with the 16-byte chunk
//     index XOR-ed with a function of the key row, filled by
//     buffer_load ... lds (hardware zero fill for keys past seq_k and for
//     head-dim padding);
//   * the V^T row operand of the second GEMM comes from ds_read_b64_tr_b16:
//     within a group of 16 lanes, lane i addresses 4 consecutive d of key
//     k0 + i/4 and receives the 4 keys k0..k0+3 at d = d0 + i.  Two such reads
//     give the 8 keys {4h..4h+3, 8+4h..8+4h+3} of a 16-key slice -- exactly
//     the keys whose probabilities the lane holds from the first GEMM;
//   * every LDS read address is "per-lane offset computed once + immediate":
//     the swizzles only depend on the low bits of the key row, which the
//     tile / slice / stage offsets (multiples of 8 rows) do not touch, and the
//     loop is unrolled over the two stages;
//   * the running-max rescale of O is skipped while no lane's maximum moved
//     (alpha == 1 exactly, so the result is unchanged);
//   * without bias and with a non-negative scale the row maximum is taken on
//     the raw scores and the scale is folded into exp2(fma(s, c, -m)).
#pragma once

namespace rk {

constexpr unsigned kAttnOob = 0x80000000u;
typedef __attribute__((address_space(3))) void attn_lds_void_t;
typedef __attribute__((address_space(3))) char attn_lds_char_t;
typedef __attribute__((address_space(3))) v4s attn_lds_v4s_t;
typedef __attribute__((address_space(3))) v4i attn_lds_v4i_t;

template <int D> struct AttnTileGeom {
  static constexpr int CPR = D / 8;         // 16-byte chunks per row
  static constexpr int ROWB = D * 2;        // bytes per row
  static constexpr int TILE_B = kBKV * ROWB;
  static constexpr int SLABS = TILE_B / 1024;
  static constexpr int PER_WAVE = SLABS / 4;
  static_assert(SLABS % 4 == 0, "tile must split over 4 waves");
};

// Chunk swizzles (XOR-ed into the 16-byte chunk index of a row).  K rows are
// read 32 rows at one chunk index.  V rows are read by the transposing load:
// 32 lanes cover 4 consecutive rows x 4 adjacent chunks (chunk bits 0-1 come
// from the lane), so the row index is XOR-ed into the chunk bits above them.
// Each function spreads its access pattern over distinct bank groups for the
// row pitch at hand (256 bytes = one full bank period for D = 128, half a
// period for D = 64, a quarter for int8 keys at D = 64), and depends only on
// the row modulo 16 (K) or 8 (V).
template <int CPR, bool IS_V> __device__ __forceinline__ int attn_swz(int row) {
  if constexpr (!IS_V) // 256 / 128 / 64 bytes per row (the last: int8 keys of a head dimension up to 64)
    return CPR == 16 ? (row & 15) : CPR == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3);
  else
    return CPR == 16 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2);
}

// One K or V tile loader: row-major [key][d] source with unit d stride.
template <int D, bool IS_V> struct AttnTileLoader {
  using Gm = AttnTileGeom<D>;
  const char *base;
  unsigned off[Gm::PER_WAVE]; // byte offset inside a tile, or kAttnOob for head-dim padding
  int row0;                   // tile row of this lane's first chunk; chunk i is ROWS_PER_SLAB*i further
  int pitch_b, rows_total, wave;
  static constexpr int ROWS_PER_SLAB = 64 / Gm::CPR;

  __device__ __forceinline__ void init(const uint16_t *base_, int64_t row_stride, int rows, int d,
                                       int wave_, int lane) {
    wave = wave_;
    rows_total = rows;
    pitch_b = (int)row_stride * 2;
    base = (const char *)base_;
#pragma unroll
    for (int i = 0; i < Gm::PER_WAVE; ++i) {
      int c = (wave * Gm::PER_WAVE + i) * 64 + lane; // physical chunk inside the tile
      int r = c / Gm::CPR, pc = c - r * Gm::CPR;
      int lc = pc ^ attn_swz<Gm::CPR, IS_V>(r);
      if (i == 0)
        row0 = r;
      off[i] = (lc * 8 < d) ? (unsigned)(r * pitch_b + lc * 16) : kAttnOob;
    }
  }
  // The descriptor is rebuilt per tile with its base at key0 (scalar work), so
  // the per-lane offsets never change; only the last tile needs the row test.
  __device__ __forceinline__ void issue(int key0, attn_lds_char_t *tile) {
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(base + (int64_t)key0 * pitch_b), 0, (int)kAttnOob, 0x00020000);
    const int left = rows_total - key0; // rows of this tile that exist (may be <= 0)
#pragma unroll
    for (int i = 0; i < Gm::PER_WAVE; ++i) {
      unsigned voff = (row0 + i * ROWS_PER_SLAB < left) ? off[i] : kAttnOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc, (attn_lds_void_t *)(tile + (wave * Gm::PER_WAVE + i) * 1024), 16, (int)voff, 0, 0, 0);
    }
  }
};

// K stored [d][seq_k] (the reference's default, rocmlir-gen.cpp:2164-2165): a
// tile holds D rows of d, each the 64 keys of the tile (128 bytes, 8 chunks),
// in the geometry of a V tile of head dimension 64 with D rows; the S^T row
// operand then comes out of it through the transposing read, exactly as V^T
// does out of a V tile (rows = the reduction index, columns = the MFMA row index).
template <int D> struct AttnKtLoader {
  static constexpr int CPR = 8;                 // 16-byte chunks per row of 64 keys
  static constexpr int ROWB = 128;
  static constexpr int TILE_B = D * ROWB;
  static constexpr int SLABS = TILE_B / 1024;
  static constexpr int PER_WAVE = SLABS / 4;
  static_assert(SLABS % 4 == 0, "tile must split over 4 waves");
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned off[PER_WAVE]; // byte offset of the chunk at key tile 0, or kAttnOob for rows of d beyond the head dimension
  int key_of_chunk;       // first key (inside a tile) of this lane's chunks: the same for all of them
  int seq_k, wave;

  __device__ __forceinline__ void init(const uint16_t *base, int64_t d_stride, int seq_k_, int d, int wave_, int lane) {
    wave = wave_;
    seq_k = seq_k_;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(base), 0, (int)kAttnOob, 0x00020000);
    const int pitch_b = (int)d_stride * 2;
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
      const int c = (wave * PER_WAVE + i) * 64 + lane; // physical chunk inside the tile
      const int r = c / CPR, pc = c - r * CPR;
      const int lc = pc ^ attn_swz<CPR, true>(r);
      // (64 lanes = 8 rows of 8 chunks, and the swizzle only flips chunk bit 2 by row bit 1: the chunk a lane fills
      // differs from slab to slab by that bit only when the slab's first row does, which it does not: slabs start
      // at multiples of 8 rows)
      if (i == 0)
        key_of_chunk = lc * 8;
      off[i] = r < d ? (unsigned)(r * pitch_b + lc * 16) : kAttnOob;
    }
  }
  // keys [key0, key0 + 64); chunks that start at or beyond seq_k read as zeros
  __device__ __forceinline__ void issue(int key0, attn_lds_char_t *tile) {
    const bool in_range = key0 + key_of_chunk < seq_k;
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
      const unsigned voff = in_range ? off[i] : kAttnOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc, (attn_lds_void_t *)(tile + (wave * PER_WAVE + i) * 1024), 16, (int)voff, key0 * 2, 0, 0);
    }
  }
};

template <int DT> __device__ __forceinline__ uint32_t pack2_fast(float a, float b) {
  if constexpr (DT == MM_F16) {
    typedef float v2f_t __attribute__((ext_vector_type(2)));
    typedef _Float16 v2h_t __attribute__((ext_vector_type(2)));
    v2f_t f = {a, b};
    v2h_t hv = __builtin_convertvector(f, v2h_t); // round to nearest even
    return __builtin_bit_cast(uint32_t, hv);
  } else {
    typedef float v2f_t __attribute__((ext_vector_type(2)));
    typedef __bf16 v2b_t __attribute__((ext_vector_type(2)));
    v2f_t f = {a, b};
    v2b_t hv = __builtin_convertvector(f, v2b_t);
    return __builtin_bit_cast(uint32_t, hv);
  }
}

// PLAIN: no bias and a non-negative scale, so the row maximum can be taken on
// the raw scores and the scale folded into the exponent.
// QKI8: Q and K are int8 and the first GEMM runs on the int8 MFMA; its int32
// sums are dequantised on the score tile in registers, (acc - zero_point) *
// scale, before anything else touches them (the quantised first GEMM of
// mlir/test/fusion/pr-e2e/attention/mixr-attention-first-gemm-i8-f16.mlir).
// V, the pre-softmax tensors and O stay DT.  D counts elements, so a K row is
// D bytes and the K tile has the geometry of a 16-bit tile of D / 2.
// KT: K is stored [d][seq_k] instead of [seq_k][d] (16-bit types).
template <int DT, int D, bool PLAIN, bool QKI8 = false, bool KT = false>
__device__ __forceinline__ void attention_body_dl(const void *Qv, const void *Kv, const void *Vv,
                                                  const void *scalev, const void *biasv, const void *maskv,
                                                  const void *otherv, void *Ov, const RockAttentionParams &p) {
  using Gm = AttnTileGeom<D>;                  // V tile
  using GmK = AttnTileGeom<QKI8 ? D / 2 : D>;  // K tile (KT: the same bytes as D rows of 64 keys)
  static_assert(!(KT && QKI8), "int8 keys stored [d][seq_k] are not built");
  constexpr int KSTEPS = QKI8 ? D / 32 : D / 16; // MFMA K steps of the first GEMM
  constexpr int DTILES = D / 32;  // 32-row tiles of O^T
  constexpr float kLog2e = 1.44269504088896340736f;
  // The plain kernel software-pipelines the two GEMMs (see tile_step); the
  // bias kernel needs its registers for the bias gather and keeps the simple
  // order "scores, softmax, PV" per tile.
  constexpr bool PIPE = PLAIN;
  static_assert(D > 128 || 4 * Gm::TILE_B <= 65536, "up to D = 128 every LDS read offset fits the 16-bit immediate");

  // Every slot is an object of its own: the compiler makes an LDS read wait for
  // the loads into LDS still in flight unless it can tell that the two touch
  // different objects, and each phase of a tile reads one slot while the next
  // tiles stream into the others.
  __shared__ __attribute__((aligned(1024))) char lds_k0_generic[GmK::TILE_B];
  __shared__ __attribute__((aligned(1024))) char lds_k1_generic[GmK::TILE_B];
  __shared__ __attribute__((aligned(1024))) char lds_v0_generic[Gm::TILE_B];
  __shared__ __attribute__((aligned(1024))) char lds_v1_generic[Gm::TILE_B];
  attn_lds_char_t *const lds_k0 = (attn_lds_char_t *)lds_k0_generic;
  attn_lds_char_t *const lds_k1 = (attn_lds_char_t *)lds_k1_generic;
  attn_lds_char_t *const lds_v0 = (attn_lds_char_t *)lds_v0_generic;
  attn_lds_char_t *const lds_v1 = (attn_lds_char_t *)lds_v1_generic;
  auto k_slot = [&](int slot) __attribute__((always_inline)) { return slot ? lds_k1 : lds_k0; };
  auto v_slot = [&](int slot) __attribute__((always_inline)) { return slot ? lds_v1 : lds_v0; };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, h = lane >> 5;

  int bid = blockIdx.x;
  {
    const int total = p.G * p.q_blocks;
    const int per = total >> 3;
    if (p.xcd_remap && bid < (per << 3))
      bid = (bid & 7) * per + (bid >> 3);
  }
  const int g = bid / p.q_blocks;
  const int qb = bid - g * p.q_blocks;
  const int q_row = qb * kBQ + wave * 32 + lq;

  const uint16_t *Q = (const uint16_t *)Qv + (int64_t)g * p.q_gs;
  const uint16_t *K = (const uint16_t *)Kv + (int64_t)g * p.k_gs;
  const uint16_t *V = (const uint16_t *)Vv + (int64_t)g * p.v_gs;
  uint16_t *O = (uint16_t *)Ov + (int64_t)g * p.o_gs;
  const uint16_t *bias = p.has_bias ? (const uint16_t *)biasv + (int64_t)g * p.bias_gs : nullptr;
  const uint16_t *scale_t = p.has_scale_tensor ? (const uint16_t *)scalev + (int64_t)g * p.bias_gs : nullptr;
  const int8_t *mask = p.has_mask ? (const int8_t *)maskv + (int64_t)g * p.bias_gs : nullptr;
  const uint16_t *other = p.has_mask ? (const uint16_t *)otherv + (int64_t)g * p.bias_gs : nullptr;

  std::conditional_t<KT, AttnKtLoader<D>, AttnTileLoader<QKI8 ? D / 2 : D, false>> lk;
  AttnTileLoader<D, true> lv;
  if constexpr (KT)
    lk.init(K, p.k_ds, p.seq_k, p.d_qk, wave, lane);
  else if constexpr (QKI8) // int8 rows seen as 16-bit rows of half the length (strides are even: host check)
    lk.init((const uint16_t *)((const char *)Kv + (int64_t)g * p.k_gs), p.k_js / 2, p.seq_k, p.d_qk / 2, wave, lane);
  else
    lk.init(K, p.k_js, p.seq_k, p.d_qk, wave, lane);
  lv.init(V, p.v_js, p.seq_k, p.d_v, wave, lane);
  lk.issue(0, k_slot(0));
  lv.issue(0, v_slot(0));
  if constexpr (PIPE)
    lk.issue(kBKV, k_slot(1));

  v4i qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    if constexpr (QKI8) {
      const int col = ks * 32 + h * 16; // 16 int8 values of this lane's query row
      const char *q8 = (const char *)Qv + (int64_t)g * p.q_gs + (int64_t)q_row * p.q_is + col;
      qf[ks] = (q_row < p.seq_q && col < p.d_qk) ? *(const v4i *)q8 : v4i{0, 0, 0, 0};
    } else {
      qf[ks] = load8<true>(Q, p.q_is, p.q_ds, q_row, ks * 16 + h * 8, p.seq_q, p.d_qk);
    }
  }

  // ---- per-lane LDS read offsets (bytes from the start of a K or V tile)
  // K fragment of key rows 32*st + lq at chunk 2*ks + h: the swizzle depends on
  // lq only, so "+ 32*st rows" and the stage are immediates.
  const int krow = lq * GmK::ROWB; // byte offset inside a K tile
  const int kswz = (h ^ attn_swz<GmK::CPR, false>(lq)) * 16; // chunk 2*ks + h: ks XORs in as a constant
  auto koff = [&](int ks) __attribute__((always_inline)) { return krow + (kswz ^ (ks * 32)); };
  // V^T fragment through the transposing read: lane (i = lane % 16, g16) of
  // half h addresses key 4*h + i/4 (+ 32*st + 16*u, + 8) at d = 32*dt + 16*g16 + 4*(i%4).
  const int tr_i = lane & 15, tr_g = (lane >> 4) & 1;
  const int tr_key = 4 * h + (tr_i >> 2);
  const int tr_chunk = 2 * tr_g + ((tr_i & 3) >> 1);
  const int vrow = tr_key * Gm::ROWB + (tr_i & 1) * 8; // byte offset inside a V tile
  const int vswz = (tr_chunk ^ attn_swz<Gm::CPR, true>(tr_key)) * 16; // chunk 4*dt + tr_chunk
  auto voff = [&](int dt) __attribute__((always_inline)) { return vrow + (vswz ^ (dt * 64)); };
  // KT: S^T row operand through the same read.  Lane (i, g16) of half h addresses row d = 16*ks + 8*h + i/4
  // (+ 4 for the second read) at keys 32*st + 16*g16 + 4*(i%4), and receives key 32*st + lq for four
  // consecutive d: two reads give the 8 consecutive d that the lane's Q fragment holds.
  const int ktrow = (8 * h + (tr_i >> 2)) * 128 + (tr_i & 1) * 8;
  const int ktswz = (tr_chunk ^ attn_swz<8, true>(tr_i >> 2)) * 16; // chunk 4*st + tr_chunk; row bit 1 comes from i/4
  auto ktoff = [&](int ks, int st) __attribute__((always_inline)) { return ktrow + ks * 16 * 128 + (ktswz ^ (st * 64)); };

  v16f o[DTILES];
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      o[dt][v] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const float c_scale = p.scale * kLog2e;
  constexpr bool plain = PLAIN;
  const int nkv = (p.seq_k + kBKV - 1) / kBKV;

  // S^T tiles of the K tile in LDS slot SLOT: rows = keys, cols = queries
  auto scores = [&](auto slot_const, v16f(&s)[2]) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_const)::value;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      if constexpr (QKI8) {
        v16i acc;
#pragma unroll
        for (int v = 0; v < 16; ++v)
          acc[v] = 0;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          v4i kf = *(const attn_lds_v4i_t *)(k_slot(SLOT) + koff(ks) + st * 32 * GmK::ROWB);
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[ks], acc, 0, 0, 0);
        }
        s[st] = __builtin_bit_cast(v16f, acc); // dequantised where the tile's softmax starts
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v)
          s[st][v] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          v4i kf;
          if constexpr (KT) {
            attn_lds_char_t *a0 = k_slot(SLOT) + ktoff(ks, st);
            v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_v4s_t *)a0);
            v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_v4s_t *)(a0 + 4 * 128));
            v2i l2 = __builtin_bit_cast(v2i, lo), h2 = __builtin_bit_cast(v2i, hi);
            kf = v4i{l2[0], l2[1], h2[0], h2[1]};
          } else {
            kf = *(const attn_lds_v4i_t *)(k_slot(SLOT) + koff(ks) + st * 32 * GmK::ROWB);
          }
          s[st] = mma32<DT>(kf, qf[ks], s[st]);
        }
      }
    }
  };

  // One step of the software pipeline.  On entry `s` holds the scores of tile
  // t (their MFMAs possibly still in flight), K[t+1] and V[t] have been
  // requested.  The step requests K[t+2] and V[t+1], issues the score MFMAs of
  // tile t+1 into `s_next`, and only then runs the softmax of tile t, so the
  // matrix pipe works on the next tile while the vector ALU exponentiates
  // this one.  K[t] and V[t] live in slot t%2 = PAR of their rings.
  auto tile_step = [&](int t, auto par_const, auto last_const, v16f(&s_in)[2], v16f(&s_next)[2])
                       __attribute__((always_inline)) {
    v16f s_here[2];
    v16f(&s)[2] = PIPE ? s_in : s_here;
    constexpr int PAR = decltype(par_const)::value;
    constexpr bool LAST = decltype(last_const)::value; // no tile t+1: nothing to issue ahead
    wait_loads_and_lds_reads();       // this wave's parts of K[t+1] and V[t] have landed ...
    __builtin_amdgcn_s_barrier();     // ... everyone's have; K[t] and V[t-1] are no longer read
    if constexpr (!PIPE) {
      // plain double buffering: request tile t+1, then compute tile t's scores
      lk.issue((t + 1) * kBKV, k_slot(PAR ^ 1)); // past the end: zeros, no traffic
      lv.issue((t + 1) * kBKV, v_slot(PAR ^ 1));
      scores(std::integral_constant<int, PAR>{}, s);
    } else if constexpr (!LAST) {
      lk.issue((t + 2) * kBKV, k_slot(PAR)); // past the end: zeros, no traffic
      lv.issue((t + 1) * kBKV, v_slot(PAR ^ 1));
    }

    if constexpr (QKI8) {
      const float zp = (float)p.zero_point;
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float raw = s[st][v]; // (a bit cast applied to a vector element directly reads element 0)
          s[st][v] = (float)__builtin_bit_cast(int, raw) - zp;
        }
    }
    // ---- online softmax on this lane's 32 scores of row q_row
    const int key_base = t * kBKV + 4 * h;
    const bool tail = LAST && (t + 1) * kBKV > p.seq_k; // only the last tile can be ragged
    if constexpr (!plain) {
      // element offsets inside one g slice of the bias fit 32 bits (host check)
      const unsigned bias_js = (unsigned)p.bias_js;
      const unsigned boff = (unsigned)q_row * (unsigned)p.bias_is + (unsigned)key_base * bias_js;
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int kofs = st * 32 + 8 * (v >> 2) + (v & 3);
          float x = s[st][v];
          const bool in_range = key_base + kofs < p.seq_k && q_row < p.seq_q;
          if (scale_t != nullptr && in_range)
            x = x * elem_to_f32<DT>(scale_t[boff + (unsigned)kofs * bias_js]);
          x = x * c_scale;
          if (bias != nullptr && in_range)
            x = x + elem_to_f32<DT>(bias[boff + (unsigned)kofs * bias_js]) * kLog2e;
          // where(mask, x, other): a select behind the element-wise chain (mixr-attn-where.mlir:11)
          if (mask != nullptr && in_range && mask[boff + (unsigned)kofs * bias_js] == 0)
            x = elem_to_f32<DT>(other[boff + (unsigned)kofs * bias_js]) * kLog2e;
          s[st][v] = x;
        }
    }
    if (tail) {
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          int key = key_base + st * 32 + 8 * (v >> 2) + (v & 3);
          s[st][v] = key < p.seq_k ? s[st][v] : -INFINITY;
        }
    }
    // row maximum: four independent chains, then across the two wave halves
    float mc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
      mc[c] = fmaxf(s[c >> 1][(c & 1) * 8], s[c >> 1][(c & 1) * 8 + 1]);
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 2; v < 8; ++v)
        mc[c] = fmaxf(mc[c], s[c >> 1][(c & 1) * 8 + v]);
    float mt = half_swap_max_fast(fmaxf(fmaxf(mc[0], mc[1]), fmaxf(mc[2], mc[3])));
    if (plain)
      mt = mt * c_scale;
    // The running maximum only moves when some row's maximum grew by more
    // than kSlack (log2 units): until then p = 2^(s - m_run) <= 2^kSlack,
    // harmless in f16/bf16 and in the f32 sums, and the final division by the
    // row sum cancels the stale maximum exactly.
    constexpr float kSlack = 8.0f;
    if (__builtin_amdgcn_ballot_w64(mt > m_run + kSlack) != 0) {
      const float m_new = fmaxf(m_run, mt);
      const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          o[dt][v] *= alpha;
      m_run = m_new;
    }
    // same basic block as the exponentials below: the scheduler interleaves
    if constexpr (PIPE && !LAST)
      scores(std::integral_constant<int, PAR ^ 1>{}, s_next);
    const float m_use = (m_run == -INFINITY) ? 0.0f : m_run;
    const float cs = plain ? c_scale : 1.0f;
    float psum = 0.0f;
    uint32_t pp[2][8];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int v = 0; v < 16; v += 2) {
        float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[st][v], cs, -m_use));
        float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[st][v + 1], cs, -m_use));
        psum += p0 + p1;
        pp[st][v >> 1] = pack2_fast<DT>(p0, p1);
      }
    l_run += psum;

    // ---- O^T += V^T * P^T ; K step (st,u) covers keys 32*st + 16*u + [0,16)
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        v4i pf = {(int)pp[st][4 * u + 0], (int)pp[st][4 * u + 1], (int)pp[st][4 * u + 2],
                  (int)pp[st][4 * u + 3]};
        constexpr int kSliceB = 16 * Gm::ROWB; // 16 keys
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) {
          attn_lds_char_t *a0 = v_slot(PAR) + voff(dt) + (st * 2 + u) * kSliceB;
          v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_v4s_t *)a0);
          v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_v4s_t *)(a0 + 8 * Gm::ROWB));
          v2i l2 = __builtin_bit_cast(v2i, lo), h2 = __builtin_bit_cast(v2i, hi);
          v4i vf = {l2[0], l2[1], h2[0], h2[1]};
          o[dt] = mma32<DT>(vf, pf, o[dt]);
        }
      }
  };

  v16f s_even[2], s_odd[2];
  if constexpr (PIPE) {
    wait_vmcnt_attn0();
    __builtin_amdgcn_s_barrier();
    scores(std::integral_constant<int, 0>{}, s_even);
  }
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  int t = 0;
  if constexpr (!PIPE) {
    for (; t < nkv; t += 2) {
      tile_step(t, C0{}, std::true_type{}, s_even, s_odd);
      if (t + 1 < nkv)
        tile_step(t + 1, C1{}, std::true_type{}, s_odd, s_even);
    }
  } else {
  for (; t + 2 < nkv; t += 2) {
    tile_step(t, C0{}, std::false_type{}, s_even, s_odd);
    tile_step(t + 1, C1{}, std::false_type{}, s_odd, s_even);
  }
  if (t + 1 < nkv) {
    tile_step(t, C0{}, std::false_type{}, s_even, s_odd);
    tile_step(t + 1, C1{}, std::true_type{}, s_odd, s_even);
  } else {
    tile_step(t, C0{}, std::true_type{}, s_even, s_odd);
  }
  }
  wait_vmcnt_attn0(); // drain the out-of-range loads of the step past the end

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
        uint16_t *dst = O + (int64_t)q_row * p.o_is + e0;
        v2i pk = {(int)pack2<DT>(o[dt][4 * vq + 0] * inv, o[dt][4 * vq + 1] * inv),
                  (int)pack2<DT>(o[dt][4 * vq + 2] * inv, o[dt][4 * vq + 3] * inv)};
        *(v2i *)dst = pk;
      }
  }
}

} // namespace rk
