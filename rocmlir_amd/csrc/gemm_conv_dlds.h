// Fast path of the contraction kernel: operands stream global -> LDS without
// passing through registers (buffer_load ... lds, 16 bytes per lane) into a
// ring of LDS stages, so K-steps of loads are in flight while one is multiplied.
//
// Same tiling and MFMA mapping as the register-staged body in
// gemm_conv_kernel.h (which remains for arbitrary strides); what differs:
//
//   * K advances RB = 64 or 128 BYTES per stage (four or two stages); a stage
//     holds BM + BN rows of RB/16 sixteen-byte chunks.  One wave-wide load
//     instruction fills a "slab" of 1 KiB (the 64 lanes' 16 bytes land back to
//     back in LDS): 16 rows of 64 bytes or 8 rows of 128.
//   * The XOR swizzle is applied on the source side: the lane that fills
//     physical chunk p of row r fetches logical chunk p ^ swz(r), so the 32
//     rows an MFMA operand reads at one chunk index fall into distinct bank
//     groups.
//   * Zero fill (rows past the end, the K tail, convolution padding) costs no
//     instruction: such lanes use a byte offset beyond the buffer
//     descriptor's range and the hardware writes zeros.  This is the
//     reference's own trick for padded loads
//     (mlir/lib/Dialect/Rock/Transforms/SugarToLoops.cpp:1162-1267).
//   * Synchronisation is explicit: the loads are counted with vmcnt, every
//     iteration waits until at most two younger K-steps are outstanding,
//     crosses ONE workgroup barrier, refills the stage that was consumed in
//     the previous iteration, then multiplies.
//
// Limits checked on the host before this path is chosen: every in-range byte
// offset relative to the block's base pointer is below 2^31.
#pragma once
#include <type_traits>
#include "gemm_conv_kernel.h"

namespace rk {

constexpr unsigned kOobOffset = 0x80000000u; // >= num_records: reads as zero

// Stage geometry.  RB = K bytes per row per stage: 64 (four stages; the big
// tiles, whose MFMA work per K-step already dwarfs the barrier) or 128 (two
// stages; the small tiles, which halve their barrier count and fetch whole
// 128-byte cache lines per row).  A wave-wide load always fills 1 KiB:
// 1024 / RB rows.
template <int RB> struct DlGeom {
  static_assert(RB == 64 || RB == 128, "stage rows are 64 or 128 bytes");
  static constexpr int CHUNKS = RB / 16;
  static constexpr int SLAB_ROWS = 1024 / RB;
  static constexpr int STAGES = RB == 64 ? 4 : 2;
  // XOR swizzle: the 32 rows an MFMA operand reads at one chunk index must fall
  // into distinct bank groups (row pitch 64 B: 4 rows per 256-byte bank period;
  // 128 B: 2 rows per period)
  static __device__ __forceinline__ int swz(int row) {
    return RB == 64 ? ((row >> 2) & 3) : ((row >> 1) & 7);
  }
};

typedef __attribute__((address_space(3))) void lds_void_t;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t dl_rsrc(const void *base) {
  // raw buffer, 2 GiB window, dword-typed data format word used by gfx9 parts
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)kOobOffset, 0x00020000);
}

// a zero the compiler cannot see through (the host build of the body, which the tests step through on the CPU,
// has no scalar registers to pin it to and needs no such barrier)
__device__ __forceinline__ int opaque_zero() {
  int zero = 0;
#ifdef __AMDGCN__
  asm volatile("" : "+s"(zero));
#endif
  return zero;
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}

// vmcnt(N) and lgkmcnt(0) together: the form used before a barrier that hands
// an LDS stage back to the loaders.  The LDS reads of that stage were issued
// before the barrier, but a read can still sit in the LDS queue when another
// wave's refill lands unless its issuer has waited for the data.
template <int N> __device__ __forceinline__ void wait_vmcnt_and_lds_reads() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0070);
}

template <int ROWS, int NW, int RB> struct SlabGeom {
  static constexpr int SLABS = ROWS / DlGeom<RB>::SLAB_ROWS;
  static constexpr int PER_WAVE = SLABS / NW;
  static_assert(ROWS % DlGeom<RB>::SLAB_ROWS == 0 && SLABS % NW == 0,
                "tile rows must split into 1 KiB slabs per wave");
};

// K-contiguous rows (GEMM operands, KYXC filters).
template <int DT, int ROWS, int NW, int RB> struct RowsDl {
  using Sg = SlabGeom<ROWS, NW, RB>;
  using Dg = DlGeom<RB>;
  static constexpr int ES = MmaTraits<DT>::ES;
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned off[Sg::PER_WAVE]; // byte offset of this lane's chunk at K-step 0, or kOobOffset
  int kb[Sg::PER_WAVE];       // byte offset of the chunk inside the 64-byte K-step
  int kbytes;
  int wave;

  __device__ __forceinline__ void init(const void *base, int64_t row_stride, int row0, int rows_total,
                                       int K, int wave_, int lane) {
    wave = wave_;
    kbytes = K * ES;
    rsrc = dl_rsrc((const char *)base + (int64_t)row0 * row_stride * ES);
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      int r = (wave * Sg::PER_WAVE + i) * Dg::SLAB_ROWS + lane / Dg::CHUNKS;
      kb[i] = ((lane % Dg::CHUNKS) ^ Dg::swz(r)) * kChunk;
      off[i] = (row0 + r < rows_total) ? (unsigned)(r * (int)row_stride * ES + kb[i]) : kOobOffset;
    }
  }
  __device__ __forceinline__ void issue(int kt, char *stage) {
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      int k0 = kt * RB;
      unsigned voff = (k0 + kb[i] < kbytes) ? off[i] + (unsigned)k0 : kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc, (lds_void_t *)(stage + (wave * Sg::PER_WAVE + i) * 1024), 16, (int)voff, 0, 0, 0);
    }
  }
};

// Convolution input as implicit-GEMM rows: row m = (n, ho, wo), reduction
// index (y, x, c) with c fastest; channel run is a whole number of chunks.
//
// When the channel run is also a whole number of K-steps (RB bytes), every lane
// of a K-step sits in the same filter tap: the tap walk is scalar state, the
// per-lane work of a step is one add, and the (hi, wi) bounds test runs once
// per tap.  Otherwise each lane tracks the tap of its own chunk.
//
// RUNS: the last chunk of a channel run holds run_valid % EPC elements of data
// and, behind them, whatever follows in memory.  Every lane remembers, per
// stage in flight, which of its chunks are such tails (`tails`), and clears the
// bytes behind the data in LDS once its loads of that stage have landed
// (zero_tails, between the wait for the stage and the barrier that hands it to
// the readers), so that nothing but data reaches the MFMAs.
template <int DT, int ROWS, int NW, int RB, bool RUNS = false> struct ConvInDl {
  using Sg = SlabGeom<ROWS, NW, RB>;
  using Dg = DlGeom<RB>;
  static constexpr int ES = MmaTraits<DT>::ES;
  static constexpr int EPC = kChunk / ES;
  static constexpr int BKE = RB / ES;
  __amdgpu_buffer_rsrc_t rsrc;
  const RockConvParams *p;
  unsigned pix[Sg::PER_WAVE]; // byte offset of input(n, g, 0, 0, 0), or kOobOffset for rows past M
  int h0[Sg::PER_WAVE], w0[Sg::PER_WAVE];
  // per-lane tap state (general case)
  int y[Sg::PER_WAVE], x[Sg::PER_WAVE], cc[Sg::PER_WAVE];
  // uniform tap state (channel run = whole K-steps)
  unsigned tapoff[Sg::PER_WAVE]; // byte offset of this lane's chunk at channel 0 of the tap, or OOB
  int kb[Sg::PER_WAVE];
  int uy, ux, uc0;               // tap and byte offset of the K-step inside the channel run
  bool uniform;
  // what one K-step (BKE elements) advances a per-lane tap by: whole filter
  // rows, taps within a row, channels within a tap
  int step_y, step_x, step_c;
  bool padded; // some window reaches outside the image
  int wave;
  unsigned tails;  // RUNS: bit (stage slot * PER_WAVE + i) set: chunk i of that stage is the tail of a run
  int run_valid;
  static_assert(!RUNS || DlGeom<RB>::STAGES * Sg::PER_WAVE <= 32, "one bit per chunk in flight");

  __device__ __forceinline__ void init(const void *in, const RockConvParams &cp, int g, int row0,
                                       int wave_, int lane) {
    p = &cp;
    wave = wave_;
    uniform = !RUNS && (cp.c * ES) % RB == 0;
    tails = 0;
    run_valid = cp.run_valid;
    // first element of this group's share of the reduction (0 unless the reduction is split over the groups)
    const int kstart = g * cp.k_group_stride;
    // n / d for 0 <= n < 2^31 with the plan's multiply-and-shift constants
    auto div = [](int n, const RockFastDiv &d) { return (int)(((uint64_t)(unsigned)n * d.mul) >> d.shift); };
    {
      const int tap0 = div(kstart, cp.div_c);
      uc0 = (kstart - tap0 * cp.c) * ES;
      uy = div(tap0, cp.div_x);
      ux = tap0 - uy * cp.x;
    }
    {
      const int taps = BKE / cp.c;
      step_c = BKE - taps * cp.c;
      step_y = taps / cp.x;
      step_x = taps - step_y * cp.x;
    }
    padded = cp.pad_h != 0 || cp.pad_w != 0 ||
             (cp.ho - 1) * cp.stride_h + (cp.y - 1) * cp.dil_h >= cp.hi ||
             (cp.wo - 1) * cp.stride_w + (cp.x - 1) * cp.dil_w >= cp.wi;
    rsrc = dl_rsrc((const char *)in + (int64_t)g * cp.in_gs * ES);
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      int r = (wave * Sg::PER_WAVE + i) * Dg::SLAB_ROWS + lane / Dg::CHUNKS;
      int m = row0 + r;
      int mm = min(m, cp.M - 1);
      int n = div(mm, cp.div_image);
      int rem = mm - n * (cp.ho * cp.wo);
      int ho = div(rem, cp.div_row);
      int wo = rem - ho * cp.wo;
      h0[i] = ho * cp.stride_h - cp.pad_h;
      w0[i] = wo * cp.stride_w - cp.pad_w;
      pix[i] = (m < cp.M) ? (unsigned)(n * (int)cp.in_ns * ES) : kOobOffset;
      int lc = (lane % Dg::CHUNKS) ^ Dg::swz(r);
      kb[i] = lc * kChunk;
      int k0 = kstart + lc * EPC;
      int tap = div(k0, cp.div_c);
      cc[i] = k0 - tap * cp.c;
      y[i] = div(tap, cp.div_x);
      x[i] = tap - y[i] * cp.x;
      tapoff[i] = kOobOffset;
    }
    if (uniform && uc0 != 0) // a share of a split reduction that starts inside a tap
      enter_tap();
  }
  // must be called with kt = 0, 1, 2, ... in order (tap state advances)
  // uniform walk: the rows' offsets at channel 0 of the tap (uy, ux)
  __device__ __forceinline__ void enter_tap() {
    const int dh = uy * p->dil_h, dw = ux * p->dil_w;
    const bool tap_ok = uy < p->y;
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      int hi = h0[i] + dh, wi = w0[i] + dw;
      bool v = tap_ok && pix[i] != kOobOffset && hi >= 0 && hi < p->hi && wi >= 0 && wi < p->wi;
      tapoff[i] = v ? pix[i] + (unsigned)((hi * (int)p->in_hs + wi * (int)p->in_ws) * ES + kb[i]) : kOobOffset;
    }
  }
  // RUNS: clears what lies behind the data in this lane's tail chunks of K-step kt (their loads have landed)
  __device__ __forceinline__ void zero_tails(int kt, char *stage) {
    if constexpr (RUNS) {
      typedef __attribute__((address_space(3))) int lds_int_t;
      const int valid_dwords = ((run_valid % EPC) * ES) >> 2;
#pragma unroll
      for (int i = 0; i < Sg::PER_WAVE; ++i) {
        if (tails & (1u << ((kt % DlGeom<RB>::STAGES) * Sg::PER_WAVE + i))) {
          lds_int_t *q = (lds_int_t *)(stage + (wave * Sg::PER_WAVE + i) * 1024 + (threadIdx.x & 63) * 16);
#pragma unroll
          for (int d = 1; d < 4; ++d)
            if (d >= valid_dwords)
              q[d] = 0;
        }
      }
    }
  }
  __device__ __forceinline__ void issue(int kt, char *stage) {
    (void)kt;
    if (uniform) {
      if (uc0 == 0) // entering a tap: one bounds test per row
        enter_tap();
#pragma unroll
      for (int i = 0; i < Sg::PER_WAVE; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc, (lds_void_t *)(stage + (wave * Sg::PER_WAVE + i) * 1024), 16,
            (int)(tapoff[i] + (unsigned)uc0), 0, 0, 0); // OOB + small stays out of range
      uc0 += RB;
      if (uc0 == p->c * ES) {
        uc0 = 0;
        if (++ux == p->x) { ux = 0; ++uy; }
      }
      return;
    }
    // per-lane taps: a K-step moves every lane's chunk on by the same
    // (taps, channels) amount, so the walk is branch-free
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      int hi = h0[i] + y[i] * p->dil_h, wi = w0[i] + x[i] * p->dil_w;
      bool v = pix[i] != kOobOffset && y[i] < p->y;
      if (padded) // uniform
        v = v && hi >= 0 && hi < p->hi && wi >= 0 && wi < p->wi;
      unsigned voff = v ? pix[i] + (unsigned)((hi * (int)p->in_hs + wi * (int)p->in_ws + cc[i]) * ES)
                        : kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc, (lds_void_t *)(stage + (wave * Sg::PER_WAVE + i) * 1024), 16, (int)voff, 0, 0, 0);
      if constexpr (RUNS) {
        const unsigned bit = 1u << ((kt % DlGeom<RB>::STAGES) * Sg::PER_WAVE + i);
        tails = (v && cc[i] + EPC > run_valid) ? (tails | bit) : (tails & ~bit);
      }
      cc[i] += step_c;
      const int carry = cc[i] >= p->c ? 1 : 0;
      cc[i] -= carry ? p->c : 0;
      x[i] += step_x + carry;
      y[i] += step_y;
      if (x[i] >= p->x) { x[i] -= p->x; ++y[i]; }
    }
  }
};

// ---------------------------------------------------------------------------
// K-major operands (A stored [K, M], B stored [K, N]: the contiguous index is
// the tile's row index, not K).  A stage holds the same bytes as for a
// K-contiguous operand, but as KR = RB/ES rows of k, each COLS*ES bytes of
// consecutive m (or n).  MFMA fragments need 16 bytes of consecutive k per
// lane, so they come out of LDS through the transposing reads
// (ds_read_b64_tr_b16 / _b8: 16 lanes fetch a 4 x 16 block of 16-bit or an
// 8 x 16 block of 8-bit elements and each lane receives one column), 32-bit
// elements through four scalar reads.  The reference reaches the same layouts
// through its generic coordinate transforms (GridwiseGemmToBlockwise.cpp:
// 2602-2760 loads "KxD" tiles for either operand orientation).
// ---------------------------------------------------------------------------
template <int DT, int COLS, int RB> struct KmGeom {
  static constexpr int ES = MmaTraits<DT>::ES;
  static constexpr int ROWB = COLS * ES;  // bytes per k-row
  static constexpr int KR = RB / ES;      // k-rows per stage
  static constexpr int CPR = ROWB / kChunk;
  static constexpr int SLAB_ROWS = 1024 / ROWB;
  static_assert(ROWB >= 64 && ROWB <= 1024 && 1024 % ROWB == 0, "a 1 KiB load slab is a whole number of k-rows");
  // Chunk swizzle.  A transposing read touches 4 (16-bit) or 8 (8-bit)
  // consecutive k-rows at the same columns; rows are a multiple of the bank
  // period apart, so each of those rows is moved to its own 64- or 32-byte
  // column group.  The 32-bit path reads one row per instruction and only has
  // to keep the two wave halves (4 rows apart) on different bank halves.
  static __device__ __forceinline__ int swz(int row) {
    int x = ES == 2 ? ((row & 3) << 2) : ES == 1 ? ((row & 7) << 1) : (((row >> 2) & 1) << 3);
    return x & (CPR - 1);
  }
};

template <int DT, int COLS, int NW, int RB> struct ColsDl {
  using Kg = KmGeom<DT, COLS, RB>;
  struct Sg { // same slab count as a K-contiguous tile of the same bytes
    static constexpr int SLABS = COLS * RB / 1024;
    static constexpr int PER_WAVE = SLABS / NW;
    static_assert(SLABS % NW == 0, "stage must split into 1 KiB slabs per wave");
  };
  static constexpr int ES = Kg::ES;
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned off[Sg::PER_WAVE]; // byte offset of this lane's chunk at K-step 0, or kOobOffset
  int krow[Sg::PER_WAVE];     // k-row of the chunk inside a stage
  int kstride_b;              // bytes between consecutive k
  int K;
  int wave;

  __device__ __forceinline__ void init(const void *base, int64_t k_stride, int col0, int cols_total, int K_,
                                       int wave_, int lane) {
    wave = wave_;
    K = K_;
    kstride_b = (int)k_stride * ES;
    rsrc = dl_rsrc((const char *)base + (int64_t)col0 * ES);
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      const int idx = (wave * Sg::PER_WAVE + i) * 64 + lane; // physical chunk inside the stage
      const int r = idx / Kg::CPR, pc = idx % Kg::CPR;
      const int lc = pc ^ Kg::swz(r);                        // logical chunk this lane fetches
      krow[i] = r;
      const bool col_ok = col0 + (lc + 1) * (kChunk / ES) <= cols_total;
      off[i] = col_ok ? (unsigned)(r * kstride_b + lc * kChunk) : kOobOffset;
    }
  }
  __device__ __forceinline__ void issue(int kt, char *stage) {
    const int k0 = kt * Kg::KR;
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      unsigned voff = (k0 + krow[i] < K) ? off[i] + (unsigned)(k0 * kstride_b) : kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc, (lds_void_t *)(stage + (wave * Sg::PER_WAVE + i) * 1024), 16, (int)voff, 0, 0, 0);
    }
  }
};

// The forward im2col matrix as a K-major operand: the reduction index is the
// output pixel m = (n, ho, wo), a stage row holds COLS consecutive columns
// (y, x, c) -- c fastest -- of one pixel, i.e. runs of input channels of the
// pixel (n, ho*s + y*d - p, wo*s + x*d - p), or zeros where that lies in the
// padding.  Which tap and channel a lane's chunk belongs to depends on the
// column only, so it is fixed for the whole loop; the pixel walks on by KR per
// K-step, carried through (wo, ho, n) without a division.  Same LDS placement
// as ColsDl, so the fragments come out through the same transposing reads.
// The reference reaches this operand through its backward-weight coordinate
// transforms (ConvToGemm.cpp:530-768).
template <int DT, int COLS, int NW, int RB> struct ConvColsDl {
  using Kg = KmGeom<DT, COLS, RB>;
  struct Sg {
    static constexpr int SLABS = COLS * RB / 1024;
    static constexpr int PER_WAVE = SLABS / NW;
    static_assert(SLABS % NW == 0, "stage must split into 1 KiB slabs per wave");
  };
  static constexpr int ES = Kg::ES;
  __amdgpu_buffer_rsrc_t rsrc;
  int krow[Sg::PER_WAVE];                // k-row (pixel) of the chunk inside a stage
  int coff[Sg::PER_WAVE];                // byte offset of the chunk's channels inside a pixel, or -1: column beyond N
  int dy[Sg::PER_WAVE], dx[Sg::PER_WAVE]; // the tap's displacement in input rows / pixels
  int n[Sg::PER_WAVE], ho[Sg::PER_WAVE], wo[Sg::PER_WAVE]; // the output pixel this lane loads for next
  int s_n, s_h, s_w;                     // KR pixels as (images, rows, pixels)
  int K, hi_, wi_, ho_, wo_, sh, sw, pix_bytes, wave;

  __device__ __forceinline__ void init(const void *in, const RockConvBwdWeightParams &p, int g, int col0, int wave_,
                                       int lane) {
    wave = wave_;
    K = p.K;
    hi_ = p.hi; wi_ = p.wi; ho_ = p.ho; wo_ = p.wo;
    sh = p.stride_h; sw = p.stride_w;
    pix_bytes = (int)p.in_pix_stride * ES;
    rsrc = dl_rsrc(in);
    {
      const int kr = Kg::KR, img = p.ho * p.wo;
      s_n = kr / img;
      const int rem = kr - s_n * img;
      s_h = rem / p.wo;
      s_w = rem - s_h * p.wo;
    }
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      const int idx = (wave * Sg::PER_WAVE + i) * 64 + lane; // physical chunk inside the stage
      const int r = idx / Kg::CPR, pc = idx % Kg::CPR;
      const int lc = pc ^ Kg::swz(r);                        // logical chunk this lane fetches
      krow[i] = r;
      const int col = col0 + lc * (kChunk / ES);             // first column of the chunk (c % 8 == 0: one tap)
      const int tap = col / p.c, y = tap / p.x, x = tap - y * p.x;
      coff[i] = col < p.N ? (col - tap * p.c) * ES : -1;
      dy[i] = y * p.dil_h - p.pad_h;
      dx[i] = x * p.dil_w - p.pad_w;
      const int m = g * p.K + r; // batch entry g reduces the pixels [g*K, (g+1)*K)
      const int img = p.ho * p.wo;
      n[i] = m / img;
      const int rem = m - n[i] * img;
      ho[i] = rem / p.wo;
      wo[i] = rem - ho[i] * p.wo;
    }
  }
  // must be called with kt = 0, 1, 2, ... in order (the pixel state advances)
  __device__ __forceinline__ void issue(int kt, char *stage) {
    const int k0 = kt * Kg::KR;
#pragma unroll
    for (int i = 0; i < Sg::PER_WAVE; ++i) {
      const int hi = ho[i] * sh + dy[i], wi = wo[i] * sw + dx[i];
      const bool ok = coff[i] >= 0 && k0 + krow[i] < K && hi >= 0 && hi < hi_ && wi >= 0 && wi < wi_;
      const unsigned voff = ok ? (unsigned)(((n[i] * hi_ + hi) * wi_ + wi) * pix_bytes + coff[i]) : kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc, (lds_void_t *)(stage + (wave * Sg::PER_WAVE + i) * 1024), 16, (int)voff, 0, 0, 0);
      wo[i] += s_w;
      const int cw = wo[i] >= wo_ ? 1 : 0;
      wo[i] -= cw ? wo_ : 0;
      ho[i] += s_h + cw;
      const int ch = ho[i] >= ho_ ? 1 : 0;
      ho[i] -= ch ? ho_ : 0;
      n[i] += s_n + ch;
    }
  }
};

typedef __attribute__((address_space(3))) v4s km_lds_v4s_t;
typedef __attribute__((address_space(3))) v2i km_lds_v2i_t;

// Fragment of the 32 columns [colblock, colblock + 32) of a K-major stage, same
// k assignment as dl_read_frag: lane (col = lane % 32, half = lane / 32) gets
// the 16 bytes of k-chunk  step*2*CHUNKS + 2*c + half.
template <int DT, int COLS, int RB>
__device__ __forceinline__ Frag<DT> dl_read_frag_km(const char *stage, int colblock, int step, int lane) {
  using Kg = KmGeom<DT, COLS, RB>;
  constexpr int ES = Kg::ES, CH = MmaTraits<DT>::CHUNKS;
  const int l16 = lane & 15, g16 = (lane >> 4) & 1, half = lane >> 5;
  Frag<DT> f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int kb = (step * 2 * CH + 2 * c + half) * (kChunk / ES); // first k-row of the chunk
    if constexpr (ES == 2) {
      const int colbyte = (colblock + 16 * g16 + 4 * (l16 & 3)) * 2;
      v2i part[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = kb + 4 * j + (l16 >> 2);
        const char *a = stage + (row * Kg::ROWB + ((((colbyte >> 4) ^ Kg::swz(row))) << 4) + (colbyte & 15));
        part[j] = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((km_lds_v4s_t *)a));
      }
      f.c[c] = v4i{part[0][0], part[0][1], part[1][0], part[1][1]};
    } else if constexpr (ES == 1) {
      const int colbyte = colblock + 16 * g16 + 8 * (l16 & 1);
      v2i part[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = kb + 8 * j + (l16 >> 1);
        const char *a = stage + (row * Kg::ROWB + ((((colbyte >> 4) ^ Kg::swz(row))) << 4) + (colbyte & 15));
        part[j] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((km_lds_v2i_t *)a);
      }
      f.c[c] = v4i{part[0][0], part[0][1], part[1][0], part[1][1]};
    } else {
      const int colbyte = (colblock + (lane & 31)) * 4;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int row = kb + t;
        f.c[c][t] = *(const int *)(stage + (row * Kg::ROWB + ((((colbyte >> 4) ^ Kg::swz(row))) << 4) + (colbyte & 15)));
      }
    }
  }
  return f;
}

template <int DT, int ROWS, int NW, int RB, int KIND>
__device__ __forceinline__ auto make_dl_a(const void *A, const RockGemmParams &p, int g, int m0, int wave, int lane) {
  static_assert(KIND == LD_ROWS_FAST || KIND == LD_COLS_FAST, "GEMM fast paths: K-contiguous or K-major");
  const char *base = (const char *)A + (int64_t)g * p.a_gs * MmaTraits<DT>::ES;
  if constexpr (KIND == LD_COLS_FAST) {
    ColsDl<DT, ROWS, NW, RB> l;
    l.init(base, p.a_ks, m0, p.M, p.K, wave, lane);
    return l;
  } else {
    RowsDl<DT, ROWS, NW, RB> l;
    l.init(base, p.a_ms, m0, p.M, p.K, wave, lane);
    return l;
  }
}
template <int DT, int ROWS, int NW, int RB, int KIND>
__device__ __forceinline__ auto make_dl_b(const void *B, const RockGemmParams &p, int g, int n0, int wave, int lane) {
  const char *base = (const char *)B + (int64_t)g * p.b_gs * MmaTraits<DT>::ES;
  if constexpr (KIND == LD_COLS_FAST) {
    ColsDl<DT, ROWS, NW, RB> l;
    l.init(base, p.b_ks, n0, p.N, p.K, wave, lane);
    return l;
  } else {
    RowsDl<DT, ROWS, NW, RB> l;
    l.init(base, p.b_ns, n0, p.N, p.K, wave, lane);
    return l;
  }
}
template <int DT, int ROWS, int NW, int RB, int KIND>
__device__ __forceinline__ auto make_dl_b(const void *in, const RockConvBwdWeightParams &p, int g, int n0, int wave,
                                          int lane) {
  static_assert(KIND == LD_CONV_COLS, "filter gradient: the second operand is the im2col matrix");
  ConvColsDl<DT, ROWS, NW, RB> l;
  l.init(in, p, g, n0, wave, lane);
  return l;
}
template <int DT, int ROWS, int NW, int RB, int KIND>
__device__ __forceinline__ auto make_dl_a(const void *in, const RockConvParams &p, int g, int m0, int wave, int lane) {
  static_assert(KIND == LD_CONV_IN_FAST || KIND == LD_CONV_IN_RUNS,
                "convolution fast path gathers channel-contiguous input");
  ConvInDl<DT, ROWS, NW, RB, KIND == LD_CONV_IN_RUNS> l;
  l.init(in, p, g, m0, wave, lane);
  return l;
}
template <int DT, int ROWS, int NW, int RB, int KIND>
__device__ __forceinline__ auto make_dl_b(const void *fil, const RockConvParams &p, int g, int n0, int wave, int lane) {
  RowsDl<DT, ROWS, NW, RB> l;
  l.init((const char *)fil + (int64_t)g * p.fil_gs * MmaTraits<DT>::ES, p.fil_ks, n0, p.N, p.K, wave, lane);
  return l;
}

// Fragment of one 32-row block out of a stage: lane (row = lane % 32,
// half = lane / 32) takes chunk  step*2*CHUNKS + 2*c + half  for c in [0, CHUNKS).
template <int DT, int RB>
__device__ __forceinline__ Frag<DT> dl_read_frag(const char *lds, int row, int step, int half) {
  Frag<DT> f;
  constexpr int CH = MmaTraits<DT>::CHUNKS;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    int chunk = step * 2 * CH + 2 * c + half;
    f.c[c] = *(const v4i *)(lds + row * RB + ((chunk ^ DlGeom<RB>::swz(row)) * kChunk));
  }
  return f;
}

// Epilogue of the direct-to-LDS bodies: lane holds m = m_wave + 32*i + lrow,
// n = n_wave + 32*j + 8*q + 4*lgrp + {0..3}.  `lds` is the block's operand
// ring (LDS_BYTES), free once every wave has passed the barrier at the top;
// NWAVES waves call this, each with its own `wave` index in [0, NWAVES); it
// contains a workgroup barrier, so every wave of the block must call it.
template <typename Params>
__device__ __forceinline__ bool dl_epilogue_staged(const Params &p, const void *Cptr) {
  return out_rows_chunk_aligned(p, Cptr, out_elem_size(p.epi.out_dtype));
}

// Epilogue with a residual tensor or a transcendental activation.  Unrolled
// over the accumulator registers, such an epilogue would repeat its loads,
// address arithmetic and math routines for every group of four outputs (128
// times in the largest tile, once more per output type) and dominate the code
// object and its build time.  Instead everything but the register moves is
// rolled: per 32-row block of the wave tile, the raw accumulators are parked in
// the wave's LDS region (16 bytes per lane per group, lane-private), ONE loop
// runs the whole epilogue on each group with the output type as a run-time
// switch and leaves the packed result in its slot, and the results take the
// same staged or direct store as the plain epilogue.
// Store side of the rolled epilogue, the element size a run-time value.
// dl_rich_emit places one slot's packed results: straight into global memory
// when the output rows cannot take 16-byte stores, else at their transposed
// position in the wave's LDS buffer, from where dl_rich_flush writes whole rows.
struct DlRichRow { // the lane's own output row of the current block
  int64_t row_off, n_stride;
  bool in_range, vec_ok;
};
template <int NI, typename Params>
__device__ __forceinline__ void dl_rich_emit(const Params &p, void *Cptr, char *wbuf, const v4i &raw, int t, int es,
                                             const DlRichRow &row, int n_wave, int lane, bool staged_ok) {
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int nloc = (t >> 2) * 32 + (t & 3) * 8 + lgrp * 4;
  if (!staged_ok) {
    const int n = n_wave + nloc;
    if (row.in_range && n < p.N)
      store_packed4(raw, es, Cptr, row.row_off + (int64_t)n * row.n_stride, row.n_stride, n, p.N, row.vec_ok);
    return;
  }
  char *dst = wbuf + lrow * (NI * 32 * es + 16) + nloc * es;
  if (es == 4)
    *(v4i *)dst = raw;
  else if (es == 2)
    *(v2i *)dst = v2i{raw[0], raw[1]};
  else
    *(int *)dst = raw[0];
}
template <int ES, int NI, typename Params>
__device__ __forceinline__ void dl_rich_flush(const Params &p, int g, void *Cptr, char *wbuf, int m_block,
                                              int n_wave, int lane) {
  constexpr int WTN = NI * 32;
  constexpr int ROWB = WTN * ES, PITCH = ROWB + 16;
  constexpr int LPR = ROWB / 16, RPI = 64 / LPR;
  const int rd_row = lane / LPR, rd_cb = (lane % LPR) * 16;
#pragma unroll
  for (int r0 = 0; r0 < 32; r0 += RPI) {
    const int row = r0 + rd_row;
    v4i d = *(const v4i *)(wbuf + row * PITCH + rd_cb);
    const int m = m_block + row;
    const int n = n_wave + rd_cb / ES;
    if (m < p.M && n < p.N) {
      int64_t row_off, n_stride;
      bool vec_ok;
      out_row_addr(p, g, m, Cptr, row_off, n_stride, vec_ok);
      *(v4i *)((char *)Cptr + (row_off + n) * ES) = d;
    }
  }
}

// The residual values of one 32-row block in the accumulator layout: slot t
// holds the 4 channels n_wave + (t/4)*32 + (t%4)*8 + lgrp*4 + {0..3} of the
// lane's row, as raw elements packed back to back.  Whole, aligned groups
// only (the caller checks); all loads sit in one basic block per element
// size so that they are in flight together.
template <int NI>
__device__ __forceinline__ void dl_load_residual_block(v4i (&rr)[NI * 4], const char *row, int es, int n_wave,
                                                       int lgrp) {
  auto one = [&](auto es_const) __attribute__((always_inline)) {
    constexpr int ES = decltype(es_const)::value;
#pragma unroll
    for (int t = 0; t < NI * 4; ++t) {
      const int n = n_wave + (t >> 2) * 32 + (t & 3) * 8 + lgrp * 4;
      const char *src = row + n * ES;
      v4i r = {0, 0, 0, 0};
      if constexpr (ES == 4)
        r = *(const v4i *)src;
      else if constexpr (ES == 2) {
        const v2i x = *(const v2i *)src;
        r[0] = x[0];
        r[1] = x[1];
      } else
        r[0] = *(const int *)src;
      rr[t] = r;
    }
  };
  if (es == 4)
    one(std::integral_constant<int, 4>{});
  else if (es == 2)
    one(std::integral_constant<int, 2>{});
  else
    one(std::integral_constant<int, 1>{});
}

// 4 packed elements of the output type widened (the inverse of epilogue_pack4)
__device__ __forceinline__ void unpack4_rt(const v4i &raw, int od, float (&f)[4]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t h = (uint32_t)raw[k >> 1] >> (16 * (k & 1));
    const uint8_t b = (uint8_t)((uint32_t)raw[0] >> (8 * k));
    const int word = raw[k]; // a copy: bit-casting the vector element itself reads element 0
    switch (od) {
    case ROCK_F32: f[k] = __builtin_bit_cast(float, word); break;
    case ROCK_F16: f[k] = (float)__builtin_bit_cast(_Float16, (uint16_t)h); break;
    case ROCK_BF16: f[k] = __builtin_bit_cast(float, h << 16); break;
    case ROCK_I8: f[k] = (float)(int8_t)b; break;
    case ROCK_FP8: f[k] = e4m3fn_to_f32(b); break;
    case ROCK_BF8: f[k] = e5m2_to_f32(b); break;
    default: f[k] = (float)word; break;
    }
  }
}

template <int DT, int MI, int NI, int NWAVES, int LDS_BYTES, typename Params>
__device__ __forceinline__ void dl_epilogue_rich(typename MmaTraits<DT>::Acc (&acc)[MI][NI], const Params &p, int g,
                                                 void *Cptr, const void *aux, const void *res, int m_wave,
                                                 int n_wave, char *lds, int wave, int lane, bool staged_ok) {
  using Tr = MmaTraits<DT>;
  constexpr int WTN = NI * 32;
  constexpr int WBUF = 32 * (WTN * 4 + 16);
  static_assert(NWAVES * WBUF <= LDS_BYTES, "staging buffers must fit in the operand stages");
  static_assert(NI * 4 * 1024 <= WBUF, "parked values must fit in the wave's staging buffer");
  using Acc4 = decltype(__builtin_shufflevector(acc[0][0], acc[0][0], 0, 1, 2, 3));
  const RockEpilogue &e = p.epi;
  const int lrow = lane & 31, lgrp = lane >> 5;
  char *wbuf = lds + wave * WBUF;
  const int od = e.out_dtype;
  const int es = out_elem_size(od);
  const bool slow = activation_is_slow(e);
  const bool int_out = Tr::INT_ACC && od == ROCK_I32;
  // Unrolled over the blocks at compile time (a loop the compiler leaves
  // rolled would index the accumulator registers dynamically, which sends them
  // through scratch memory); the bulk of each block's code is the rolled slot
  // loop below.
  // Per block: the lane's own row and its residual values.  Rows whose groups
  // of four are whole and aligned (the usual case) load them as vectors, all
  // in flight together and one block ahead of their use; otherwise element by
  // element in the slot loop.
  DlRichRow rows[MI];
  bool res_vecs[MI];
  v4i rr2[2][NI * 4];
  auto prefetch = [&](auto ibc) __attribute__((always_inline)) {
    constexpr int ib = decltype(ibc)::value;
    const int m = m_wave + ib * 32 + lrow;
    DlRichRow row{0, 1, m < p.M, false};
    if (row.in_range)
      out_row_addr(p, g, m, Cptr, row.row_off, row.n_stride, row.vec_ok);
    bool rv = false;
    if (e.residual_op && row.in_range) {
      const char *rowp = (const char *)res + row.row_off * es;
      rv = row.n_stride == 1 && (((uintptr_t)rowp) & (uintptr_t)(4 * es - 1)) == 0 && n_wave + WTN <= p.N;
      if (rv)
        dl_load_residual_block<NI>(rr2[ib & 1], rowp, es, n_wave, lgrp);
    }
    rows[ib] = row;
    res_vecs[ib] = rv;
  };
  prefetch(std::integral_constant<int, 0>{});
  static_for<MI>([&](auto ic) __attribute__((always_inline)) {
    constexpr int i = decltype(ic)::value;
    if constexpr (i + 1 < MI)
      prefetch(std::integral_constant<int, i + 1>{});
    const DlRichRow row = rows[i];
    const bool res_vec = res_vecs[i];
    v4i(&rr)[NI * 4] = rr2[i & 1];
    const bool with_res = e.residual_op && row.in_range;
    const int64_t res_off = row.row_off, res_ns = row.n_stride;
    // Steps 1-3 where the accumulators sit.  With a clamp-type activation and
    // no ragged residual in this wave the results are finished in registers;
    // otherwise they are parked in LDS as f32 and finished by the rolled slot
    // loop, the single copy of the activation routines.
    const bool ragged = with_res && !res_vec;
    const bool park = !int_out && (slow || __builtin_amdgcn_ballot_w64(ragged) != 0);
    const bool park_int = int_out && __builtin_amdgcn_ballot_w64(ragged) != 0;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int t = j * 4 + q;
        const int n = n_wave + j * 32 + q * 8 + lgrp * 4;
        Acc4 a4 = {acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        char *slot = wbuf + (t * 64 + lane) * 16;
        if (int_out) {
          if constexpr (Tr::INT_ACC) {
            v4i v = epilogue_convert4<true, ROCK_I32>(a4, e, aux, n, p.N);
            if (res_vec) {
#pragma unroll
              for (int k = 0; k < 4; ++k)
                v[k] = e.residual_op == ROCK_RES_ADD ? v[k] + rr[t][k] : v[k] * rr[t][k];
            }
            if (park_int)
              *(v4i *)slot = v;
            else
              dl_rich_emit<NI>(p, Cptr, wbuf, v, t, es, row, n_wave, lane, staged_ok);
          }
        } else {
          float v[4];
          epilogue_affine4<Tr::INT_ACC, ROCK_DTYPE_COUNT, true>(a4, e, aux, n, p.N, nullptr, 0, 1, v);
          if (res_vec) {
            float rf[4];
            unpack4_rt(rr[t], od, rf);
#pragma unroll
            for (int k = 0; k < 4; ++k)
              v[k] = e.residual_op == ROCK_RES_ADD ? v[k] + rf[k] : v[k] * rf[k];
          }
          if (park) {
            *(v4f *)slot = v4f{v[0], v[1], v[2], v[3]};
          } else {
            if (e.activation) {
#pragma unroll
              for (int k = 0; k < 4; ++k)
                v[k] = activation_fast(v[k], e);
            }
            dl_rich_emit<NI>(p, Cptr, wbuf, epilogue_pack4_rt(v, od, e, n, p.N), t, es, row, n_wave, lane, staged_ok);
          }
        }
      }
    }
    if (park || park_int) {
      if (ragged) { // ragged or unaligned rows: one residual element at a time
#pragma unroll 1
        for (int t = 0; t < NI * 4; ++t) {
          char *slot = wbuf + (t * 64 + lane) * 16;
          const int n = n_wave + (t >> 2) * 32 + (t & 3) * 8 + lgrp * 4;
#pragma unroll 1
          for (int r = 0; r < 4; ++r) {
            if (n + r >= p.N)
              continue;
            const int64_t idx = res_off + (int64_t)(n + r) * res_ns;
            if (int_out) {
              int *f = (int *)slot + r;
              const int rv = ((const int *)res)[idx];
              *f = e.residual_op == ROCK_RES_ADD ? *f + rv : *f * rv;
            } else {
              float *f = (float *)slot + r;
              const float rv = load_out_elem_rt(res, idx, od);
              *f = e.residual_op == ROCK_RES_ADD ? *f + rv : *f * rv;
            }
          }
        }
      }
      if (!int_out) {
#pragma unroll 1
        for (int t = 0; t < NI * 4; ++t) {
          char *slot = wbuf + (t * 64 + lane) * 16;
          if (slow) {
#pragma unroll 1
            for (int r = 0; r < 4; ++r) {
              float *f = (float *)slot + r;
              *f = activation_slow(*f, e.activation);
            }
          }
          const v4f x = *(const v4f *)slot;
          float v[4] = {x[0], x[1], x[2], x[3]};
          if (!slow && e.activation) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              v[r] = activation_fast(v[r], e);
          }
          *(v4i *)slot = epilogue_pack4_rt(v, od, e, n_wave + (t >> 2) * 32 + (t & 3) * 8 + lgrp * 4, p.N);
        }
      }
      // results back into registers, then to their store positions: every lane
      // has read its slots before any overwrites them (LDS operations of one
      // wave complete in order)
      v4i raw[NI * 4];
#pragma unroll
      for (int t = 0; t < NI * 4; ++t)
        raw[t] = *(const v4i *)(wbuf + (t * 64 + lane) * 16);
      RK_WAVE_LDS_ORDER();
#pragma unroll
      for (int t = 0; t < NI * 4; ++t)
        dl_rich_emit<NI>(p, Cptr, wbuf, raw[t], t, es, row, n_wave, lane, staged_ok);
    }
    if (staged_ok) {
      RK_WAVE_LDS_ORDER();
      if (es == 4)
        dl_rich_flush<4, NI>(p, g, Cptr, wbuf, m_wave + i * 32, n_wave, lane);
      else if (es == 2)
        dl_rich_flush<2, NI>(p, g, Cptr, wbuf, m_wave + i * 32, n_wave, lane);
      else
        dl_rich_flush<1, NI>(p, g, Cptr, wbuf, m_wave + i * 32, n_wave, lane);
      RK_WAVE_LDS_ORDER();
    }
  });
}

// RICH kernels are separate instantiations (kernel name suffix "_e") so that
// the plain kernels' register allocation is untouched by the rich path.
template <int DT, int MI, int NI, int NWAVES, int LDS_BYTES, bool RICH = false, typename Params>
__device__ __forceinline__ void dl_epilogue(typename MmaTraits<DT>::Acc (&acc)[MI][NI], const Params &p_in, int g,
                                            void *Cptr, const void *aux, const void *res, int m_wave, int n_wave, char *lds,
                                            int wave, int lane) {
  using Tr = MmaTraits<DT>;
  Params p = p_in; // a convolution's per-channel pointers moved on to this block's group
  group_channel_pointers(p, aux, g);
  constexpr int WTN = NI * 32;
  const int lrow = lane & 31, lgrp = lane >> 5;
  const RockEpilogue &e = p.epi;
  using Acc4 = decltype(__builtin_shufflevector(acc[0][0], acc[0][0], 0, 1, 2, 3));
  const bool staged_ok = dl_epilogue_staged(p, Cptr);
  if constexpr (RICH) {
    __builtin_amdgcn_s_barrier(); // every wave is done reading the operand stages
    dl_epilogue_rich<DT, MI, NI, NWAVES, LDS_BYTES>(acc, p, g, Cptr, aux, res, m_wave, n_wave, lds, wave, lane,
                                                    staged_ok);
    return;
  }
  // (the 16-byte vectors of consecutive rows start at multiples of 16 bytes from the wave's first row and must
  // neither straddle an image nor run past the last row: the implicit-GEMM tiles start at multiples of 32 rows,
  // the window-resident kernel's at any multiple of the output width and end with their last output row)
  const int out_es = out_elem_size(e.out_dtype);
  const bool cols_ok = !staged_ok && out_cols_chunk_aligned(p, Cptr, out_es) &&
                       (((int64_t)m_wave * out_es | (int64_t)p.M * out_es) & 15) == 0;
  if (staged_ok || cols_ok)
    __builtin_amdgcn_s_barrier(); // every wave is done reading the operand stages

  dispatch_out_dtype<Tr::INT_ACC>(e.out_dtype, [&](auto od_const) __attribute__((always_inline)) {
    constexpr int OD = decltype(od_const)::value;
    // plain epilogue (scale, bias, relu / clip, narrowing): unrolled over the registers
    if (cols_ok) {
      // m-contiguous output (NCHW-style convolution output, transposed C): each
      // 32-row block goes through the wave's LDS region as [channel][row], and
      // leaves as 16-byte vectors of consecutive rows
      constexpr int ES = OutElemSize<OD>::value;
      constexpr int MP = 32 * ES + (ES == 4 ? 0 : 16); // bytes per channel row in LDS
      constexpr int VPR = 32 * ES / 16;                // 16-byte vectors per channel row
      constexpr int WBUF = 32 * (WTN * 4 + 16);
      static_assert(WTN * MP <= WBUF && NWAVES * WBUF <= LDS_BYTES, "transposed block must fit in the wave's region");
      char *wbuf = lds + wave * WBUF;
#pragma unroll
      for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int nloc = j * 32 + q * 8 + lgrp * 4;
            Acc4 a4 = {acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                       acc[i][j][4 * q + 3]};
            const v4i raw = epilogue_convert4<Tr::INT_ACC, OD>(a4, e, aux, n_wave + nloc, p.N);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              char *dst = wbuf + (nloc + r) * MP + lrow * ES;
              if constexpr (ES == 4)
                *(int *)dst = raw[r];
              else if constexpr (ES == 2)
                *(uint16_t *)dst = (uint16_t)((uint32_t)raw[r >> 1] >> (16 * (r & 1)));
              else
                *(uint8_t *)dst = (uint8_t)((uint32_t)raw[0] >> (8 * r));
            }
          }
        }
        RK_WAVE_LDS_ORDER();
#pragma unroll
        for (int it = 0; it < WTN * VPR / 64; ++it) {
          const int v = it * 64 + lane;
          const int nloc = v / VPR, mloc = (v % VPR) * (16 / ES);
          const v4i d = *(const v4i *)(wbuf + nloc * MP + mloc * ES);
          const int m = m_wave + i * 32 + mloc, n = n_wave + nloc;
          if (m < p.M && n < p.N) {
            int64_t off, n_stride;
            out_col_addr(p, g, m, off, n_stride);
            *(v4i *)((char *)Cptr + (off + (int64_t)n * n_stride) * ES) = d;
          }
        }
        RK_WAVE_LDS_ORDER();
      }
      return;
    }
    if (!staged_ok) {
      direct_epilogue<Tr::INT_ACC, OD, MI, NI, Acc4, false>(acc, p, g, Cptr, aux, nullptr, m_wave + lrow,
                                                           n_wave + lgrp * 4);
      return;
    }
    // Staged store: each wave transposes one 32-row block of its tile at a
    // time through a private LDS region, so that global stores are 16 bytes
    // per lane and cover whole rows of the wave tile (WTN * ES contiguous
    // bytes per 64/LPR lanes).
    constexpr int ES = OutElemSize<OD>::value;
    constexpr int ROWB = WTN * ES, PITCH = ROWB + 16;
    constexpr int LPR = ROWB / 16, RPI = 64 / LPR;
    constexpr int WBUF = 32 * (WTN * 4 + 16);
    static_assert(NWAVES * WBUF <= LDS_BYTES, "staging buffers must fit in the operand stages");
    char *wbuf = lds + wave * WBUF;
    const int rd_row = lane / LPR, rd_cb = (lane % LPR) * 16;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int j = 0; j < NI; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int nloc = j * 32 + q * 8 + lgrp * 4;
          Acc4 a4 = {acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                     acc[i][j][4 * q + 3]};
          v4i raw = epilogue_convert4<Tr::INT_ACC, OD>(a4, e, aux, n_wave + nloc, p.N);
          char *dst = wbuf + lrow * PITCH + nloc * ES;
          if constexpr (ES == 4)
            *(v4i *)dst = raw;
          else if constexpr (ES == 2)
            *(v2i *)dst = v2i{raw[0], raw[1]};
          else
            *(int *)dst = raw[0];
        }
      }
      RK_WAVE_LDS_ORDER();
#pragma unroll
      for (int r0 = 0; r0 < 32; r0 += RPI) {
        const int row = r0 + rd_row;
        v4i d = *(const v4i *)(wbuf + row * PITCH + rd_cb);
        const int m = m_wave + i * 32 + row;
        const int n = n_wave + rd_cb / ES;
        if (m < p.M && n < p.N) {
          int64_t row_off, n_stride;
          bool vec_ok;
          out_row_addr(p, g, m, Cptr, row_off, n_stride, vec_ok);
          // streaming hint: the kernel never reads its output back, and the burst of
          // whole-row stores that every block issues at the same moment drains faster
          __builtin_nontemporal_store(d, (v4i *)((char *)Cptr + (row_off + n) * ES));
        }
      }
      RK_WAVE_LDS_ORDER();
    }
  });
}


template <int DT, int BM, int BN, int WAVES_M, int WAVES_N, int RB, int LDA, int LDB, bool RICH = false,
          typename Params>
__device__ __forceinline__ void contraction_body_dl(const void *Aptr, const void *Bptr, void *Cptr,
                                                    const void *aux, const void *res, const Params &p) {
  using Tr = MmaTraits<DT>;
  using Acc = typename Tr::Acc;
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N; // wave tile
  constexpr int MI = WTM / 32, NI = WTN / 32;
  constexpr int kDlStages = DlGeom<RB>::STAGES;
  constexpr int STEPS = DlGeom<RB>::CHUNKS / (2 * Tr::CHUNKS); // MFMA K steps per stage
  constexpr int A_BYTES = BM * RB, B_BYTES = BN * RB;
  constexpr int STAGE = A_BYTES + B_BYTES;
  constexpr int BKE = RB / Tr::ES;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32");

  // With a K-major operand the two stages are two LDS objects and the loop is
  // unrolled over them: the compiler puts an s_waitcnt vmcnt(0) in front of every
  // transposing LDS read that follows a load into LDS unless it can tell that
  // the two touch different objects -- between the refill of one stage and the
  // fragment reads of the other that wait would expose the whole load latency
  // in every K-step of the loading waves.
  // (Not for the 256x256 tile of the 8-bit float types: 128 accumulators and 96
  // fragment registers leave the unrolled loop no room and it spills.)
  constexpr bool KM = (LDA == LD_COLS_FAST || LDB == LD_COLS_FAST || LDB == LD_CONV_COLS) &&
                      !(Tr::CHUNKS == 2 && BM * BN >= 256 * 256);
  static_assert(!KM || kDlStages == 2, "K-major operands: two stages, one LDS object each");
  constexpr int WBUF = 32 * (WTN * 4 + 16); // the epilogue's staging region per wave
  static_assert(!KM || (NW / 2) * WBUF <= STAGE, "half the waves stage their stores in each stage");
  __shared__ __attribute__((aligned(1024))) char lds[KM ? STAGE : kDlStages * STAGE];
  __shared__ __attribute__((aligned(1024))) char lds_hi[KM ? STAGE : 1024]; // K-major only

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  const int lrow = lane & 31, lgrp = lane >> 5;

  int g, tm, tn;
  decode_block(p.tiles_m, p.tiles_n, p_batch(p), p.group_m, p.xcd_remap, g, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // Eight-wave blocks put two waves on every SIMD.  Only the upper four issue
  // loads: a burst of load instructions from all eight backs up in the
  // texture path and stalls every wave at once, idling the matrix pipe; this
  // way the lower wave of each SIMD starts its MFMAs right after the barrier
  // and the upper one follows when its loads are out.
  constexpr int NLOAD = NW == 8 ? 4 : NW;
  const bool loader = wave >= NW - NLOAD;
  const int lwave = loader ? wave - (NW - NLOAD) : 0;
  auto la = make_dl_a<DT, BM, NLOAD, RB, LDA>(Aptr, p, g, m0, lwave, lane);
  auto lb = make_dl_b<DT, BN, NLOAD, RB, LDB>(Bptr, p, g, n0, lwave, lane);
  constexpr int LOADS_PER_STEP = decltype(la)::Sg::PER_WAVE + decltype(lb)::Sg::PER_WAVE;

  Acc acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        acc[i][j][v] = 0;

  const int nk = (p.K + BKE - 1) / BKE;

  // K-steps past the end are issued all the same: every lane is then out of
  // range, no memory is touched, and the outstanding-load count stays uniform.
#pragma unroll
  for (int s = 0; s < kDlStages - 1; ++s) {
    if (loader) {
      la.issue(s, lds + s * STAGE);
      lb.issue(s, lds + s * STAGE + A_BYTES);
    }
  }

  // K-step kt: multiplies the stage at `sa`, refills the stage at `refill`
  auto kstep = [&](int kt, const char *sa, char *refill) __attribute__((always_inline)) {
    if constexpr (KM) {
      // The unrolled loop has every fragment address of either stage as a loop
      // invariant, and hoisting them all costs the 8-bit kernels their registers
      // (the second stage lies beyond the reach of the reads' 16-bit offset
      // field).  An offset of zero that the compiler cannot see through keeps
      // the address arithmetic of a step inside the step, one add per read.
      sa += opaque_zero();
    }
    // this wave's loads of K-step kt have landed (two younger steps may be in flight) ...
    wait_vmcnt_and_lds_reads<(kDlStages - 2) * LOADS_PER_STEP>();
    if constexpr (LDA == LD_CONV_IN_RUNS) {
      if (loader)
        la.zero_tails(kt, const_cast<char *>(sa));
      __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the clearing stores are in LDS before the barrier
    }
    // ... and so have everyone else's; everyone is also done reading step kt-1
    __builtin_amdgcn_s_barrier();
    if (loader) {
      la.issue(kt + kDlStages - 1, refill);
      lb.issue(kt + kDlStages - 1, refill + A_BYTES);
    }
    const char *sb = sa + A_BYTES;
    // the fragments of MFMA step s + 1 are fetched while the MFMAs of step s run
    Frag<DT> fa[2][MI], fb[2][NI];
    auto fetch = [&](int s, Frag<DT> *a, Frag<DT> *b) {
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        if constexpr (LDB == LD_COLS_FAST || LDB == LD_CONV_COLS)
          b[j] = dl_read_frag_km<DT, BN, RB>(sb, wn * WTN + j * 32, s, lane);
        else
          b[j] = dl_read_frag<DT, RB>(sb, wn * WTN + j * 32 + lrow, s, lgrp);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        if constexpr (LDA == LD_COLS_FAST)
          a[i] = dl_read_frag_km<DT, BM, RB>(sa, wm * WTM + i * 32, s, lane);
        else
          a[i] = dl_read_frag<DT, RB>(sa, wm * WTM + i * 32 + lrow, s, lgrp);
      }
    };
    fetch(0, fa[0], fb[0]);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (s + 1 < STEPS)
        fetch(s + 1, fa[(s + 1) & 1], fb[(s + 1) & 1]);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
          mma32x32<DT>(fb[s & 1][j], fa[s & 1][i], acc[i][j]);
    }
    // Issue order for the scheduler: the first step's fragment reads, then per
    // step one LDS read of the next step's fragments after every MFMA until
    // they are all out, then the step's remaining MFMAs.
    if constexpr (LDA != LD_COLS_FAST && LDB != LD_COLS_FAST && LDB != LD_CONV_COLS && MI * NI >= MI + NI) {
      __builtin_amdgcn_sched_group_barrier(0x100, MI + NI, 0);
#pragma unroll
      for (int s = 0; s + 1 < STEPS; ++s) {
#pragma unroll
        for (int r = 0; r < MI + NI; ++r) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        if constexpr (MI * NI > MI + NI)
          __builtin_amdgcn_sched_group_barrier(0x008, MI * NI - (MI + NI), 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, MI * NI, 0);
    }
  };
  if constexpr (KM) {
    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
      kstep(kt, lds, lds_hi);
      kstep(kt + 1, lds_hi, lds);
    }
    if (kt < nk)
      kstep(kt, lds, lds_hi);
  } else {
    for (int kt = 0; kt < nk; ++kt)
      kstep(kt, lds + (kt % kDlStages) * STAGE, lds + ((kt + kDlStages - 1) % kDlStages) * STAGE);
  }
  // drain the out-of-range loads issued for steps >= nk before the LDS is released
  wait_vmcnt<0>();

  // the epilogue's staging region of wave w starts WBUF * w bytes behind the pointer it is given
  char *staging = lds;
  if constexpr (KM)
    staging = wave < NW / 2 ? lds : lds_hi - (NW / 2) * WBUF;
  dl_epilogue<DT, MI, NI, NW, kDlStages * STAGE, RICH>(acc, p, g, Cptr, aux, res, m0 + wm * WTM, n0 + wn * WTN, staging,
                                                       wave, lane);
}

} // namespace rk
