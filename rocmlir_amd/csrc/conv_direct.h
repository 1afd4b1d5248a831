// Forward convolution with the input window resident in LDS (stride 1,
// dilation 1, channel-contiguous input, KYXC filter).
//
// The implicit-GEMM kernel (gemm_conv_dlds.h) streams an im2col row tile per
// K-step, so every input pixel travels global -> LDS once per filter tap that
// touches it: Y*X times.  For small-channel 3x3 layers that traffic, not the
// matrix cores, sets the pace (a 128x128 tile needs the texture path's full
// 64 B/clk to keep the MFMAs fed).  Here a block owns TH consecutive output
// rows (n, ho) of full width, loads the (TH + Y - 1) x (Wi + 2 pad) x C input
// window ONCE, and then walks the reduction (y, x, c) with only the filter
// slice streaming through a small LDS ring; the A fragments of every tap are
// read from the same window at a shifted pixel offset.  The reference does not
// have this schedule: it lowers every convolution to the im2col GEMM
// (ConvToGemm.cpp:1139-1399).
//
// Window rows are "virtual padded rows": V = n * (Hi + 2 pad_h) + hi + pad_h.
// Consecutive output rows of one image need consecutive V, and an image
// boundary inside a tile simply adds the 2 pad_h rows of zero between the two
// images' rows, so a tile may span two images.  Rows whose hi falls outside
// the image, and the pad_w columns, are zero-filled by the load hardware
// (out-of-range buffer offsets), like every other padding in this library.
//
// LDS layout of the window: row v at v * pitch, pitch = the row's bytes
// rounded up to whole 1 KiB load slabs; pixel wp of a row at wp * C bytes; the
// 16-byte chunks of a pixel (v, wp) XOR-swizzled with the key (v*Wo + wp) & 15.
// The 16 lanes of a fragment read hold 16 consecutive output pixels q of one
// tap, whose window pixels have keys (q + const) & 15 -- distinct even where
// the 16 pixels wrap from one output row to the next, so the reads are free
// of bank conflicts for any output width.  The row loop of the fill is
// scalar work (image and input row -> one scalar byte offset, passed as the
// load's soffset); per lane and load only the swizzle is recomputed.
//
// Block = 4 waves; wave w owns output channels [32 w, 32 w + 32) of the
// block's 128 and all TMB 32-pixel blocks of the tile (TMB accumulator
// tiles).  MFMA operand roles, accumulator layout and epilogue are those of
// the implicit-GEMM kernel.
#pragma once
#include "gemm_conv_dlds.h"

namespace rk {

constexpr int kDirectWindowBytes = 96 * 1024;
constexpr int kDirectSlabsPerWave = 8; // a window row is at most 32 KiB

template <int DT, int TMB, int MSPLIT, bool RICH = false>
__device__ __forceinline__ void conv_direct_body(const void *in, const void *fil, void *out, const void *aux,
                                                 const void *res, const RockConvParams &p) {
  using Tr = MmaTraits<DT>;
  using Acc = typename Tr::Acc;
  constexpr int ES = Tr::ES;
  constexpr int NWAVE = 4 * MSPLIT, BN = 128, RB = 128, NS = 3;
  constexpr int TMW = (TMB + MSPLIT - 1) / MSPLIT; // 32-pixel blocks per wave
  constexpr int B_STAGE = BN * RB;
  constexpr int STEPS = DlGeom<RB>::CHUNKS / (2 * Tr::CHUNKS); // MFMA K steps per 128-byte K-step
  constexpr int B_LOADS = SlabGeom<BN, NWAVE, RB>::PER_WAVE;
  typedef __attribute__((address_space(3))) void lds_void;

  __shared__ __attribute__((aligned(1024))) char lds[kDirectWindowBytes + NS * B_STAGE];
  char *win = lds;
  char *ring = lds + kDirectWindowBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int nb = wave & 3, mh = wave >> 2; // this wave's 32-channel block and share of the pixel blocks

  int g, tm, tn;
  decode_block(p.tiles_m, p.tiles_n, p.g, p.group_m, p.xcd_remap, g, tm, tn);
  const int n0 = tn * BN;

  // ---- the tile: output rows r = n*Ho + ho in [r0, r_end)
  const int TH = p.rows_per_tile;
  const int rows_total = p.n * p.ho;
  const int r0 = tm * TH;
  const int r_end = min(r0 + TH, rows_total);
  const int Hp = p.hi + 2 * p.pad_h, Wp = p.wi + 2 * p.pad_w;
  const int n_first = r0 / p.ho, ho_first = r0 - n_first * p.ho;
  const int r_last = r_end - 1;
  const int n_last = r_last / p.ho;
  const int nv = (n_last - n_first) * Hp + (r_last - n_last * p.ho) - ho_first + p.y; // window rows
  const int cb = p.c * ES;                    // bytes per pixel (power of two, >= 128)
  const int cpp_log = 31 - __builtin_clz(cb) - 4; // log2(chunks per pixel)
  // chunk swizzle: 16 adjacent pixels must spread over one 256-byte bank
  // period, so columns are counted in units of "pixels per period"
  const int swz_mask = min((1 << cpp_log) - 1, 15);
  const int swz_shift = max(0, 4 - cpp_log);
  const int row_slabs = (Wp * cb + 1023) >> 10; // 1 KiB load slabs per window row
  const int pitch = row_slabs << 10;

  // ---- window fill: slab j of every row is issued by wave j % 4
  {
    __amdgpu_buffer_rsrc_t rsrc = dl_rsrc((const char *)in + (int64_t)g * p.in_gs * ES);
    // per slab of a row: this lane's window column, physical chunk and source offset inside an input row
    int col_wp[kDirectSlabsPerWave], col_pc[kDirectSlabsPerWave];
    unsigned col_off[kDirectSlabsPerWave];
#pragma unroll
    for (int jj = 0; jj < kDirectSlabsPerWave; ++jj) {
      const int c = ((wave + jj * NWAVE) << 6) + lane; // chunk index inside the window row
      const int wp = c >> cpp_log;
      const int wi = wp - p.pad_w;
      col_wp[jj] = wp;
      col_pc[jj] = c & ((1 << cpp_log) - 1);
      col_off[jj] = (wp < Wp && wi >= 0 && wi < p.wi) ? (unsigned)(wi * (int)p.in_ws * ES) : kOobOffset;
    }
    int n = n_first, hp = ho_first; // image and padded input row of window row v (scalar)
    for (int v = 0; v < nv; ++v) {
      const int hi = hp - p.pad_h;
      const bool row_ok = hi >= 0 && hi < p.hi;
      const int soff = row_ok ? (n * (int)p.in_ns + hi * (int)p.in_hs) * ES : 0;
      const int key_row = v * p.wo;
#pragma unroll
      for (int jj = 0; jj < kDirectSlabsPerWave; ++jj) {
        const int j = wave + jj * NWAVE;
        if (j < row_slabs) {
          // physical chunk pc holds logical chunk lc
          const int lc = col_pc[jj] ^ (((key_row + col_wp[jj]) >> swz_shift) & swz_mask);
          const unsigned voff = (row_ok && col_off[jj] != kOobOffset) ? col_off[jj] + (unsigned)(lc * kChunk) : kOobOffset;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void *)(win + v * pitch + (j << 10)), 16, (int)voff,
                                                   soff, 0, 0);
        }
      }
      if (++hp == Hp) {
        hp = 0;
        ++n;
      }
    }
  }

  // ---- filter slices: K-contiguous rows through a ring of NS stages
  auto lb = make_dl_b<DT, BN, NWAVE, RB, LD_ROWS_FAST>(fil, p, g, n0, wave, lane);
  const int nk = (p.K * ES + RB - 1) / RB;
#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    lb.issue(s, ring + s * B_STAGE);

  // ---- window row and column (tap 0,0) of each of this lane's TMB output pixels
  int rowbase[TMW], col[TMW], keybase[TMW]; // LDS row offset, column, swizzle key of the (0,0) tap
  {
    const int q_end = (r_end - r0) * p.wo;
    int q = mh * TMW * 32 + lrow;
    int rl = q / p.wo, wo = q - rl * p.wo;
#pragma unroll
    for (int mb = 0; mb < TMW; ++mb) {
      int ho = ho_first + rl, img = 0;
      if (ho >= p.ho) {
        ho -= p.ho;
        img = 1;
      }
      // pixels past the end of the tile read the window's first pixel; their results are dropped
      const bool live = q < q_end;
      const int vq = live ? img * Hp + ho - ho_first : 0;
      rowbase[mb] = vq * pitch;
      col[mb] = live ? wo : 0;
      keybase[mb] = vq * p.wo + col[mb];
      q += 32;
      wo += 32;
      while (wo >= p.wo) {
        wo -= p.wo;
        ++rl;
      }
    }
  }

  Acc acc[TMW][1];
#pragma unroll
  for (int mb = 0; mb < TMW; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      acc[mb][0][v] = 0;

  const int steps_per_tap = cb / RB;
  int tap_y = 0, tap_x = 0, tap_step = 0; // filter tap and K-step inside the tap's channel run
  int rowaddr[TMW], sw[TMW];

  for (int kt = 0; kt < nk; ++kt) {
    // the window (first iteration) and filter step kt have landed; this wave's
    // LDS reads of step kt-1 have returned
    wait_vmcnt_and_lds_reads<(NS - 2) * B_LOADS>();
    __builtin_amdgcn_s_barrier();
    lb.issue(kt + NS - 1, ring + ((kt + NS - 1) % NS) * B_STAGE);

    if (tap_step == 0) {
#pragma unroll
      for (int mb = 0; mb < TMW; ++mb) {
        const int wp = col[mb] + tap_x;
        rowaddr[mb] = rowbase[mb] + tap_y * pitch + (wp << (cpp_log + 4));
        sw[mb] = ((keybase[mb] + tap_y * p.wo + tap_x) >> swz_shift) & swz_mask;
      }
    }
    const int chunk0 = tap_step * (RB / kChunk); // first chunk of this K-step inside the pixel
    const char *sb = ring + (kt % NS) * B_STAGE;
    // Fragments are double-buffered in registers and the reads of MFMA step
    // s+1 are pinned ahead of the MFMAs of step s: with one wave per SIMD
    // nothing else hides the LDS latency, and left alone the scheduler sinks
    // every read to just before its use.
    Frag<DT> fa[2][TMW], fb[2];
    auto read_step = [&](int s, int buf) __attribute__((always_inline)) {
      fb[buf] = dl_read_frag<DT, RB>(sb, nb * 32 + lrow, s, lgrp);
#pragma unroll
      for (int mb = 0; mb < TMW; ++mb)
#pragma unroll
        for (int c = 0; c < Tr::CHUNKS; ++c) {
          const int chunk = chunk0 + s * 2 * Tr::CHUNKS + 2 * c + lgrp;
          fa[buf][mb].c[c] = *(const v4i *)(win + rowaddr[mb] + ((chunk ^ sw[mb]) << 4));
        }
    };
    read_step(0, 0);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (s + 1 < STEPS)
        read_step(s + 1, (s + 1) & 1);
#pragma unroll
      for (int mb = 0; mb < TMW; ++mb)
        mma32x32<DT>(fb[s & 1], fa[s & 1][mb], acc[mb][0]);
    }
    if (++tap_step == steps_per_tap) {
      tap_step = 0;
      if (++tap_x == p.x) {
        tap_x = 0;
        ++tap_y;
      }
    }
  }
  wait_vmcnt<0>(); // drain the out-of-range filter loads before the ring is reused

  // ---- epilogue: the tile is the contiguous pixel range [r0*Wo, r_end*Wo) of the implicit GEMM's M
  RockConvParams pe = p;
  pe.M = r_end * p.wo;
  dl_epilogue<DT, TMW, 1, NWAVE, NS * B_STAGE, RICH>(acc, pe, g, out, aux, res, r0 * p.wo + mh * TMW * 32, n0 + nb * 32, ring,
                                               wave, lane);
}

} // namespace rk
