// Forward convolution with the input window resident in LDS (stride 1,
// dilation 1, channel-contiguous input, filter repacked by a conversion kernel).
//
// The implicit-GEMM kernel (gemm_conv_dlds.h) streams an im2col row tile per
// K-step, so every input pixel travels global -> LDS once per filter tap that
// touches it: Y*X times, and for small-channel 3x3 layers that traffic through
// the 64 B/clk texture path, not the matrix cores, sets the pace.  Here a block
// owns TH consecutive output rows (n, ho) of full width and 128 output
// channels, loads the (TH + Y - 1) x (Wi + 2 pad) x C input window ONCE, and
// walks the reduction (y, x, c) over it: the A fragments of every tap are read
// from the same window at a shifted pixel offset.  The reference does not have
// this schedule: it lowers every convolution to the im2col GEMM
// (ConvToGemm.cpp:1139-1399).
//
// The filter does not pass through LDS at all.  A conversion kernel that runs
// first (rock_relayout_b*, planned by the host) stores it fragment-major:
//   F'[g][32-channel block][K-step of 128 bytes][chunk 0..7][channel 0..31][16 B]
// so that the 64 lanes of a wave fetch one MFMA operand chunk for their 32
// channels with ONE coalesced dwordx4 load straight into registers, two
// K-steps ahead of its use.  With the window static and the filter private to
// each wave, the main loop has no barrier: the four waves of a block (and the
// two blocks that share a CU: 80 KiB of LDS and at most 256 registers each)
// drift apart freely, and one wave's fragment reads and loads hide under the
// others' MFMAs.
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
// tiles).  MFMA operand roles, accumulator layout, order of the reduction and
// epilogue are those of the implicit-GEMM kernel, and so are the results, bit
// for bit.
#pragma once
#include "gemm_conv_dlds.h"

namespace rk {

constexpr int kDirectWindowBytes = 80 * 1024; // two blocks per CU
constexpr int kDirectSlabsPerWave = 8;        // a window row is at most 32 KiB
constexpr int kDirectFilterBlock = 4096;      // bytes of one (32 channels, K-step) block of the repacked filter

// 32-pixel blocks per tile and filter prefetch distance by operand type: the types whose MFMA operands are 32
// bytes per lane (f32, fp8, bf8) hold twice the fragment registers per block, so their tiles are 4 blocks (128
// pixels) against 7 (224 pixels), both inside 256 registers
template <int DT> constexpr int kDirectPixelBlocks = MmaTraits<DT>::CHUNKS == 2 ? 4 : 7;
template <int DT> constexpr int kDirectPrefetch = MmaTraits<DT>::CHUNKS == 2 ? 1 : 2;

// PF: K-steps between the load of a filter fragment set and its use
template <int DT, int TMB, bool RICH = false, int PF = 2>
__device__ __forceinline__ void conv_direct_body(const void *in, const void *filp, void *out, const void *aux,
                                                 const void *res, const RockConvParams &p) {
  using Tr = MmaTraits<DT>;
  using Acc = typename Tr::Acc;
  constexpr int ES = Tr::ES;
  constexpr int NWAVE = 4, BN = 128, RB = 128;
  constexpr int CH = Tr::CHUNKS;
  constexpr int STEPS = DlGeom<RB>::CHUNKS / (2 * CH);
  typedef __attribute__((address_space(3))) void lds_void;
  __shared__ __attribute__((aligned(1024))) char win[kDirectWindowBytes];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int nb = wave;

  int g, tm, tn;
  decode_block(p.tiles_m, p.tiles_n, p.g, p.group_m, p.xcd_remap, g, tm, tn);
  const int n0 = tn * BN;

  const int TH = p.rows_per_tile;
  const int rows_total = p.n * p.ho;
  const int r0 = tm * TH;
  const int r_end = min(r0 + TH, rows_total);
  const int Hp = p.hi + 2 * p.pad_h, Wp = p.wi + 2 * p.pad_w;
  const int n_first = r0 / p.ho, ho_first = r0 - n_first * p.ho;
  const int r_last = r_end - 1;
  const int n_last = r_last / p.ho;
  const int nv = (n_last - n_first) * Hp + (r_last - n_last * p.ho) - ho_first + p.y;
  const int cb = p.c * ES;
  const int cpp_log = 31 - __builtin_clz(cb) - 4;
  const int swz_mask = min((1 << cpp_log) - 1, 15);
  const int swz_shift = max(0, 4 - cpp_log);
  const int row_slabs = (Wp * cb + 1023) >> 10;
  const int pitch = row_slabs << 10;

  // this wave's stream of filter fragments: nk consecutive 4 KiB blocks, one dwordx4 load per fragment chunk
  const int nk = (p.K * ES + RB - 1) / RB;
  const int nblk = (g * p.tiles_n + tn) * 4 + nb; // the repacked filter pads every group to whole 128-channel tiles
  __amdgpu_buffer_rsrc_t frsrc = dl_rsrc((const char *)filp + (int64_t)nblk * nk * kDirectFilterBlock);
  auto load_b = [&](int kt, Frag<DT> *dst) __attribute__((always_inline)) {
    const unsigned voff = kt < nk ? (unsigned)(lane * 16) : kOobOffset;
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int c = 0; c < CH; ++c)
        dst[s].c[c] = __builtin_bit_cast(
            v4i, __builtin_amdgcn_raw_buffer_load_b128(frsrc, (int)voff, kt * kDirectFilterBlock + (s * 2 * CH + 2 * c) * 512, 0));
  };
  Frag<DT> fb[PF + 1][STEPS];
#pragma unroll
  for (int s = 0; s < PF; ++s)
    load_b(s, fb[s]);

  {
    __amdgpu_buffer_rsrc_t rsrc = dl_rsrc((const char *)in + (int64_t)g * p.in_gs * ES);
    int col_wp[kDirectSlabsPerWave], col_pc[kDirectSlabsPerWave];
    unsigned col_off[kDirectSlabsPerWave];
#pragma unroll
    for (int jj = 0; jj < kDirectSlabsPerWave; ++jj) {
      const int c = ((wave + jj * NWAVE) << 6) + lane;
      const int wp = c >> cpp_log;
      const int wi = wp - p.pad_w;
      col_wp[jj] = wp;
      col_pc[jj] = c & ((1 << cpp_log) - 1);
      col_off[jj] = (wp < Wp && wi >= 0 && wi < p.wi) ? (unsigned)(wi * (int)p.in_ws * ES) : kOobOffset;
    }
    int n = n_first, hp = ho_first;
    for (int v = 0; v < nv; ++v) {
      const int hi = hp - p.pad_h;
      const bool row_ok = hi >= 0 && hi < p.hi;
      const int soff = row_ok ? (n * (int)p.in_ns + hi * (int)p.in_hs) * ES : 0;
      const int key_row = v * p.wo;
#pragma unroll
      for (int jj = 0; jj < kDirectSlabsPerWave; ++jj) {
        const int j = wave + jj * NWAVE;
        if (j < row_slabs) {
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

  int rowbase[TMB], col[TMB], keybase[TMB];
  {
    const int q_end = (r_end - r0) * p.wo;
    int q = lrow;
    int rl = q / p.wo, wo = q - rl * p.wo;
#pragma unroll
    for (int mb = 0; mb < TMB; ++mb) {
      int ho = ho_first + rl, img = 0;
      if (ho >= p.ho) {
        ho -= p.ho;
        img = 1;
      }
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

  Acc acc[TMB][1];
#pragma unroll
  for (int mb = 0; mb < TMB; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      acc[mb][0][v] = 0;

  // the window has landed for every wave
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();

  const int steps_per_tap = cb / RB;
  // (tap, K-step inside the tap's channel run) of the step whose fragments are being READ: one MFMA step ahead of
  // the step being multiplied, across K-step boundaries too (the window does not change, nothing to wait for)
  int tap_y = 0, tap_x = 0, tap_step = 0;
  // Address of the fragment chunk of pixel block mb at MFMA step s: the pixel's window offset, with the chunk
  // index (K-step inside the tap, MFMA step, lane half -- disjoint bit fields below the pixel's alignment) XORed
  // with the swizzle key.  Everything but the MFMA step is folded into one base per pixel block and K-step, so a
  // read costs one XOR with a constant (none at step 0).
  int base2[TMB];
  auto tap_addresses = [&]() __attribute__((always_inline)) {
    const int ty = min(tap_y, p.y - 1); // past the last step: any address inside the window
    const int tap_off = ty * pitch + (tap_x << (cpp_log + 4)), tap_key = ty * p.wo + tap_x;
    const int chunk0 = tap_step * (RB / kChunk);
#pragma unroll
    for (int mb = 0; mb < TMB; ++mb) {
      const int sw = ((keybase[mb] + tap_key) >> swz_shift) & swz_mask;
      base2[mb] = (rowbase[mb] + tap_off + (col[mb] << (cpp_log + 4))) ^ (((chunk0 | lgrp) ^ sw) << 4);
    }
  };
  Frag<DT> fa[2][TMB];
  auto read_step = [&](int s, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int mb = 0; mb < TMB; ++mb)
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        fa[buf][mb].c[c] = *(const v4i *)(win + (base2[mb] ^ ((s * 2 * CH + 2 * c) << 4)));
      }
  };
  tap_addresses();
  read_step(0, 0);
  static_assert(STEPS % 2 == 0, "the fragment buffers alternate per MFMA step");

  auto kstep = [&](int kt, const Frag<DT> *fbk) __attribute__((always_inline)) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (s + 1 < STEPS) {
        read_step(s + 1, (s + 1) & 1);
      } else {
        // (selects, not branches: the step stays one scheduling region)
        const int wrap_s = (tap_step + 1 == steps_per_tap) ? 1 : 0;
        tap_step = wrap_s ? 0 : tap_step + 1;
        const int wrap_x = (tap_x + wrap_s == p.x) ? 1 : 0;
        tap_x = wrap_x ? 0 : tap_x + wrap_s;
        tap_y += wrap_x;
        tap_addresses();
        read_step(0, 0);
      }
#pragma unroll
      for (int mb = 0; mb < TMB; ++mb)
        mma32x32<DT>(fbk[s], fa[s & 1][mb], acc[mb][0]);
    }
    // issue order: one fragment read of the next MFMA step behind every MFMA
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int mb = 0; mb < TMB; ++mb) {
        __builtin_amdgcn_sched_group_barrier(0x100, CH, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, DT == MM_F32 ? 4 : 1, 0); // (f32: four 32x32x2 MFMAs per chunk)
      }
  };
  // PF + 1 register buffers in rotation; the loop is unrolled over them so that each is a fixed set of registers
  int kt = 0;
  for (; kt + PF + 1 <= nk; kt += PF + 1) {
#pragma unroll
    for (int u = 0; u < PF + 1; ++u) {
      load_b(kt + u + PF, fb[(u + PF) % (PF + 1)]);
      kstep(kt + u, fb[u]);
    }
  }
#pragma unroll
  for (int u = 0; u < PF + 1; ++u) {
    if (kt + u < nk) {
      load_b(kt + u + PF, fb[(u + PF) % (PF + 1)]);
      kstep(kt + u, fb[u]);
    }
  }

  // (the epilogue opens with a barrier: every wave is done with the window before it becomes the staging area)
  RockConvParams pe = p;
  pe.M = r_end * p.wo;
  dl_epilogue<DT, TMB, 1, NWAVE, kDirectWindowBytes, RICH>(acc, pe, g, out, aux, res, r0 * p.wo, n0 + nb * 32, win, wave,
                                                             lane);
}

} // namespace rk
