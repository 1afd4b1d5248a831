// Small-output GEMM: one 32x32 output tile per block, the K range split over
// the block's four waves, partial tiles summed through LDS at the end.
//
// The reference reaches for split-K with atomic adds across workgroups when a
// problem has too few output tiles to fill the chip
// (mlir/lib/Dialect/Rock/Transforms/GemmToGridwise.cpp:268-394, likelihood
// test mlir/lib/Dialect/Rock/Tuning/RockTuningImpl.cpp:962-1008).  Here the
// split stays inside one workgroup: no zero-filled C, no atomics, and a fixed
// summation order ((w0 + w1) + w2) + w3.  For a 512^3 problem the 64x64 tiling
// gives 64 blocks on 256 CUs and 32 serial K-steps per wave; this kernel
// gives 256 blocks and 8 K-steps per wave.
//
// Each wave runs a private copy of the direct-to-LDS pipeline of
// gemm_conv_dlds.h (same loaders, same swizzle, same fragment reads) on its
// own quarter of K and its own LDS stages, so the main loop has no workgroup
// barrier at all; only the final reduction synchronises the block.
#pragma once
#include "gemm_conv_dlds.h"

namespace rk {

template <int DT, bool RICH = false>
__device__ __forceinline__ void gemm_body_splitk(const void *Aptr, const void *Bptr, void *Cptr,
                                                 const void *aux, const void *res, const RockGemmParams &p) {
  using Tr = MmaTraits<DT>;
  using Acc = typename Tr::Acc;
  constexpr int T = 32;      // output tile edge
  constexpr int NWAVE = 4;   // K split
  constexpr int RB = 64;     // K bytes per row per stage
  constexpr int kDlStages = DlGeom<RB>::STAGES;
  constexpr int STEPS = DlGeom<RB>::CHUNKS / (2 * Tr::CHUNKS);
  constexpr int A_BYTES = T * RB, STAGE = 2 * A_BYTES; // per wave
  constexpr int WAVE_LDS = kDlStages * STAGE;
  constexpr int BKE = RB / Tr::ES;
  constexpr int LOADS_PER_STEP = 2 * SlabGeom<T, 1, RB>::PER_WAVE;
  static_assert(WAVE_LDS >= 16 * 64 * 4, "a wave's stages must hold its partial tile");

  __shared__ __attribute__((aligned(1024))) char lds[NWAVE * WAVE_LDS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lgrp = lane >> 5;
  char *wlds = lds + wave * WAVE_LDS;

  int g, tm, tn;
  decode_block(p.tiles_m, p.tiles_n, p.G, p.group_m, p.xcd_remap, g, tm, tn);
  const int m0 = tm * T, n0 = tn * T;

  // every wave loads whole 32-row operand tiles for its own K-steps: the
  // loaders are told they are "wave 0 of 1"
  RowsDl<DT, T, 1, RB> la, lb;
  la.init((const char *)Aptr + (int64_t)g * p.a_gs * Tr::ES, p.a_ms, m0, p.M, p.K, 0, lane);
  lb.init((const char *)Bptr + (int64_t)g * p.b_gs * Tr::ES, p.b_ns, n0, p.N, p.K, 0, lane);

  Acc acc;
#pragma unroll
  for (int v = 0; v < 16; ++v)
    acc[v] = 0;

  const int nk = (p.K + BKE - 1) / BKE;
  const int per_wave = (nk + NWAVE - 1) / NWAVE;
  const int k_begin = wave * per_wave; // steps past nk load zeros and add nothing

#pragma unroll
  for (int s = 0; s < kDlStages - 1; ++s) {
    la.issue(k_begin + s, wlds + s * STAGE);
    lb.issue(k_begin + s, wlds + s * STAGE + A_BYTES);
  }
  for (int i = 0; i < per_wave; ++i) {
    // this wave's loads of step i have landed and its reads of the stage about
    // to be refilled have returned; nobody else touches its stages
    wait_vmcnt_and_lds_reads<(kDlStages - 2) * LOADS_PER_STEP>();
    {
      char *refill = wlds + ((i + kDlStages - 1) % kDlStages) * STAGE;
      const int kt = (i + kDlStages - 1 < per_wave) ? k_begin + i + kDlStages - 1 : nk; // nk = out of range
      la.issue(kt, refill);
      lb.issue(kt, refill + A_BYTES);
    }
    const char *sa = wlds + (i % kDlStages) * STAGE;
    const char *sb = sa + A_BYTES;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      Frag<DT> fb = dl_read_frag<DT, RB>(sb, lrow, s, lgrp);
      Frag<DT> fa = dl_read_frag<DT, RB>(sa, lrow, s, lgrp);
      mma32x32<DT>(fb, fa, acc);
    }
  }
  wait_vmcnt<0>();

  // ---- reduce the four partial tiles: value v of lane l at red[v*64 + l]
  using Elem = decltype(acc[0] + acc[0]);
  Elem *red = (Elem *)wlds;
  if (wave != 0) {
#pragma unroll
    for (int v = 0; v < 16; ++v)
      red[v * 64 + lane] = acc[v];
  }
  __syncthreads();
  if (wave != 0)
    return;
#pragma unroll
  for (int w = 1; w < NWAVE; ++w) {
    const Elem *other = (const Elem *)(lds + w * WAVE_LDS);
#pragma unroll
    for (int v = 0; v < 16; ++v)
      acc[v] = acc[v] + other[v * 64 + lane];
  }

  using Acc4 = decltype(__builtin_shufflevector(acc, acc, 0, 1, 2, 3));
  Acc tile[1][1] = {{acc}};
  dispatch_out_dtype<Tr::INT_ACC>(p.epi.out_dtype, [&](auto od_const) __attribute__((always_inline)) {
    constexpr int OD = decltype(od_const)::value;
    // RICH (kernel suffix "_e"): residual tensor and out-of-line transcendental activations
    direct_epilogue<Tr::INT_ACC, OD, 1, 1, Acc4, RICH>(tile, p, g, Cptr, aux, RICH ? res : nullptr, m0 + lrow,
                                                       n0 + lgrp * 4);
  });
}

} // namespace rk
