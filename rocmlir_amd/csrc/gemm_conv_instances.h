// Kernel-defining macros of the contraction kernels.  Every kernel is compiled
// into a code object of its own: the build (rocmlir_amd/_build.py, which holds
// the list of kernels) writes one small source per kernel that defines
// ROCK_DT / ROCK_DTNAME, includes this header and invokes ONE of the macros
// below.  The host library picks a kernel by name from its perf-config table
// and hands out that kernel's code object.
#pragma once
#include "gemm_splitk.h"
#include "conv_direct.h"

#ifndef ROCK_DT
#error "compile with -DROCK_DT=<operand type code> -DROCK_DTNAME=<suffix>"
#endif

#define RK_CAT_(a, b) a##b
#define RK_CAT(a, b) RK_CAT_(a, b)
#define RK_GEMM_NAME(NAME) RK_CAT(RK_CAT(rock_gemm_, ROCK_DTNAME), NAME)
#define RK_CONV_NAME(NAME) RK_CAT(RK_CAT(rock_conv_, ROCK_DTNAME), NAME)

// element-wise loaders: any strides
#define RK_GEMM(NAME, BM, BN, WM, WN, LA, LB)                                                         \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_GEMM_NAME(NAME)(                       \
      const void *A, const void *B, void *C, const void *aux, const void *res, RockGemmParams p) {   \
    rk::contraction_body<ROCK_DT, BM, BN, WM, WN, LA, LB>(A, B, C, aux, res, p);                      \
  }

// convolution pointer order follows the reference: filter, input, output
#define RK_CONV(NAME, BM, BN, WM, WN, LA, LB)                                                         \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CONV_NAME(NAME)(                       \
      const void *fil, const void *in, void *out, const void *aux, const void *res, RockConvParams p) { \
    rk::contraction_body<ROCK_DT, BM, BN, WM, WN, LA, LB>(in, fil, out, aux, res, p);                 \
  }

// Direct-to-LDS loads: operands of whole 16-byte chunks, each K-contiguous
// (rk::LD_ROWS_FAST) or K-major (rk::LD_COLS_FAST).  RICH = false: the plain
// epilogue (scale, bias, relu / clip, narrowing) unrolled over the
// accumulators; RICH = true (kernel names ending in "_e"): the rolled epilogue
// that also takes a residual tensor and the transcendental activations.
#define RK_GEMM_DL(NAME, BM, BN, WM, WN, RB, LA, LB, RICH)                                            \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_GEMM_NAME(NAME)(                       \
      const void *A, const void *B, void *C, const void *aux, const void *res, RockGemmParams p) {   \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, RB, LA, LB, RICH>(A, B, C, aux, res, p);         \
  }
#define RK_CONV_DL(NAME, BM, BN, WM, WN, RB, RICH)                                                    \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CONV_NAME(NAME)(                       \
      const void *fil, const void *in, void *out, const void *aux, const void *res, RockConvParams p) { \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, RB, rk::LD_CONV_IN_FAST, rk::LD_ROWS_FAST, RICH>( \
        in, fil, out, aux, res, p);                                                                   \
  }

// channel runs whose last chunk holds bytes that are not data (rows of filter taps over narrow pixels)
#define RK_CONV_DL_RUNS(NAME, BM, BN, WM, WN, RB, RICH)                                               \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CONV_NAME(NAME)(                       \
      const void *fil, const void *in, void *out, const void *aux, const void *res, RockConvParams p) { \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, RB, rk::LD_CONV_IN_RUNS, rk::LD_ROWS_FAST, RICH>( \
        in, fil, out, aux, res, p);                                                                   \
  }

// small outputs: 32x32 tile per block, K split over the block's four waves
#define RK_GEMM_SPLITK(NAME, RICH)                                                                    \
  extern "C" __global__ __launch_bounds__(256) void RK_GEMM_NAME(NAME)(                               \
      const void *A, const void *B, void *C, const void *aux, const void *res, RockGemmParams p) {   \
    rk::gemm_body_splitk<ROCK_DT, RICH>(A, B, C, aux, res, p);                                        \
  }

// input window resident in LDS: 224 (types with 32-byte MFMA operands: 128) output pixels x 128 channels per
// block, two blocks per CU;
// `fil` is the filter as the conversion kernel in front repacked it
#define RK_CONV_DIRECT(NAME, RICH)                                                                    \
  extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void RK_CONV_NAME(NAME)( \
      const void *fil, const void *in, void *out, const void *aux, const void *res, RockConvParams p) { \
    rk::conv_direct_body<ROCK_DT, rk::kDirectPixelBlocks<ROCK_DT>, RICH, rk::kDirectPrefetch<ROCK_DT>>(in, fil, out, aux, \
                                                                                                       res, p);        \
  }

// filter gradient: A = the output gradient [k][pixel], B = the im2col matrix [(y, x, c)][pixel], both K-major
#define RK_CONV_BWD_WEIGHT(NAME, BM, BN, WM, WN)                                                      \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CAT(RK_CAT(rock_conv_bwd_weight_, ROCK_DTNAME), NAME)( \
      const void *dy, const void *in, void *dw, const void *aux, const void *res,                      \
      RockConvBwdWeightParams p) {                                                                     \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, 128, rk::LD_COLS_FAST, rk::LD_CONV_COLS, false>(dy, in, dw, aux, \
                                                                                                      res, p);    \
  }
