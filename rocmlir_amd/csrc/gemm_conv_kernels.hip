// Instantiations of the contraction kernel for one operand type.  Compiled
// once per type with -DROCK_DT=<code> -DROCK_DTNAME=<name> into a gfx950 code
// object; the host library picks a kernel by name from its perf-config table.
#include "gemm_splitk.h"
#include "conv_direct.h"

#ifndef ROCK_DT
#error "compile with -DROCK_DT=<operand type code> -DROCK_DTNAME=<suffix>"
#endif

#define RK_CAT_(a, b) a##b
#define RK_CAT(a, b) RK_CAT_(a, b)

#define RK_GEMM(NAME, BM, BN, WM, WN, LA, LB)                                           \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CAT(                     \
      RK_CAT(rock_gemm_, ROCK_DTNAME), NAME)(const void *A, const void *B, void *C,     \
                                             const void *aux, const void *res, RockGemmParams p) {       \
    rk::contraction_body<ROCK_DT, BM, BN, WM, WN, LA, LB>(A, B, C, aux, res, p);             \
  }

// convolution pointer order follows the reference: filter, input, output
#define RK_CONV(NAME, BM, BN, WM, WN, LA, LB)                                           \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CAT(                     \
      RK_CAT(rock_conv_, ROCK_DTNAME), NAME)(const void *fil, const void *in, void *out,\
                                             const void *aux, const void *res, RockConvParams p) {       \
    rk::contraction_body<ROCK_DT, BM, BN, WM, WN, LA, LB>(in, fil, out, aux, res, p);        \
  }

// fast variants: direct-to-LDS loads, K-contiguous 16-byte aligned operands.
// Each exists twice: NAME with the plain epilogue (scale, bias, relu / clip,
// narrowing) and NAME_e with the rolled epilogue that also takes a residual
// tensor and the transcendental activations.
#define RK_GEMM_DL_X(NAME, BM, BN, WM, WN, RB, LA, LB)                                   \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CAT(                     \
      RK_CAT(rock_gemm_, ROCK_DTNAME), NAME)(const void *A, const void *B, void *C,     \
                                             const void *aux, const void *res, RockGemmParams p) { \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, RB, LA, LB, false>(A, B, C, aux, res, p); \
  }                                                                                     \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CAT(                     \
      RK_CAT(rock_gemm_, ROCK_DTNAME), RK_CAT(NAME, _e))(const void *A, const void *B, void *C, \
                                             const void *aux, const void *res, RockGemmParams p) { \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, RB, LA, LB, true>(A, B, C, aux, res, p); \
  }
#define RK_GEMM_DL(NAME, BM, BN, WM, WN, RB) \
  RK_GEMM_DL_X(NAME, BM, BN, WM, WN, RB, rk::LD_ROWS_FAST, rk::LD_ROWS_FAST)
#define RK_CONV_DL(NAME, BM, BN, WM, WN, RB)                                             \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CAT(                     \
      RK_CAT(rock_conv_, ROCK_DTNAME), NAME)(const void *fil, const void *in, void *out,\
                                             const void *aux, const void *res, RockConvParams p) { \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, RB, rk::LD_CONV_IN_FAST,           \
                            rk::LD_ROWS_FAST, false>(in, fil, out, aux, res, p);        \
  }                                                                                     \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void RK_CAT(                     \
      RK_CAT(rock_conv_, ROCK_DTNAME), RK_CAT(NAME, _e))(const void *fil, const void *in, void *out, \
                                             const void *aux, const void *res, RockConvParams p) { \
    rk::contraction_body_dl<ROCK_DT, BM, BN, WM, WN, RB, rk::LD_CONV_IN_FAST,           \
                            rk::LD_ROWS_FAST, true>(in, fil, out, aux, res, p);         \
  }

// K-major operands: LA / LB name how A and B are stored
#define RK_GEMM_DL_TRANSPOSED(TILE, BM, BN, WM, WN)                                                  \
  RK_GEMM_DL_X(RK_CAT(TILE, _fast_nn), BM, BN, WM, WN, 128, rk::LD_ROWS_FAST, rk::LD_COLS_FAST)      \
  RK_GEMM_DL_X(RK_CAT(TILE, _fast_tn), BM, BN, WM, WN, 128, rk::LD_COLS_FAST, rk::LD_COLS_FAST)      \
  RK_GEMM_DL_X(RK_CAT(TILE, _fast_tt), BM, BN, WM, WN, 128, rk::LD_COLS_FAST, rk::LD_ROWS_FAST)

RK_GEMM_DL(_256x256_fast, 256, 256, 2, 4, 128)
RK_GEMM_DL(_256x128_fast, 256, 128, 4, 2, 128)
RK_GEMM_DL(_128x128_fast, 128, 128, 2, 2, 128)
RK_GEMM_DL(_64x64_fast, 64, 64, 2, 2, 128)
RK_GEMM_DL_TRANSPOSED(_256x256, 256, 256, 2, 4)
RK_GEMM_DL_TRANSPOSED(_128x128, 128, 128, 2, 2)
RK_GEMM_DL_TRANSPOSED(_64x64, 64, 64, 2, 2)
RK_GEMM(_64x64_generic, 64, 64, 2, 2, rk::LD_ROWS_GENERIC, rk::LD_ROWS_GENERIC)

// small outputs: 32x32 tile per block, K split over the block's four waves
extern "C" __global__ __launch_bounds__(256) void RK_CAT(RK_CAT(rock_gemm_, ROCK_DTNAME), _32x32_splitk)(
    const void *A, const void *B, void *C, const void *aux, const void *res, RockGemmParams p) {
  rk::gemm_body_splitk<ROCK_DT, false>(A, B, C, aux, res, p);
}
extern "C" __global__ __launch_bounds__(256) void RK_CAT(RK_CAT(rock_gemm_, ROCK_DTNAME), _32x32_splitk_e)(
    const void *A, const void *B, void *C, const void *aux, const void *res, RockGemmParams p) {
  rk::gemm_body_splitk<ROCK_DT, true>(A, B, C, aux, res, p);
}

#if ROCK_DT != 7 && ROCK_DT != 8
RK_CONV_DL(_256x128_fast, 256, 128, 4, 2, 128)
RK_CONV_DL(_128x128_fast, 128, 128, 2, 2, 128)
RK_CONV_DL(_64x64_fast, 64, 64, 2, 2, 128)
RK_CONV(_64x64_generic, 64, 64, 2, 2, rk::LD_CONV_IN_GENERIC, rk::LD_CONV_FIL_GENERIC)
// input window resident in LDS: 224 output pixels x 128 channels per block
extern "C" __global__ __launch_bounds__(512) void RK_CAT(RK_CAT(rock_conv_, ROCK_DTNAME), _direct224)(
    const void *fil, const void *in, void *out, const void *aux, const void *res, RockConvParams p) {
  rk::conv_direct_body<ROCK_DT, 7, 2, false>(in, fil, out, aux, res, p);
}
extern "C" __global__ __launch_bounds__(512) void RK_CAT(RK_CAT(rock_conv_, ROCK_DTNAME), _direct224_e)(
    const void *fil, const void *in, void *out, const void *aux, const void *res, RockConvParams p) {
  rk::conv_direct_body<ROCK_DT, 7, 2, true>(in, fil, out, aux, res, p);
}
#endif
