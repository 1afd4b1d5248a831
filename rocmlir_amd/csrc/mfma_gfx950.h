// gfx950 (CDNA4) matrix-core wrappers: one 32x32 output block per call, a
// 16-byte K-chunk (two for the 8-bit floats) per lane and operand.
//
// Lane mapping shared by every 32x32xK MFMA used here (64 lanes, l = lane id):
//   first operand  ("rows"):  row  = l % 32, K slice = l / 32
//   second operand ("cols"):  col  = l % 32, K slice = l / 32
//   result (16 values/lane):  col  = l % 32,
//                             row  = 8*(v/4) + 4*(l/32) + v%4   for value v
// A K slice is whatever 16 bytes (32 for the 8-bit floats) the lane holds; the
// dot product only needs both operands to use the same slicing, so each lane
// simply reads the same 16-byte chunk index from both LDS tiles.
//
// Measured on MI355X, the 32x32 shapes run at the matrix cores' full rate
// (i8 4.6 POP/s, f8 5.0 PFLOP/s, f16 2.5 PFLOP/s, f32 155 TFLOP/s issue-only)
// while the 16x16 shapes of int8 and f16 reach only 55-58 % of it, so
// everything here is built from 32x32 blocks.  The reference selects among the
// gfx908-gfx942 instructions (mlir/lib/Dialect/Rock/IR/MfmaInsnGroup.cpp:
// 324-408); these are the double-K gfx950 forms it does not know.
#pragma once
#include <hip/hip_runtime.h>
#include "kernel_params.h"

// Where lanes of a wave hand data to each other through LDS with no instruction between the store and the load
// (a wave's LDS operations complete in order).  Nothing on the GPU; the CPU build of the kernels that the tests
// step through runs the lanes one after the other and makes them meet at these points.
#ifndef RK_WAVE_LDS_ORDER
#define RK_WAVE_LDS_ORDER() ((void)0)
#endif

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));

// Internal operand-type codes: the public RockDType values plus the two mixed
// 8-bit float pairs (A type, B type).
enum : int {
  MM_F32 = ROCK_F32,
  MM_F16 = ROCK_F16,
  MM_BF16 = ROCK_BF16,
  MM_I8 = ROCK_I8,
  MM_FP8 = ROCK_FP8,
  MM_BF8 = ROCK_BF8,
  MM_FP8_BF8 = 7, // A e4m3fn, B e5m2
  MM_BF8_FP8 = 8  // A e5m2, B e4m3fn
};

template <int DT> struct MmaTraits;

// K bytes consumed per lane and step is 16, except for the 8-bit floats whose
// 32x32x64 instruction wants 32 bytes per lane (two chunks).
template <> struct MmaTraits<MM_I8> {
  static constexpr int ES = 1;        // element size in bytes
  static constexpr int CHUNKS = 1;    // 16-byte chunks per lane per MFMA step
  static constexpr bool INT_ACC = true;
  using Acc = v16i;
};
template <> struct MmaTraits<MM_F16> {
  static constexpr int ES = 2;
  static constexpr int CHUNKS = 1;
  static constexpr bool INT_ACC = false;
  using Acc = v16f;
};
template <> struct MmaTraits<MM_BF16> : MmaTraits<MM_F16> {};
template <> struct MmaTraits<MM_F32> {
  static constexpr int ES = 4;
  static constexpr int CHUNKS = 1;
  static constexpr bool INT_ACC = false;
  using Acc = v16f;
};
template <> struct MmaTraits<MM_FP8> {
  static constexpr int ES = 1;
  static constexpr int CHUNKS = 2;
  static constexpr bool INT_ACC = false;
  using Acc = v16f;
};
template <> struct MmaTraits<MM_BF8> : MmaTraits<MM_FP8> {};
template <> struct MmaTraits<MM_FP8_BF8> : MmaTraits<MM_FP8> {};
template <> struct MmaTraits<MM_BF8_FP8> : MmaTraits<MM_FP8> {};

// One operand fragment: CHUNKS 16-byte chunks.
template <int DT> struct Frag {
  v4i c[MmaTraits<DT>::CHUNKS];
};

// acc += rows x cols over the K slice held in the fragments.
// `rows` feeds the MFMA's first matrix, `cols` its second.  The kernels feed
// the problem's B-matrix rows as MFMA rows and its A-matrix rows as columns.
template <int DT>
__device__ __forceinline__ void mma32x32(const Frag<DT> &rows, const Frag<DT> &cols,
                                         typename MmaTraits<DT>::Acc &acc) {
  if constexpr (DT == MM_I8) {
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(rows.c[0], cols.c[0], acc, 0, 0, 0);
  } else if constexpr (DT == MM_F16) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(v8h, rows.c[0]), __builtin_bit_cast(v8h, cols.c[0]), acc, 0, 0, 0);
  } else if constexpr (DT == MM_BF16) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(v8bf, rows.c[0]), __builtin_bit_cast(v8bf, cols.c[0]), acc, 0, 0, 0);
  } else if constexpr (DT == MM_F32) {
    v4f r = __builtin_bit_cast(v4f, rows.c[0]);
    v4f c = __builtin_bit_cast(v4f, cols.c[0]);
#pragma unroll
    for (int t = 0; t < 4; ++t)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(r[t], c[t], acc, 0, 0, 0);
  } else {
    // 8-bit floats: format codes 0 = e4m3, 1 = e5m2.
    constexpr int fmtA = (DT == MM_BF8 || DT == MM_BF8_FP8) ? 1 : 0;
    constexpr int fmtB = (DT == MM_BF8 || DT == MM_FP8_BF8) ? 1 : 0;
    v8i r = {rows.c[0][0], rows.c[0][1], rows.c[0][2], rows.c[0][3],
             rows.c[1][0], rows.c[1][1], rows.c[1][2], rows.c[1][3]};
    v8i c = {cols.c[0][0], cols.c[0][1], cols.c[0][2], cols.c[0][3],
             cols.c[1][0], cols.c[1][1], cols.c[1][2], cols.c[1][3]};
    // block scales of 2^0 (E8M0 code 127) on both operands
    acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
        r, c, acc, fmtB, fmtA, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
  }
}

// ---- output conversions (round to nearest even; fp8 saturates) -------------
__device__ __forceinline__ float clamp_fp8_range(float v, float lim) {
  // NaN passes through; +-inf and finite overflow clamp to the largest finite
  return v != v ? v : fminf(fmaxf(v, -lim), lim);
}

__device__ __forceinline__ uint8_t f32_to_e4m3fn_sat(float v) {
  v = clamp_fp8_range(v, 448.0f);
  int packed = __builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0, false);
  return (uint8_t)(packed & 0xff);
}
__device__ __forceinline__ uint8_t f32_to_e5m2_sat(float v) {
  v = clamp_fp8_range(v, 57344.0f);
  int packed = __builtin_amdgcn_cvt_pk_bf8_f32(v, v, 0, false);
  return (uint8_t)(packed & 0xff);
}
__device__ __forceinline__ float e4m3fn_to_f32(uint8_t v) {
  return __builtin_amdgcn_cvt_f32_fp8((int)v, 0);
}
__device__ __forceinline__ float e5m2_to_f32(uint8_t v) {
  return __builtin_amdgcn_cvt_f32_bf8((int)v, 0);
}
__device__ __forceinline__ int8_t f32_to_i8_sat(float v) {
  float r = __builtin_rintf(v); // ties to even
  r = fminf(fmaxf(r, -128.0f), 127.0f);
  return (int8_t)(int)r;
}
