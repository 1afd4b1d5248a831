// Matrix-core issue-rate probe: every wave runs a long chain of independent
// 32x32 MFMAs on register operands (no memory traffic), so the time per
// launch is the ceiling the matrix cores reach for that operand type.  With
// `random_data` the operands carry hashed bit patterns instead of constants:
// on MI355X that alone lowers the sustained clock (power), so the two numbers
// bracket what any kernel on real data can reach.
#include "mfma_gfx950.h"

namespace {
__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

template <int DT>
__device__ __forceinline__ void probe_body(float *out, int iters, int random_data) {
  const int gid = threadIdx.x + blockIdx.x * blockDim.x;
  unsigned r[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    r[i] = random_data ? probe_hash(gid * 8 + i + 1) : 0x01010101u;
    if (DT == MM_FP8)
      r[i] &= 0x3f3f3f3fu;               // finite, modest magnitudes
    if (DT == MM_F16 || DT == MM_BF16)
      r[i] = (r[i] & 0x3fff3fffu) | 0x20002000u;
    if (DT == MM_F32)
      r[i] = (r[i] & 0x007fffffu) | 0x3f000000u; // [0.5, 1)
  }
  Frag<DT> a[2], b[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int c = 0; c < MmaTraits<DT>::CHUNKS; ++c) {
      a[j].c[c] = v4i{(int)r[0] + j, (int)r[1], (int)r[2] + c, (int)r[3]};
      b[j].c[c] = v4i{(int)r[4], (int)r[5] + j, (int)r[6], (int)r[7] + c};
    }
  typename MmaTraits<DT>::Acc acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      acc[j][v] = 0;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      mma32x32<DT>(a[j & 1], b[j >> 1], acc[j]);
  }
  out[gid] = (float)(acc[0][0] + acc[1][0] + acc[2][0] + acc[3][0]);
}
} // namespace

#define RK_PROBE(NAME, DT)                                                                   \
  extern "C" __global__ __launch_bounds__(256) void rock_probe_mfma_##NAME(float *out, int iters, \
                                                                           int random_data) { \
    probe_body<DT>(out, iters, random_data);                                                 \
  }
// one code object per kernel: the build compiles this file once per operand
// type with -DROCK_KERNEL=<RockDType value> (the preprocessor does not see the enumerators)
#ifndef ROCK_KERNEL
#define ROCK_KERNEL -1
#endif
#define RK_SELECTED(n) (ROCK_KERNEL < 0 || ROCK_KERNEL == (n))
#if RK_SELECTED(0) // MM_F32
RK_PROBE(f32, MM_F32)
#endif
#if RK_SELECTED(1) // MM_F16
RK_PROBE(f16, MM_F16)
#endif
#if RK_SELECTED(2) // MM_BF16
RK_PROBE(bf16, MM_BF16)
#endif
#if RK_SELECTED(3) // MM_I8
RK_PROBE(i8, MM_I8)
#endif
#if RK_SELECTED(4) // MM_FP8
RK_PROBE(fp8, MM_FP8)
#endif
