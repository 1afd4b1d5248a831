// Layout conversion kernels (1-, 2- and 4-byte elements): see
// RockRelayoutParams in kernel_params.h.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "kernel_params.h"

namespace {

// One block moves a 32 x 32 tile over (dst_fast, src_fast); blockIdx.x
// enumerates tiles, fastest over the src_fast tiles, then dst_fast tiles, then
// the remaining three dimensions in index order.
template <typename T>
__device__ __forceinline__ void relayout_body(const T *src, T *dst, const RockRelayoutParams &p) {
  __shared__ T tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8
  const int sf = p.src_fast, df = p.dst_fast;
  const bool transposed = sf != df;
  const int size_s = p.size[sf], size_d = p.size[df];
  unsigned b = blockIdx.x;
  // tile origin along the two fast dimensions (a plain strided copy takes
  // 1024 consecutive elements of the common fast dimension per block)
  const unsigned ts = transposed ? (size_s + 31) / 32 : (size_s + 1023) / 1024;
  const int org_s = (int)(b % ts) * (transposed ? 32 : 1024);
  b /= ts;
  int org_d = 0;
  if (transposed) {
    const unsigned td = (size_d + 31) / 32;
    org_d = (int)(b % td) * 32;
    b /= td;
  }
  int64_t so = 0, dof = 0;
#pragma unroll
  for (int d = 4; d >= 0; --d) {
    int i;
    if (d == sf) {
      i = org_s;
    } else if (d == df) {
      i = org_d;
    } else {
      i = (int)(b % (unsigned)p.size[d]);
      b /= (unsigned)p.size[d];
    }
    so += (int64_t)i * p.src_stride[d];
    dof += (int64_t)i * p.dst_stride[d];
  }
  const int64_t ss_s = p.src_stride[sf], ss_d = p.src_stride[df];
  const int64_t ds_s = p.dst_stride[sf], ds_d = p.dst_stride[df];
  if (!transposed) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = j * 256 + threadIdx.x;
      if (org_s + e < size_s)
        dst[dof + (int64_t)e * ds_s] = src[so + (int64_t)e * ss_s];
    }
    return;
  }
  // read: tx walks the source's contiguous dimension
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = ty + 8 * j; // position along dst_fast
    if (org_d + r < size_d && org_s + tx < size_s)
      tile[r][tx] = src[so + (int64_t)r * ss_d + (int64_t)tx * ss_s];
  }
  __syncthreads();
  // write: tx walks the destination's contiguous dimension
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = ty + 8 * j; // position along src_fast
    if (org_s + c < size_s && org_d + tx < size_d)
      dst[dof + (int64_t)c * ds_s + (int64_t)tx * ds_d] = tile[tx][c];
  }
}

} // namespace

extern "C" __global__ __launch_bounds__(256) void rock_relayout_b1(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint8_t>((const uint8_t *)src, (uint8_t *)dst, p);
}
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b2(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint16_t>((const uint16_t *)src, (uint16_t *)dst, p);
}
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b4(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint32_t>((const uint32_t *)src, (uint32_t *)dst, p);
}
