// Utility kernels: layout conversion (1-, 2- and 4-byte elements), zero fill
// and the reduction of K-split partial sums: see RockRelayoutParams,
// RockFillParams and RockReduceParams in kernel_params.h.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "kernel_params.h"

// Every kernel goes into a code object of its own: the build compiles this
// file once per kernel with -DROCK_KERNEL=<n>, n counting the kernels below
// from 0 in file order (rocmlir_amd/_build.py holds the matching list of
// names and checks each object's symbol against it).
#ifndef ROCK_KERNEL
#define ROCK_KERNEL -1
#endif
#define RK_SELECTED(n) (ROCK_KERNEL < 0 || ROCK_KERNEL == (n))

namespace {

// RELAYOUT_TRANSPOSE: one block moves a tile of tile_d x (1024 / tile_d)
// elements over (dst_fast, src_fast) through LDS, so that the source is read
// along its contiguous dimension and the destination written along its own;
// tile_d is 32, or 16 or 8 when the destination's contiguous dimension is that
// short (a padded 3-channel image).  blockIdx.x enumerates tiles, fastest over
// the src_fast tiles, then dst_fast tiles, then the remaining three
// dimensions in index order.
template <typename T>
__device__ __forceinline__ void relayout_transpose(const T *src, T *dst, const RockRelayoutParams &p, unsigned block) {
  __shared__ T tile[1024 + 128];
  const int sf = p.src_fast, df = p.dst_fast;
  const int td = p.tile_d, ts = 1024 / td; // both powers of two
  const int td_shift = __builtin_ctz(td), ts_shift = 10 - td_shift;
  const int size_s = p.size[sf], size_d = p.size[df];
  const int src_s = p.src_size[sf], src_d = p.src_size[df]; // shorter than the destination when padding
  unsigned b = block;
  const unsigned tiles_s = (size_s + ts - 1) >> ts_shift, tiles_d = (size_d + td - 1) >> td_shift;
  const int org_s = (int)(b % tiles_s) << ts_shift;
  b /= tiles_s;
  const int org_d = (int)(b % tiles_d) << td_shift;
  b /= tiles_d;
  int64_t so = 0, dof = 0;
  bool outer_in = true; // the block's position in the other three dimensions lies inside the source
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
      outer_in = outer_in && i < p.src_size[d];
    }
    so += (int64_t)i * p.src_stride[d];
    dof += (int64_t)i * p.dst_stride[d];
  }
  const int64_t ss_s = p.src_stride[sf], ss_d = p.src_stride[df];
  const int64_t ds_s = p.dst_stride[sf], ds_d = p.dst_stride[df];
  // read: consecutive threads walk the source's contiguous dimension
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int idx = j * 256 + (int)threadIdx.x;
    const int r = idx >> ts_shift, cs = idx & (ts - 1); // along dst_fast, along src_fast
    if (org_d + r < size_d && org_s + cs < size_s)
      tile[r * (ts + 1) + cs] =
          (outer_in && org_d + r < src_d && org_s + cs < src_s) ? src[so + (int64_t)r * ss_d + (int64_t)cs * ss_s] : (T)0;
  }
  __syncthreads();
  // write: consecutive threads walk the destination's contiguous dimension
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int idx = j * 256 + (int)threadIdx.x;
    const int cs = idx >> td_shift, r = idx & (td - 1);
    if (org_s + cs < size_s && org_d + r < size_d)
      dst[dof + (int64_t)cs * ds_s + (int64_t)r * ds_d] = tile[r * (ts + 1) + cs];
  }
}

// RELAYOUT_TRANSPOSE_VEC: the same transposition in tiles of 128 bytes x 128
// bytes' worth of elements (64 x 64 of 16-bit), moved with 16-byte accesses on
// both sides wherever a lane's run is whole, in range and 16-byte aligned, and
// element by element elsewhere.  Requires unit stride of src_fast in the source
// and of dst_fast in the destination.
template <typename T>
__device__ __forceinline__ void relayout_transpose_vec(const T *src, T *dst, const RockRelayoutParams &p, unsigned block) {
  constexpr int V = 16 / (int)sizeof(T); // elements per 16-byte vector
  constexpr int TILE = 8 * V;            // tile side in elements
  constexpr int PITCH = TILE + V;        // keeps LDS rows 16-byte aligned
  __shared__ __attribute__((aligned(16))) T tile[TILE * PITCH];
  const int sf = p.src_fast, df = p.dst_fast;
  const int size_s = p.size[sf], size_d = p.size[df];
  const int src_s = p.src_size[sf], src_d = p.src_size[df];
  unsigned b = block;
  const unsigned tiles_s = (size_s + TILE - 1) / TILE, tiles_d = (size_d + TILE - 1) / TILE;
  const int org_s = (int)(b % tiles_s) * TILE;
  b /= tiles_s;
  const int org_d = (int)(b % tiles_d) * TILE;
  b /= tiles_d;
  int64_t so = 0, dof = 0;
  bool outer_in = true; // the block's position in the other three dimensions lies inside the source
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
      outer_in = outer_in && i < p.src_size[d];
    }
    so += (int64_t)i * p.src_stride[d];
    dof += (int64_t)i * p.dst_stride[d];
  }
  const int64_t ss_d = p.src_stride[df], ds_s = p.dst_stride[sf];
  union Vec {
    T e[V];
    uint4 v;
  };
  // read: eight lanes cover one source row of the tile
#pragma unroll
  for (int j = 0; j < TILE * 8 / 256; ++j) {
    const int vi = j * 256 + (int)threadIdx.x;
    const int r = vi >> 3, cs0 = (vi & 7) * V; // along dst_fast, along src_fast
    if (org_d + r >= size_d || org_s + cs0 >= size_s)
      continue;
    const T *g = src + so + (int64_t)r * ss_d + cs0;
    Vec u;
    if (outer_in && org_d + r < src_d && org_s + cs0 + V <= src_s && ((uintptr_t)g & 15) == 0) {
      u.v = *(const uint4 *)g;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        u.e[e] = (outer_in && org_d + r < src_d && org_s + cs0 + e < src_s) ? g[e] : (T)0;
    }
    *(uint4 *)&tile[r * PITCH + cs0] = u.v;
  }
  __syncthreads();
  // write: eight lanes cover one destination row of the tile
#pragma unroll
  for (int j = 0; j < TILE * 8 / 256; ++j) {
    const int vi = j * 256 + (int)threadIdx.x;
    const int cs = vi >> 3, d0 = (vi & 7) * V;
    if (org_s + cs >= size_s || org_d + d0 >= size_d)
      continue;
    Vec u;
#pragma unroll
    for (int e = 0; e < V; ++e)
      u.e[e] = tile[(d0 + e) * PITCH + cs];
    T *g = dst + dof + (int64_t)cs * ds_s + d0;
    if (org_d + d0 + V <= size_d && ((uintptr_t)g & 15) == 0) {
      *(uint4 *)g = u.v;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (org_d + d0 + e < size_d)
          g[e] = u.e[e];
    }
  }
}

// RELAYOUT_COPY: source and destination share their contiguous dimension
// (index 4) but not its length or the other strides.  The destination's runs
// along it are whole 16-byte chunks; a thread builds one chunk, reading zero
// beyond the source's extent.  blockIdx.x enumerates groups of 256 chunks over
// the flattened dimensions (2, 3, chunk), then dimensions 1 and 0.
template <typename T>
__device__ __forceinline__ void relayout_copy(const T *src, T *dst, const RockRelayoutParams &p, unsigned block) {
  constexpr int EPC = 16 / (int)sizeof(T); // elements per chunk
  const unsigned chunks4 = (unsigned)p.size[4] / EPC;
  const unsigned inner = (unsigned)p.size[2] * (unsigned)p.size[3] * chunks4;
  const unsigned per = (inner + 255) / 256;
  unsigned b = block;
  unsigned q = (b % per) * 256 + threadIdx.x;
  b /= per;
  const unsigned i1 = b % (unsigned)p.size[1], i0 = b / (unsigned)p.size[1];
  if (q >= inner)
    return;
  const unsigned ch = q % chunks4;
  q /= chunks4;
  const unsigned i3 = q % (unsigned)p.size[3], i2 = q / (unsigned)p.size[3];
  const int64_t so = (int64_t)i0 * p.src_stride[0] + (int64_t)i1 * p.src_stride[1] +
                     (int64_t)i2 * p.src_stride[2] + (int64_t)i3 * p.src_stride[3];
  const int64_t dof = (int64_t)i0 * p.dst_stride[0] + (int64_t)i1 * p.dst_stride[1] +
                      (int64_t)i2 * p.dst_stride[2] + (int64_t)i3 * p.dst_stride[3] + (int64_t)ch * EPC;
  // zero beyond the source's extent in EVERY dimension (a filter padded with whole rows as well as channels)
  const bool outer_in = i0 < (unsigned)p.src_size[0] && i1 < (unsigned)p.src_size[1] && i2 < (unsigned)p.src_size[2] &&
                        i3 < (unsigned)p.src_size[3];
  const int e0 = (int)ch * EPC, lim = outer_in ? p.src_size[4] : 0;
  const int64_t ss = p.src_stride[4];
  union {
    T e[EPC];
    uint4 v;
  } u;
#pragma unroll
  for (int j = 0; j < EPC; ++j)
    u.e[j] = e0 + j < lim ? src[so + (int64_t)(e0 + j) * ss] : (T)0;
  *(uint4 *)(dst + dof) = u.v;
}

template <typename T>
__device__ __forceinline__ void relayout_body(const T *src, T *dst, const RockRelayoutParams &p,
                                              unsigned block = blockIdx.x) {
  if (p.mode == RELAYOUT_COPY)
    relayout_copy<T>(src, dst, p, block);
  else if (p.mode == RELAYOUT_TRANSPOSE_VEC)
    relayout_transpose_vec<T>(src, dst, p, block);
  else
    relayout_transpose<T>(src, dst, p, block);
}

// Two conversions in one launch (both operands of a GEMM copied into padded
// rows): blocks [0, first_blocks) convert the first tensor, the rest the second.
template <typename T>
__device__ __forceinline__ void relayout_pair_body(const void *src0, void *dst0, const void *src1, void *dst1,
                                                   const RockRelayoutPairParams &p) {
  if (blockIdx.x < (unsigned)p.first_blocks) // uniform per block
    relayout_body<T>((const T *)src0, (T *)dst0, p.first, blockIdx.x);
  else
    relayout_body<T>((const T *)src1, (T *)dst1, p.second, blockIdx.x - (unsigned)p.first_blocks);
}

} // namespace

#if RK_SELECTED(0)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b1(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint8_t>((const uint8_t *)src, (uint8_t *)dst, p);
}
#endif
#if RK_SELECTED(1)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b2(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint16_t>((const uint16_t *)src, (uint16_t *)dst, p);
}
#endif
#if RK_SELECTED(2)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b4(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint32_t>((const uint32_t *)src, (uint32_t *)dst, p);
}
#endif

// 16 bytes per thread; the tail of a size that is not a multiple of 16 byte by byte
#if RK_SELECTED(3)
extern "C" __global__ __launch_bounds__(256) void rock_fill_zero(void *dst, RockFillParams p) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 16;
  if (i + 16 <= p.bytes) {
    *(uint4 *)((char *)dst + i) = uint4{0, 0, 0, 0};
  } else {
    for (int64_t b = i; b < p.bytes; ++b)
      ((char *)dst)[b] = 0;
  }
}
#endif

// one output element per thread
#if RK_SELECTED(4)
extern "C" __global__ __launch_bounds__(256) void rock_reduce_splits(const float *partials, void *dst,
                                                                     RockReduceParams p) {
  const int64_t total = (int64_t)p.size[0] * p.size[1] * p.size[2] * p.size[3];
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total)
    return;
  float acc = 0.0f;
  for (int s = 0; s < p.splits; ++s)
    acc = acc + partials[(int64_t)s * p.split_stride + i];
  int64_t rem = i, off = 0;
#pragma unroll
  for (int d = 3; d >= 0; --d) {
    off += (rem % p.size[d]) * p.dst_stride[d];
    rem /= p.size[d];
  }
  if (p.out_dtype == ROCK_F32) {
    ((float *)dst)[off] = acc;
  } else if (p.out_dtype == ROCK_F16) {
    ((_Float16 *)dst)[off] = (_Float16)acc;
  } else {
    ((__bf16 *)dst)[off] = (__bf16)acc;
  }
}
#endif

namespace {
__device__ __forceinline__ float load_as_f32(const void *base, int64_t idx, int dtype) {
  if (dtype == ROCK_F32)
    return ((const float *)base)[idx];
  if (dtype == ROCK_F16)
    return (float)((const _Float16 *)base)[idx];
  return __builtin_bit_cast(float, (uint32_t)((const uint16_t *)base)[idx] << 16);
}

__device__ __forceinline__ float block_reduce(float v, bool take_max, float *scratch) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, 64);
    v = take_max ? fmaxf(v, o) : v + o;
  }
  __syncthreads(); // scratch may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0)
    scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int w = 1; w < 4; ++w)
    r = take_max ? fmaxf(r, scratch[w]) : r + scratch[w];
  return r;
}
} // namespace

// One block per row, three passes over it (maximum, sum, normalise); the last
// pass loads a chunk of scores into registers before any thread overwrites the
// narrower results over them.
#if RK_SELECTED(5)
extern "C" __global__ __launch_bounds__(256) void rock_softmax_rows(float *S, const void *scale_t, const void *bias,
                                                                    RockSoftmaxParams p) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const int g = (int)(row / p.seq_q), i = (int)(row - (int64_t)g * p.seq_q);
  float *s = S + row * p.row_pitch;
  const int64_t t_off = (int64_t)g * p.t_gs + (int64_t)i * p.t_is;
  auto score = [&](int j) {
    float x = s[j];
    if (p.has_scale_tensor)
      x = x * load_as_f32(scale_t, t_off + (int64_t)j * p.t_js, p.dtype);
    x = x * p.scale;
    if (p.has_bias)
      x = x + load_as_f32(bias, t_off + (int64_t)j * p.t_js, p.dtype);
    return x;
  };
  float m = -INFINITY;
  for (int j = threadIdx.x; j < p.seq_k; j += 256)
    m = fmaxf(m, score(j));
  m = block_reduce(m, true, scratch);
  float l = 0.0f;
  for (int j = threadIdx.x; j < p.seq_k; j += 256)
    l = l + expf(score(j) - m);
  l = block_reduce(l, false, scratch);
  const float inv = 1.0f / l;
  for (int j0 = 0; j0 < p.seq_k; j0 += 256) {
    const int j = j0 + (int)threadIdx.x;
    float e = 0.0f;
    if (j < p.seq_k)
      e = expf(score(j) - m) * inv;
    __syncthreads(); // every score of this chunk is in a register
    if (j < p.seq_k) {
      if (p.dtype == ROCK_F32)
        s[j] = e;
      else if (p.dtype == ROCK_F16)
        ((_Float16 *)s)[j] = (_Float16)e;
      else
        ((__bf16 *)s)[j] = (__bf16)e;
    }
  }
}
#endif
#if RK_SELECTED(6)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_pair_b1(const void *src0, void *dst0, const void *src1,
                                                                         void *dst1, RockRelayoutPairParams p) {
  relayout_pair_body<uint8_t>(src0, dst0, src1, dst1, p);
}
#endif
#if RK_SELECTED(7)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_pair_b2(const void *src0, void *dst0, const void *src1,
                                                                         void *dst1, RockRelayoutPairParams p) {
  relayout_pair_body<uint16_t>(src0, dst0, src1, dst1, p);
}
#endif
#if RK_SELECTED(8)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_pair_b4(const void *src0, void *dst0, const void *src1,
                                                                         void *dst1, RockRelayoutPairParams p) {
  relayout_pair_body<uint32_t>(src0, dst0, src1, dst1, p);
}
#endif

// one input element per thread, channels fastest
#if RK_SELECTED(9)
extern "C" __global__ __launch_bounds__(256) void rock_fold_depth(const void *T, void *dst, RockFoldDepthParams p) {
  const int64_t total = (int64_t)p.n * p.di * p.hi * p.wi * p.g * p.c;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total)
    return;
  int64_t rem = i;
  const int c = (int)(rem % p.c); rem /= p.c;
  const int g = (int)(rem % p.g); rem /= p.g;
  const int w = (int)(rem % p.wi); rem /= p.wi;
  const int h = (int)(rem % p.hi); rem /= p.hi;
  const int d = (int)(rem % p.di);
  const int64_t n = rem / p.di;
  float acc = 0.0f;
  for (int z = 0; z < p.z; ++z) {
    const int num = d + p.pad_d - z * p.dil_d;
    if (num < 0)
      break;
    if (num % p.stride_d != 0)
      continue;
    const int od = num / p.stride_d;
    if (od >= p.d_out)
      continue;
    const int64_t pix = ((n * p.d_out + od) * p.hi + h) * p.wi + w;
    acc = acc + load_as_f32(T, pix * p.t_pix + ((int64_t)g * p.z + z) * p.cp + c, p.dtype);
  }
  const int64_t off = n * p.dst_stride[0] + g * p.dst_stride[1] + c * p.dst_stride[2] + h * p.dst_stride[3] +
                      w * p.dst_stride[4] + d * p.dst_stride[5];
  if (p.dtype == ROCK_F32) {
    ((float *)dst)[off] = acc;
  } else if (p.dtype == ROCK_F16) {
    ((_Float16 *)dst)[off] = (_Float16)acc;
  } else {
    ((__bf16 *)dst)[off] = (__bf16)acc;
  }
}
#endif
