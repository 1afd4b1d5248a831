// Utility kernels: layout conversion (1-, 2- and 4-byte elements), zero fill
// and the reduction of K-split partial sums: see RockRelayoutParams,
// RockFillParams and RockReduceParams in kernel_params.h.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "kernel_params.h"
#include "relayout_body.h"

// Every kernel goes into a code object of its own: the build compiles this
// file once per kernel with -DROCK_KERNEL=<n>, n counting the kernels below
// from 0 in file order (rocmlir_amd/_build.py holds the matching list of
// names and checks each object's symbol against it).
#ifndef ROCK_KERNEL
#define ROCK_KERNEL -1
#endif
#define RK_SELECTED(n) (ROCK_KERNEL < 0 || ROCK_KERNEL == (n))

namespace {

// One conversion by the calling block: rock_relayout::relayout_phase
// (relayout_body.h) before and after the block's barrier.  nblocks is the
// number of blocks of this conversion, block this block's index among them.
template <typename T>
__device__ __forceinline__ void relayout_body(const T *src, T *dst, const RockRelayoutParams &p, unsigned block,
                                              unsigned nblocks) {
  __shared__ __attribute__((aligned(16))) T lds[rock_relayout::lds_elems<T>()];
  rock_relayout::relayout_phase<T>(0, src, dst, p, block, nblocks, (int)threadIdx.x, lds);
  __syncthreads();
  rock_relayout::relayout_phase<T>(1, src, dst, p, block, nblocks, (int)threadIdx.x, lds);
}

// Two conversions in one launch (both operands of a GEMM copied into padded
// rows): blocks [0, first_blocks) convert the first tensor, the rest the second.
template <typename T>
__device__ __forceinline__ void relayout_pair_body(const void *src0, void *dst0, const void *src1, void *dst1,
                                                   const RockRelayoutPairParams &p) {
  const bool first = blockIdx.x < (unsigned)p.first_blocks; // uniform per block
  relayout_body<T>((const T *)(first ? src0 : src1), (T *)(first ? dst0 : dst1), first ? p.first : p.second,
                   first ? blockIdx.x : blockIdx.x - (unsigned)p.first_blocks,
                   first ? (unsigned)p.first_blocks : gridDim.x - (unsigned)p.first_blocks);
}

} // namespace

#if RK_SELECTED(0)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b1(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint8_t>((const uint8_t *)src, (uint8_t *)dst, p, blockIdx.x, gridDim.x);
}
#endif
#if RK_SELECTED(1)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b2(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint16_t>((const uint16_t *)src, (uint16_t *)dst, p, blockIdx.x, gridDim.x);
}
#endif
#if RK_SELECTED(2)
extern "C" __global__ __launch_bounds__(256) void rock_relayout_b4(const void *src, void *dst,
                                                                    RockRelayoutParams p) {
  relayout_body<uint32_t>((const uint32_t *)src, (uint32_t *)dst, p, blockIdx.x, gridDim.x);
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
  int64_t rem = i, off = 0;
  bool padding = false;
#pragma unroll
  for (int d = 3; d >= 0; --d) {
    const int64_t at = rem % p.size[d];
    padding = padding || (p.valid[d] != 0 && at >= p.valid[d]);
    off += at * p.dst_stride[d];
    rem /= p.size[d];
  }
  if (padding)
    return;
  if (p.int_partials) { // integer sums: exact in any order
    const int *ip = (const int *)partials;
    int acc = 0;
    for (int s = 0; s < p.splits; ++s)
      acc += ip[(int64_t)s * p.split_stride + i];
    ((int *)dst)[off] = acc;
    return;
  }
  // summed in split order; sixteen loads are in flight at a time, the additions stay sequential
  float acc = 0.0f;
  int s = 0;
  for (; s + 16 <= p.splits; s += 16) {
    float v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j)
      v[j] = partials[(int64_t)(s + j) * p.split_stride + i];
#pragma unroll
    for (int j = 0; j < 16; ++j)
      acc = acc + v[j];
  }
  for (; s < p.splits; ++s)
    acc = acc + partials[(int64_t)s * p.split_stride + i];
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
  if (dtype == ROCK_I8)
    return (float)((const int8_t *)base)[idx];
  return __builtin_bit_cast(float, (uint32_t)((const uint16_t *)base)[idx] << 16);
}

// The pre-softmax program of a score: postfix code over a stack of four floats whose top is always s0 (pushes
// and pops shift the other three, so no stack slot is ever addressed with a run-time index).
__device__ __forceinline__ float run_attention_program(const RockSoftmaxParams &p, float x, int64_t at) {
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  for (int i = 0; i < p.prog_len; ++i) {
    const int op = p.prog[i] & 255, arg = p.prog[i] >> 8;
    if (op <= ROCK_AOP_CONST) {
      const float v = op == ROCK_AOP_SCORE    ? x
                      : op == ROCK_AOP_TENSOR ? load_as_f32(p.tensors[arg], p.t_base + at, p.tensor_dtype[arg])
                                              : p.consts[arg];
      s3 = s2; s2 = s1; s1 = s0; s0 = v;
    } else if (op < ROCK_AOP_EXP) {
      const float a = s1, b = s0;
      const float r = op == ROCK_AOP_ADD   ? a + b
                      : op == ROCK_AOP_SUB ? a - b
                      : op == ROCK_AOP_MUL ? a * b
                      : op == ROCK_AOP_DIV ? a / b
                      : op == ROCK_AOP_MAX ? fmaxf(a, b)
                                           : fminf(a, b);
      s0 = r; s1 = s2; s2 = s3;
    } else if (op < ROCK_AOP_WHERE) {
      const float a = s0;
      s0 = op == ROCK_AOP_EXP       ? expf(a)
           : op == ROCK_AOP_NEG     ? -a
           : op == ROCK_AOP_TANH    ? tanhf(a)
           : op == ROCK_AOP_SIGMOID ? 1.0f / (1.0f + expf(-a))
           : op == ROCK_AOP_RELU    ? fmaxf(a, 0.0f)
           : op == ROCK_AOP_ABS     ? fabsf(a)
                                    : erff(a);
    } else {
      s0 = s2 != 0.0f ? s1 : s0;
      s1 = s3;
    }
  }
  return s0;
}

// over the block's waves (at most 16); scratch holds one float per wave
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
  const int waves = (int)blockDim.x >> 6;
  float r = scratch[0];
  for (int w = 1; w < waves; ++w)
    r = take_max ? fmaxf(r, scratch[w]) : r + scratch[w];
  return r;
}
} // namespace

// One block per row: 256 threads, or 1024 for rows above 4096 scores (the
// host picks).  A row of up to 16 scores per thread is read once into
// registers (the pre-softmax tensors applied on the way), reduced twice and
// written once -- 4 bytes read and one result written per score; longer rows
// take three passes over memory (maximum, sum, normalise).  Either way every
// score of a stretch is in a register before any thread writes the narrower
// results over the row.
namespace {
struct SoftmaxRow {
  float *s;
  const void *scale_t, *bias, *mask, *other;
  int64_t t_off;
  const RockSoftmaxParams &p;
  __device__ __forceinline__ float score(int j) const {
    float x = s[j];
    if (p.prog_len)
      return run_attention_program(p, x, t_off + (int64_t)j * p.t_js);
    if (p.has_scale_tensor)
      x = x * load_as_f32(scale_t, t_off + (int64_t)j * p.t_js, p.dtype);
    x = x * p.scale;
    if (p.has_bias)
      x = x + load_as_f32(bias, t_off + (int64_t)j * p.t_js, p.dtype);
    if (p.has_mask && ((const int8_t *)mask)[t_off + (int64_t)j * p.t_js] == 0) // where(mask, x, other)
      x = load_as_f32(other, t_off + (int64_t)j * p.t_js, p.dtype);
    return x;
  }
  __device__ __forceinline__ void store(int j, float e) const {
    if (p.dtype == ROCK_F32)
      s[j] = e;
    else if (p.dtype == ROCK_F16)
      ((_Float16 *)s)[j] = (_Float16)e;
    else
      ((__bf16 *)s)[j] = (__bf16)e;
  }
};

__device__ __forceinline__ float widen(float x) { return x; }
__device__ __forceinline__ float widen(_Float16 x) { return (float)x; }
__device__ __forceinline__ float widen(__bf16 x) { return (float)x; }

// Rows of at most EPT * NT scores, NT threads; T is the type of P and of the
// pre-softmax tensors.  Loads are unconditional (columns beyond the row read its last
// score and are set to -inf afterwards) and each tensor has a loop of its
// own, so that a thread's loads are all in flight together.
template <int EPT, int NT, typename T>
__device__ __forceinline__ void softmax_row_in_registers(const SoftmaxRow &row, float *scratch) {
  const RockSoftmaxParams &p = row.p;
  const int n = p.seq_k, tid = (int)threadIdx.x;
  float v[EPT];
#pragma unroll
  for (int c = 0; c < EPT; ++c)
    v[c] = row.s[min(c * NT + tid, n - 1)];
  if (p.has_scale_tensor) {
    const T *t = (const T *)row.scale_t + row.t_off;
#pragma unroll
    for (int c = 0; c < EPT; ++c)
      v[c] = v[c] * widen(t[(int64_t)min(c * NT + tid, n - 1) * p.t_js]);
  }
#pragma unroll
  for (int c = 0; c < EPT; ++c)
    v[c] = v[c] * p.scale;
  if (p.has_bias) {
    const T *t = (const T *)row.bias + row.t_off;
#pragma unroll
    for (int c = 0; c < EPT; ++c)
      v[c] = v[c] + widen(t[(int64_t)min(c * NT + tid, n - 1) * p.t_js]);
  }
  if (p.has_mask) { // where(mask, x, other)
    const int8_t *mk = (const int8_t *)row.mask + row.t_off;
    const T *t = (const T *)row.other + row.t_off;
#pragma unroll
    for (int c = 0; c < EPT; ++c) {
      const int64_t at = (int64_t)min(c * NT + tid, n - 1) * p.t_js;
      const float o = widen(t[at]);
      v[c] = mk[at] == 0 ? o : v[c];
    }
  }
  float m = -INFINITY;
#pragma unroll
  for (int c = 0; c < EPT; ++c) {
    v[c] = c * NT + tid < n ? v[c] : -INFINITY;
    m = fmaxf(m, v[c]);
  }
  m = block_reduce(m, true, scratch);
  float l = 0.0f;
#pragma unroll
  for (int c = 0; c < EPT; ++c) {
    v[c] = expf(v[c] - m); // (columns beyond the row: exp(-inf) = 0)
    l = l + v[c];
  }
  l = block_reduce(l, false, scratch); // its barriers also separate the reads above from the stores below
  const float inv = 1.0f / l;
  T *out = (T *)row.s;
#pragma unroll
  for (int c = 0; c < EPT; ++c) {
    const int j = c * NT + tid;
    if (j < n)
      out[j] = (T)(v[c] * inv);
  }
}

template <typename T>
__device__ __forceinline__ bool softmax_short_row(const SoftmaxRow &row, float *scratch) {
  const int n = row.p.seq_k;
  if (blockDim.x == 1024) {
    if (n > 16 * 1024)
      return false;
    softmax_row_in_registers<16, 1024, T>(row, scratch);
  } else if (n <= 4 * 256) {
    softmax_row_in_registers<4, 256, T>(row, scratch);
  } else if (n <= 16 * 256) {
    softmax_row_in_registers<16, 256, T>(row, scratch);
  } else {
    return false;
  }
  return true;
}
} // namespace
#if RK_SELECTED(5)
extern "C" __global__ __launch_bounds__(1024) void rock_softmax_rows(float *S, const void *scale_t, const void *bias,
                                                                     const void *mask, const void *other,
                                                                     RockSoftmaxParams p) {
  __shared__ float scratch[16];
  const int64_t r = blockIdx.x;
  const int g = (int)(r / p.seq_q), i = (int)(r - (int64_t)g * p.seq_q);
  const SoftmaxRow row{S + r * p.row_pitch, scale_t, bias, mask, other, (int64_t)g * p.t_gs + (int64_t)i * p.t_is, p};
  // (a program runs on the three-pass path below: its loads and branches do not fit the register-resident form)
  const int nt = (int)blockDim.x, tid = (int)threadIdx.x;
  // (every path has read all scores of the row before its last stores, so the bytes behind P's last element,
  // which may be a score's, are free by now)
  auto zero_padding = [&]() {
    for (int j = p.seq_k + tid; j < p.seq_k_padded; j += nt)
      row.store(j, 0.0f);
  };
  if (p.prog_len == 0 && (p.dtype == ROCK_F32   ? softmax_short_row<float>(row, scratch)
                          : p.dtype == ROCK_F16 ? softmax_short_row<_Float16>(row, scratch)
                                                : softmax_short_row<__bf16>(row, scratch))) {
    zero_padding();
    return;
  }
  float m = -INFINITY;
  for (int j = tid; j < p.seq_k; j += nt)
    m = fmaxf(m, row.score(j));
  m = block_reduce(m, true, scratch);
  float l = 0.0f;
  for (int j = tid; j < p.seq_k; j += nt)
    l = l + expf(row.score(j) - m);
  l = block_reduce(l, false, scratch);
  const float inv = 1.0f / l;
  for (int j0 = 0; j0 < p.seq_k; j0 += nt) {
    const int j = j0 + tid;
    float e = 0.0f;
    if (j < p.seq_k)
      e = expf(row.score(j) - m) * inv;
    __syncthreads(); // every score of this stretch is in a register
    if (j < p.seq_k)
      row.store(j, e);
  }
  zero_padding();
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
