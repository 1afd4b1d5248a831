// Host stand-in for the device environment of the contraction kernels
// (rocmlir_amd/csrc/gemm_conv_dlds.h and what it includes), used by
// tests/test_kernel_host_model.py.  Test infrastructure only.
//
// Every thread of a launch runs the kernel body to its end, one after the
// other.  The DATA a thread reads from LDS is therefore not what its
// neighbours would have put there and the matrix instructions do nothing, but
// every ADDRESS a thread forms is the one the GPU thread forms: addresses never
// depend on data in these kernels.  Buffer loads are checked against the
// registered tensors (the runner's hm_alloc) the way the hardware checks them
// against the descriptor's range; plain loads and stores run into canary and
// guard pages around the tensors, and a 16-byte access that is not 16-byte
// aligned traps, as x86 vector moves do.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#define __device__
#define __host__
#define __global__
#define __forceinline__ inline __attribute__((always_inline))
#define __shared__ static
#define __launch_bounds__(...)
#define amdgpu_waves_per_eu(...)
#define address_space(x)
using std::max;
using std::min;

struct HmDim {
  unsigned x, y, z;
};
extern HmDim threadIdx, blockIdx, blockDim, gridDim;

void hm_check_global(const void *p, size_t n, const char *what);

// buffer descriptor: base and range only (raw buffers, no stride, no swizzle)
struct HmRsrc {
  const char *base;
  unsigned num_records;
};
#define __amdgpu_buffer_rsrc_t HmRsrc
inline HmRsrc hm_make_rsrc(void *base, int, int num, int) { return HmRsrc{(const char *)base, (unsigned)num}; }
#define __builtin_amdgcn_make_buffer_rsrc hm_make_rsrc

// a lane whose offset lies at or beyond the range reads zeros and touches no memory
inline bool hm_in_range(const HmRsrc &r, int voff, int soff, int ioff, const char *&src) {
  const uint64_t off = (uint64_t)(unsigned)voff + (unsigned)ioff;
  if (off >= r.num_records || off + (unsigned)soff >= r.num_records)
    return false;
  src = r.base + off + (unsigned)soff;
  return true;
}
inline void hm_load_lds(HmRsrc r, void *lds, int size, int voff, int soff, int ioff, int) {
  char *dst = (char *)lds + (threadIdx.x & 63) * size; // the wave's lanes land back to back
  const char *src;
  if (!hm_in_range(r, voff, soff, ioff, src)) {
    std::memset(dst, 0, size);
    return;
  }
  hm_check_global(src, size, "buffer load into LDS");
  std::memcpy(dst, src, size);
}
#define __builtin_amdgcn_raw_ptr_buffer_load_lds hm_load_lds
typedef int hm_v4i __attribute__((ext_vector_type(4)));
inline hm_v4i hm_load_b128(HmRsrc r, int voff, int soff, int) {
  hm_v4i v = {0, 0, 0, 0};
  const char *src;
  if (!hm_in_range(r, voff, soff, 0, src))
    return v;
  hm_check_global(src, 16, "buffer load");
  std::memcpy(&v, src, 16);
  return v;
}
#define __builtin_amdgcn_raw_buffer_load_b128 hm_load_b128

// synchronisation and scheduling: nothing to do for one thread at a time
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_s_barrier() ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __syncthreads() ((void)0)
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_ballot_w64(x) ((x) ? ~0ull : 0ull)
#define __builtin_amdgcn_ds_bpermute(a, v) (v)

// arithmetic that addresses do not depend on
template <typename A, typename B, typename C> inline C hm_mfma(A, B, C c, int, int, int) { return c; }
#define __builtin_amdgcn_mfma_i32_32x32x32_i8 hm_mfma
#define __builtin_amdgcn_mfma_f32_32x32x16_f16 hm_mfma
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16 hm_mfma
#define __builtin_amdgcn_mfma_f32_32x32x2f32 hm_mfma
template <typename A, typename B, typename C> inline C hm_mfma_scale(A, B, C c, int, int, int, int, int, int) {
  return c;
}
#define __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4 hm_mfma_scale
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, c, d) (0)
#define __builtin_amdgcn_cvt_pk_bf8_f32(a, b, c, d) (0)
#define __builtin_amdgcn_cvt_f32_fp8(a, b) (0.0f)
#define __builtin_amdgcn_cvt_f32_bf8(a, b) (0.0f)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
inline float __frcp_rn(float x) { return 1.0f / x; }
inline float __expf(float x) { return expf(x); }

// transposing LDS reads: eight bytes from the lane's address
typedef short hm_v4s __attribute__((ext_vector_type(4)));
typedef int hm_v2i __attribute__((ext_vector_type(2)));
inline hm_v4s hm_read_tr16(const void *p) {
  hm_v4s v;
  std::memcpy(&v, p, 8);
  return v;
}
inline hm_v2i hm_read_tr8(const void *p) {
  hm_v2i v;
  std::memcpy(&v, p, 8);
  return v;
}
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) hm_read_tr16((const void *)(p))
#define __builtin_amdgcn_ds_read_tr8_b64_v2i32(p) hm_read_tr8((const void *)(p))
