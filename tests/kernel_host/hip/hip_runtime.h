// Host stand-in for the device environment of the kernels in rocmlir_amd/csrc,
// used by tests/test_kernel_host_model.py.  Test infrastructure only.
//
// A block runs as one cooperative fiber per thread (runner.cpp).  A thread runs
// until it reaches an operation that involves other threads -- a workgroup
// barrier, a matrix instruction, a cross-lane read -- and waits there until the
// other lanes of its wave (or threads of its block) have arrived, so that such
// operations see every lane's operands and LDS holds what the GPU's LDS holds
// at that point.  Lanes of a wave that hand data to each other through LDS
// with no instruction between them to meet at (the GPU orders a wave's LDS
// operations by itself) meet at RK_WAVE_LDS_ORDER(), which the kernels' sources
// place there and which is empty on the GPU.
//
// A load into LDS lands either when it is issued or, with hm_set_late_loads(1), not before the wait that covers
// it (vmcnt): the two extremes of what the hardware may do.  A kernel that reads a stage too early fails under the
// second, one that refills a stage too early under the first.
//
// Buffer loads are checked against the registered tensors (the runner's
// hm_alloc) the way the hardware checks them against the descriptor's range;
// plain loads and stores run into canary and guard pages around the tensors,
// and a 16-byte access that is not 16-byte aligned traps, as x86 vector moves
// do.  The matrix instructions multiply in double precision and add to the
// accumulator once per instruction: exact, like the hardware's, on the
// integer-valued data the tests use.
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
struct alignas(16) uint4 {
  unsigned x, y, z, w;
};
extern HmDim threadIdx, blockIdx, blockDim, gridDim;

// ---- runner.cpp ----------------------------------------------------------------
void hm_check_global(const void *p, size_t n, const char *what);
void hm_wave_sync();  // returns when every live lane of the wave has called it
void hm_block_sync(); // returns when every live thread of the block has called it

#define RK_WAVE_LDS_ORDER() hm_wave_sync()
#define __builtin_amdgcn_s_barrier() hm_block_sync()
#define __syncthreads() hm_block_sync()
// A wait for loads: the lane's loads into LDS beyond the count the instruction allows to stay in flight land (see
// hm_set_late_loads in runner.cpp), then the wave meets, so that behind a wait every lane's loads are in LDS.
void hm_waitcnt(int immediate);
#define __builtin_amdgcn_s_waitcnt(x) hm_waitcnt(x)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)

// ---- buffer descriptors: base and range (raw buffers, no stride, no swizzle) -----
struct HmRsrc {
  const char *base;
  unsigned num_records;
};
#define __amdgpu_buffer_rsrc_t HmRsrc
inline HmRsrc hm_make_rsrc(void *base, int, int num, int) { return HmRsrc{(const char *)base, (unsigned)num}; }
#define __builtin_amdgcn_make_buffer_rsrc hm_make_rsrc

// a lane whose offset lies at or beyond the range reads zeros and touches no memory (runner.cpp)
void hm_load_lds(HmRsrc r, void *lds, int size, int voff, int soff, int ioff, int aux);
#define __builtin_amdgcn_raw_ptr_buffer_load_lds hm_load_lds
typedef int hm_v4i __attribute__((ext_vector_type(4)));
hm_v4i hm_load_b128(HmRsrc r, int voff, int soff, int aux);
#define __builtin_amdgcn_raw_buffer_load_b128 hm_load_b128

// ---- cross-lane operations (runner.cpp) -----------------------------------------------
void hm_first_lane(void *value, size_t bytes);           // value <- lane 0's value
uint64_t hm_ballot(bool p);
int hm_bpermute(int byte_index, int v);
void hm_shuffle_xor(void *value, size_t bytes, int mask, int width);
template <typename T> inline T hm_readfirstlane(T v) { // (the kernels use it on wave-uniform values)
  hm_first_lane(&v, sizeof v);
  return v;
}
#define __builtin_amdgcn_readfirstlane(x) hm_readfirstlane(x)
#define __builtin_amdgcn_ballot_w64(x) hm_ballot(x)
#define __builtin_amdgcn_ds_bpermute(a, v) hm_bpermute(a, v)
template <typename T> inline T __shfl_xor(T v, int mask, int width = 64) {
  hm_shuffle_xor(&v, sizeof v, mask, width);
  return v;
}

// Transposing LDS reads.  16 lanes each name 8 bytes, the rows of a block of 4 rows x 16 sixteen-bit (8 rows x 16
// eight-bit) elements: lane 4r + q (2r + h) names columns 4q..4q+3 (8h..8h+7) of row r; lane i receives column i,
// top to bottom.
typedef short hm_v4s __attribute__((ext_vector_type(4)));
typedef int hm_v2i __attribute__((ext_vector_type(2)));
void hm_read_transposed(const void *p, int elem_bytes, void *out8);
inline hm_v4s hm_read_tr16(const void *p) {
  hm_v4s v;
  hm_read_transposed(p, 2, &v);
  return v;
}
inline hm_v2i hm_read_tr8(const void *p) {
  hm_v2i v;
  hm_read_transposed(p, 1, &v);
  return v;
}
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) hm_read_tr16((const void *)(p))
#define __builtin_amdgcn_ds_read_tr8_b64_v2i32(p) hm_read_tr8((const void *)(p))

// ---- 8-bit float codecs (OCP e4m3fn, e5m2; runner.cpp) ----------------------------------
float hm_f8_to_f32(unsigned code, int ebits);
int hm_cvt_pk_f8(float a, float b, int old, bool hi, int ebits); // round to nearest even; the callers clamp first
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, hi) hm_cvt_pk_f8(a, b, old, hi, 4)
#define __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, hi) hm_cvt_pk_f8(a, b, old, hi, 5)
#define __builtin_amdgcn_cvt_f32_fp8(v, sel) hm_f8_to_f32(((unsigned)(v) >> (8 * (sel))) & 255, 4)
#define __builtin_amdgcn_cvt_f32_bf8(v, sel) hm_f8_to_f32(((unsigned)(v) >> (8 * (sel))) & 255, 5)

// ---- matrix instructions: D (32 x 32) += A (32 x K) * B (K x 32) (runner.cpp) ------------
// Lane l holds its share of row (column) l % 32: the consecutive k starting at (k per lane) * (l / 32); it
// receives column l % 32 of D, rows 8 * (v / 4) + 4 * (l / 32) + v % 4 for its values v = 0..15.
enum { HM_F32, HM_F16, HM_BF16, HM_I8, HM_E4M3, HM_E5M2 };
void hm_mfma_32x32(int type_a, int type_b, const void *a, const void *b, int lane_bytes, void *acc16);
template <typename V, typename Acc> inline Acc hm_mfma_f16(V a, V b, Acc c, int, int, int) {
  hm_mfma_32x32(HM_F16, HM_F16, &a, &b, 16, &c);
  return c;
}
template <typename V, typename Acc> inline Acc hm_mfma_bf16(V a, V b, Acc c, int, int, int) {
  hm_mfma_32x32(HM_BF16, HM_BF16, &a, &b, 16, &c);
  return c;
}
template <typename Acc> inline Acc hm_mfma_f32(float a, float b, Acc c, int, int, int) {
  hm_mfma_32x32(HM_F32, HM_F32, &a, &b, 4, &c);
  return c;
}
template <typename V, typename Acc> inline Acc hm_mfma_i8(V a, V b, Acc c, int, int, int) {
  hm_mfma_32x32(HM_I8, HM_I8, &a, &b, 16, &c);
  return c;
}
// (the 8-bit float instruction: formats 0 = e4m3, 1 = e5m2 per operand, unit block scales)
template <typename V, typename Acc> inline Acc hm_mfma_f8(V a, V b, Acc c, int fmt_a, int fmt_b, int, int, int, int) {
  hm_mfma_32x32(fmt_a ? HM_E5M2 : HM_E4M3, fmt_b ? HM_E5M2 : HM_E4M3, &a, &b, 32, &c);
  return c;
}
#define __builtin_amdgcn_mfma_f32_32x32x16_f16 hm_mfma_f16
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16 hm_mfma_bf16
#define __builtin_amdgcn_mfma_f32_32x32x2f32 hm_mfma_f32
#define __builtin_amdgcn_mfma_i32_32x32x32_i8 hm_mfma_i8
#define __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4 hm_mfma_f8

#define __builtin_amdgcn_exp2f(x) exp2f(x)
inline float __frcp_rn(float x) { return 1.0f / x; }
inline float __expf(float x) { return expf(x); }
