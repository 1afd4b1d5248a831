// rockamdLaunchStaticWorkspace: rockamdLaunch for callers that cannot
// allocate device memory (code under HIP graph capture, serving loops and
// harnesses that forbid hipMalloc).  Problems that lower to several kernels
// pass intermediate results through a workspace which rockamdLaunch's caller
// allocates; here that workspace is an array in the library's own device
// image, so the call needs the problem's tensors only and allocates nothing.
//
// The array exists once per GPU (every device that loads the library's device
// image holds its own copy until the process ends) and keeps the last call's
// contents.  Nothing has to be cleared between problems: every kernel list of
// this library writes each workspace byte whose value reaches a result before
// a later kernel of the same list reads it.  The one exception reads stale
// bytes without using them: the rows-of-taps copies of an input are sized one
// run of taps past their last row, the contraction loads that slack (left over
// from an earlier problem) and discards it -- the forward kernel zeroes the
// row tails, the filter gradient drops those columns.  All calls on one GPU share the array, so two problems whose
// kernel lists overlap in time on the same GPU (different streams or threads)
// race on it; serialise them or use rockamdLaunch with separate workspaces.
#include <hip/hip_runtime.h>

#include "../../include/rocmlir_amd.h"
#include "rock_internal.h"

namespace {

constexpr size_t kScratchBytes = ROCKAMD_STATIC_WORKSPACE_BYTES;
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// Device address of `scratch` on each GPU.  The array's name is a host-side
// stand-in, not an address a kernel can use: the address comes from
// hipGetSymbolAddress, once per device with that device current, and only the
// pointer kept here is ever handed to a kernel.
void *g_scratch_ptr[kMaxDevices];

} // namespace

extern "C" ROCMLIR_AMD_API int rockamdLaunchStaticWorkspace(MiirHandle handle, void *const *pointers,
                                                           int num_pointers, void *stream) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return (int)e;
  if (dev < 0 || dev >= kMaxDevices)
    return (int)hipErrorInvalidDevice;
  void *ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!ptr) { // first call on this device (two racing threads resolve the same address)
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
    __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
  }
  return rock_launch_with_workspace(handle, pointers, num_pointers, ptr, kScratchBytes, stream);
}
