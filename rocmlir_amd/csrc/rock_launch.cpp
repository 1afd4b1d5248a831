// Module cache and kernel launches.
#include "rock_host.h"

namespace rockhost {

// --------------------------------------------------------------------------
// module cache: one hipModule per (device, code object)
// --------------------------------------------------------------------------
namespace {
std::mutex g_module_mutex;
std::map<std::pair<int, const Blob *>, hipModule_t> g_modules;
} // namespace

int load_module(const Blob *blob, hipModule_t *module) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return (int)e;
  std::lock_guard<std::mutex> lock(g_module_mutex);
  const auto key = std::make_pair(dev, blob);
  auto it = g_modules.find(key);
  if (it == g_modules.end()) {
    e = hipModuleLoadData(module, blob->start);
    if (e != hipSuccess) {
      set_error(std::string("hipModuleLoadData failed for ") + blob->name + ": " + hipGetErrorString(e));
      return (int)e;
    }
    g_modules[key] = *module;
  } else {
    *module = it->second;
  }
  return 0;
}

int get_function(Handle *h, hipFunction_t *fn) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return (int)e;
  auto it = h->functions.find(dev);
  if (it != h->functions.end()) {
    *fn = it->second;
    return 0;
  }
  hipModule_t mod;
  const int rc = load_module(h->blob, &mod);
  if (rc != 0)
    return rc;
  e = hipModuleGetFunction(fn, mod, h->kernel_name.c_str());
  if (e != hipSuccess) {
    set_error("kernel " + h->kernel_name + " not found in code object: " + hipGetErrorString(e));
    return (int)e;
  }
  h->functions[dev] = *fn;
  return 0;
}

int launch_once(Handle *h, hipFunction_t fn, void *const *pointers, hipStream_t stream) {
  // argument buffer: the pointers, then the parameter block (8-byte aligned)
  constexpr size_t kMaxPointers = 8, kMaxParams = 1024;
  char buf[kMaxPointers * 8 + kMaxParams];
  if ((size_t)h->num_pointers > kMaxPointers || h->params.size() > kMaxParams) {
    set_error("launch: kernel argument block larger than the launch buffer");
    return (int)hipErrorInvalidValue;
  }
  size_t off = 0;
  for (int i = 0; i < h->num_pointers; ++i, off += 8) {
    const void *ptr = h->ptr_map.empty()           ? pointers[i]
                      : h->ptr_map[i].source < 0   ? nullptr
                                                   : (const char *)pointers[h->ptr_map[i].source] + h->ptr_map[i].offset;
    std::memcpy(buf + off, &ptr, 8);
  }
  std::memcpy(buf + off, h->params.data(), h->params.size());
  for (const Handle::ParamPtr &pp : h->param_ptrs) // tensors whose pointers ride inside the block
    std::memcpy(buf + off + pp.offset, &pointers[pp.source], 8);
  size_t size = off + h->params.size();
  void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, buf, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                    HIP_LAUNCH_PARAM_END};
  return (int)hipModuleLaunchKernel(fn, h->grid_size, 1, 1, h->block_size, 1, 1, 0, stream,
                                    nullptr, config);
}

bool check_launch_args(Handle *h, void *const *pointers, int num_pointers) {
  const int expected = h ? (h->caller_pointers ? h->caller_pointers : h->num_pointers) : 0;
  if (!h || !pointers || num_pointers != expected) {
    set_error("launch: wrong number of pointer arguments");
    return false;
  }
  if (!h->lowered) {
    set_error("launch: miirLowerBin has not been called on this handle");
    return false;
  }
  // the vector paths assume 16-byte aligned tensors (true for any allocator)
  for (int i = 0; i < num_pointers; ++i)
    if (((uintptr_t)pointers[i] & 15) != 0) {
      set_error("launch: tensor pointers must be 16-byte aligned");
      return false;
    }
  int aux_index = 3; // the bias slot, which may be NULL when the problem has no bias
  bool need_aux = h->epi && h->epi->has_bias != 0;
  if (h->op == OP_ATTENTION) {
    const auto *ap = reinterpret_cast<RockAttentionParams *>(h->params.data());
    need_aux = ap->has_bias != 0;
    aux_index = ap->has_scale_tensor ? 4 : 3;
  }
  for (int i = 0; i < num_pointers; ++i)
    if (!pointers[i] && (i != aux_index || need_aux)) {
      set_error("launch: NULL tensor pointer");
      return false;
    }
  return true; // (a residual, when the problem names one, is pointer 4 and covered by the loop)
}

} // namespace rockhost

using namespace rockhost;

// see rock_internal.h
int rock_launch_with_workspace(void *handle, void *const *pointers, int num_pointers, void *workspace,
                               size_t capacity, void *stream) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !pointers) {
    set_error("launch: NULL handle or pointer list");
    return (int)hipErrorInvalidValue;
  }
  const int expected = h->caller_pointers ? h->caller_pointers : h->num_pointers;
  const bool has_workspace = h->workspace_bytes != 0;
  void *full[16];
  if (num_pointers != expected - (has_workspace ? 1 : 0) || expected > 16) {
    set_error("launch: wrong number of pointer arguments (the workspace is not one of them here)");
    return (int)hipErrorInvalidValue;
  }
  if (h->workspace_bytes > capacity) {
    char msg[160];
    std::snprintf(msg, sizeof msg, "launch: the problem needs a workspace of %zu bytes, the built-in one holds %zu",
                  h->workspace_bytes, capacity);
    set_error(msg);
    return (int)hipErrorInvalidValue;
  }
  for (int i = 0; i < num_pointers; ++i)
    full[i] = pointers[i];
  if (has_workspace)
    full[num_pointers] = workspace; // the workspace closes every multi-kernel problem's caller list
  if (!check_launch_args(h, full, expected))
    return (int)hipErrorInvalidValue;
  hipFunction_t fn;
  int rc = get_function(h, &fn);
  if (rc != 0)
    return rc;
  rc = launch_once(h, fn, full, (hipStream_t)stream);
  if (rc != 0)
    set_error(std::string("launch failed: ") + hipGetErrorString((hipError_t)rc));
  return rc;
}
