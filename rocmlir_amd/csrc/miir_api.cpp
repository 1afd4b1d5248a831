// The exported C ABI: the Miir entry points (rocmlir-lib.cpp:117-316) and this library's own.
#include "rock_host.h"

using namespace rockhost;

// ============================================================================
// C ABI
// ============================================================================
extern "C" {

MiirHandle miirCreateHandle(const char *options) {
  g_last_error.clear();
  OptMap o;
  if (!parse_options(options, o)) {
    set_error("could not parse the options string");
    return nullptr;
  }
  return build_handle(o);
}

int miirGetKernelCount(MiirHandle handle) {
  return handle ? static_cast<Handle *>(handle)->kernel_count : -1;
}

int miirGetWorkspaceSize(MiirHandle handle) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return -1;
  return h->workspace_bytes > (size_t)INT32_MAX ? -1 : (int)h->workspace_bytes;
}

size_t rockamdGetWorkspaceSize64(MiirHandle handle) {
  auto *h = static_cast<Handle *>(handle);
  return h ? h->workspace_bytes : (size_t)-1;
}

MiirStatus miirLowerTuningParams(MiirHandle handle) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return MIIR_INVALID_PARAM;
  h->tuned = true;
  return MIIR_SUCCESS;
}

MiirStatus miirLowerBin(MiirHandle handle) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return MIIR_INVALID_PARAM;
  if (!h->blob || h->blob->end <= h->blob->start)
    return MIIR_BUILD_FAILURE;
  h->tuned = true;
  h->lowered = true;
  return MIIR_SUCCESS;
}

MiirStatus miirBufferGet(MiirHandle handle, char *buffer, size_t *size) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !size)
    return MIIR_INVALID_PARAM;
  if (!h->lowered)
    return MIIR_INVALID_MODULE;
  size_t n = (size_t)(h->blob->end - h->blob->start);
  if (buffer) {
    if (*size < n)
      return MIIR_INVALID_PARAM;
    std::memcpy(buffer, h->blob->start, n);
  }
  *size = n;
  return MIIR_SUCCESS;
}

MiirStatus miirGetExecutionDims(MiirHandle handle, size_t *global_size, size_t *local_size) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !global_size || !local_size)
    return MIIR_INVALID_PARAM;
  if (!h->tuned)
    return MIIR_INVALID_MODULE;
  *global_size = (size_t)h->grid_size * h->block_size;
  *local_size = h->block_size;
  return MIIR_SUCCESS;
}

MiirStatus miirDestroyHandle(MiirHandle handle) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return MIIR_INVALID_PARAM;
  delete h;
  return MIIR_SUCCESS;
}

MiirStatus rockamdGetKernelName(MiirHandle handle, char *buffer, size_t *size) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !size)
    return MIIR_INVALID_PARAM;
  size_t n = h->kernel_name.size() + 1;
  if (buffer) {
    if (*size < n)
      return MIIR_INVALID_PARAM;
    std::memcpy(buffer, h->kernel_name.c_str(), n);
  }
  *size = n;
  return MIIR_SUCCESS;
}

MiirStatus rockamdGetKernelAttrs(MiirHandle handle, uint32_t attrs[2]) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !attrs)
    return MIIR_INVALID_PARAM;
  attrs[0] = h->block_size;
  attrs[1] = h->grid_size;
  return MIIR_SUCCESS;
}

MiirStatus rockamdGetKernelArgs(MiirHandle handle, int *num_pointers, void *params,
                                size_t *params_size) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !params_size)
    return MIIR_INVALID_PARAM;
  if (num_pointers)
    *num_pointers = h->num_pointers;
  if (params) {
    if (*params_size < h->params.size())
      return MIIR_INVALID_PARAM;
    std::memcpy(params, h->params.data(), h->params.size());
  }
  *params_size = h->params.size();
  return MIIR_SUCCESS;
}

MiirStatus rockamdGetArgumentInfo(MiirHandle handle, int index, int *dtype, int *rank, int64_t *dims) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || index < 0 || index >= (int)h->args.size())
    return MIIR_INVALID_PARAM;
  const auto &a = h->args[index];
  if (dtype)
    *dtype = a.dtype;
  if (rank)
    *rank = (int)a.dims.size();
  if (dims)
    for (size_t i = 0; i < a.dims.size(); ++i)
      dims[i] = a.dims[i];
  return MIIR_SUCCESS;
}

MiirStatus rockamdCheckArgumentSizes(MiirHandle handle, const size_t *bytes, int num_pointers) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !bytes || num_pointers != (int)h->args.size()) {
    set_error("argument sizes: one size per pointer of the caller's list");
    return MIIR_INVALID_PARAM;
  }
  for (int i = 0; i < num_pointers; ++i) {
    const auto &a = h->args[i];
    uint64_t need = a.dtype < 0 ? 1 : (uint64_t)dtype_size(a.dtype);
    for (int64_t d : a.dims)
      need *= (uint64_t)d;
    if (bytes[i] != 0 && bytes[i] < need) {
      set_error("argument " + std::to_string(i) + " holds " + std::to_string(bytes[i]) + " bytes, the kernel list addresses " +
                std::to_string(need));
      return MIIR_INVALID_PARAM;
    }
  }
  return MIIR_SUCCESS;
}

// Copies as much of s as fits and ALWAYS terminates it; returns the full
// length, so a result >= buffer_size tells the caller the text was cut.  (The
// reference's strncpy, mlir/lib/CAPI/Dialect/Rock.cpp:86,142, leaves a short
// buffer unterminated; with a buffer that is large enough the two agree.)
static size_t copy_string(const std::string &s, char *buffer, size_t buffer_size) {
  if (buffer && buffer_size > 0) {
    const size_t n = std::min(s.size(), buffer_size - 1);
    std::memcpy(buffer, s.data(), n);
    buffer[n] = '\0';
  }
  return s.size();
}

size_t rockamdGetPerfConfig(MiirHandle handle, char *buffer, size_t buffer_size) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return (size_t)-1;
  return copy_string(h->perf_config, buffer, buffer_size);
}

size_t rockamdGetProblemKey(MiirHandle handle, char *buffer, size_t buffer_size) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return (size_t)-1;
  return copy_string(h->problem_key, buffer, buffer_size);
}

MiirStatus rockamdGetPointerMap(MiirHandle handle, int *caller_pointers, int *kernel_pointers,
                                int32_t *source, int64_t *offset) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return MIIR_INVALID_PARAM;
  if (caller_pointers)
    *caller_pointers = h->caller_pointers ? h->caller_pointers : h->num_pointers;
  if (kernel_pointers)
    *kernel_pointers = h->num_pointers;
  for (int i = 0; i < h->num_pointers; ++i) {
    if (source)
      source[i] = h->ptr_map.empty() ? i : h->ptr_map[i].source;
    if (offset)
      offset[i] = h->ptr_map.empty() ? 0 : h->ptr_map[i].offset;
  }
  return MIIR_SUCCESS;
}

MiirStatus rockamdGetParamPointers(MiirHandle handle, int *count, int32_t *param_offset, int32_t *source) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !count)
    return MIIR_INVALID_PARAM;
  *count = (int)h->param_ptrs.size();
  for (size_t i = 0; i < h->param_ptrs.size(); ++i) {
    if (param_offset)
      param_offset[i] = h->param_ptrs[i].offset;
    if (source)
      source[i] = h->param_ptrs[i].source;
  }
  return MIIR_SUCCESS;
}

MiirStatus rockamdSetScale(MiirHandle handle, float scale) {
  auto *h = static_cast<Handle *>(handle);
  if (!h)
    return MIIR_INVALID_PARAM;
  if (h->op == OP_ATTENTION) {
    auto *ap = reinterpret_cast<RockAttentionParams *>(h->params.data());
    // The plain fused kernel takes the row maximum of the raw scores and
    // scales afterwards, which is only right for a non-negative scale: a
    // negative one moves such a handle to the kernel that scales first.  A
    // handle that the caller, the table or the tuner put on the scale-first
    // kernel is valid for either sign and stays there; one that a negative scale
    // moved comes back when the scale turns non-negative again.
    const std::string plain = "_fast", first = "_fast_bias";
    // (the kernels for K stored [d, seq_k] carry "_kt" behind the variant)
    std::string name = h->kernel_name, layout;
    if (name.size() > 3 && name.compare(name.size() - 3, 3, "_kt") == 0) {
      layout = "_kt";
      name.erase(name.size() - 3);
    }
    auto ends_with = [&](const std::string &suffix) {
      return name.size() >= suffix.size() && name.compare(name.size() - suffix.size(), suffix.size(), suffix) == 0;
    };
    std::string target;
    if (scale < 0.0f && ends_with(plain))
      target = name + "_bias" + layout;
    else if (scale >= 0.0f && h->moved_for_scale_sign && ends_with(first))
      target = name.substr(0, name.size() - 5) + layout;
    if (!target.empty()) {
      const Blob *blob = find_blob(target);
      if (!blob) { // never leave a handle without its code object
        set_error("attention kernel " + target + " is not in this library");
        return MIIR_INVALID_PARAM;
      }
      const bool to_first = scale < 0.0f;
      h->kernel_name = target;
      h->blob = blob; // one code object per kernel: the handle's follows its kernel
      h->functions.clear();
      h->moved_for_scale_sign = to_first;
      const int dmax = target.find("_d64x") != std::string::npos    ? 64
                       : target.find("_d256x") != std::string::npos ? 256
                                                                     : 128;
      h->perf_config = attn_perf_string(kAttnVariants[to_first ? 1 : 0], dmax);
    }
    ap->scale = scale;
  } else if (h->epi)
    h->epi->scale = scale;
  else
    return MIIR_INVALID_PARAM; // a layout-conversion kernel has no epilogue
  return MIIR_SUCCESS;
}

MiirStatus rockamdSetZeroPoint(MiirHandle handle, int32_t zero_point) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || h->op == OP_ATTENTION || !h->epi)
    return MIIR_INVALID_PARAM;
  h->epi->zero_point = zero_point;
  return MIIR_SUCCESS;
}

int rockamdLaunch(MiirHandle handle, void *const *pointers, int num_pointers, void *stream) {
  auto *h = static_cast<Handle *>(handle);
  if (!check_launch_args(h, pointers, num_pointers))
    return (int)hipErrorInvalidValue;
  hipFunction_t fn;
  int rc = get_function(h, &fn);
  if (rc != 0)
    return rc;
  rc = launch_once(h, fn, pointers, (hipStream_t)stream);
  if (rc != 0)
    set_error(std::string("launch failed: ") + hipGetErrorString((hipError_t)rc));
  return rc;
}

// ---- tuning surface ---------------------------------------------------------
RockamdTuningSpace rockamdTuningSpaceCreate(MiirHandle handle, int kind) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || (kind != ROCKAMD_TUNING_QUICK && kind != ROCKAMD_TUNING_FULL && kind != ROCKAMD_TUNING_EXHAUSTIVE))
    return nullptr;
  auto *sp = new TuningSpace;
  sp->params = tuning_candidates(*h, kind);
  return sp;
}

unsigned rockamdTuningGetNumParams(RockamdTuningSpace space) {
  return space ? (unsigned)static_cast<TuningSpace *>(space)->params.size() : 0u;
}

size_t rockamdTuningParamToString(RockamdTuningSpace space, unsigned pos, char *buffer, size_t buffer_size) {
  auto *sp = static_cast<TuningSpace *>(space);
  if (!sp || pos >= sp->params.size())
    return (size_t)-1;
  return copy_string(sp->params[pos], buffer, buffer_size);
}

void rockamdTuningSpaceDestroy(RockamdTuningSpace space) { delete static_cast<TuningSpace *>(space); }

int rockamdTuningSetFromStr(MiirHandle handle, const char *perf_config) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !perf_config)
    return 0;
  OptMap o = h->options;
  o["perf_config"] = perf_config;
  Handle *n = build_handle(o);
  if (!n)
    return 0;
  if (n->epi && h->epi)
    *n->epi = *h->epi; // scalars changed with rockamdSetScale / SetZeroPoint stay
  *h = std::move(*n); // params moves with its buffer, so the typed views stay valid
  delete n;
  return 1;
}

RockamdTuningTable rockamdTuningTableCreate(void) { return new TuningTable; }

void rockamdTuningTableDestroy(RockamdTuningTable table) { delete static_cast<TuningTable *>(table); }

int rockamdTuningUpdateTable(RockamdTuningTable table, const char *problem_key, const char *perf_config,
                             float time) {
  auto *t = static_cast<TuningTable *>(table);
  if (!t || !problem_key || !perf_config)
    return 0;
  std::lock_guard<std::mutex> lock(t->mutex);
  auto it = t->best.find(problem_key);
  if (it != t->best.end() && it->second.second <= time)
    return 0; // a better-performing entry exists
  t->best[problem_key] = std::make_pair(std::string(perf_config), time);
  return 1;
}

int rockamdTuningSetFromTable(RockamdTuningTable table, MiirHandle handle) {
  auto *t = static_cast<TuningTable *>(table);
  auto *h = static_cast<Handle *>(handle);
  if (!t || !h)
    return 0;
  std::string perf_config;
  {
    std::lock_guard<std::mutex> lock(t->mutex);
    auto it = t->best.find(h->problem_key);
    if (it == t->best.end())
      return 0;
    perf_config = it->second.first;
  }
  return rockamdTuningSetFromStr(handle, perf_config.c_str());
}

int rockamdIsSplitKFaster(int64_t g, int64_t m, int64_t n, int64_t k, int64_t num_cu, int element_size) {
  if (g <= 0 || m <= 0 || n <= 0 || k <= 0 || num_cu <= 0 || element_size <= 0)
    return ROCKAMD_SPLITK_NEVER;
  if (k * element_size < 16 * 64)
    return ROCKAMD_SPLITK_NEVER; // a K range this short gives each wave less than one 64-byte step
  const int64_t tiles64 = (int64_t)ceil_div(m, 64) * ceil_div(n, 64) * g;
  if (tiles64 * 2 <= num_cu)
    return ROCKAMD_SPLITK_ALWAYS; // make_gemm's own rule: 64x64 tiles would leave half the CUs idle
  return tiles64 <= num_cu ? ROCKAMD_SPLITK_MAYBE : ROCKAMD_SPLITK_NEVER;
}

int rockamdIsFusible(MiirHandle handle, const char *perf_config) {
  auto *h = static_cast<Handle *>(handle);
  if (!h || !perf_config)
    return 0;
  // The reference refuses an element-wise tail behind a split reduction
  // because its partial sums meet in memory through atomic adds
  // (RockTuningImpl.cpp:1010-1015).  Here a requested split (seventh field of
  // the perf_config > 1) is the kernel that divides K over the waves of one
  // block and sums the partial tiles in LDS BEFORE the epilogue, and the split
  // over blocks through a workspace is only ever planned for an identity
  // epilogue: whatever the handle resolves to under the string keeps its tail.
  OptMap o = h->options;
  o["perf_config"] = perf_config;
  const std::string keep_error = g_last_error;
  Handle *c = build_handle(o);
  g_last_error = keep_error;
  if (!c)
    return 0;
  delete c;
  return 1;
}

size_t rockamdGetNumPrefillArgs(MiirHandle handle) {
  (void)handle; // no kernel of this library accumulates into memory it has not written itself
  return 0;
}

void rockamdGetPrefillArgsInfo(MiirHandle handle, size_t *indices, float *init_values, size_t length) {
  (void)handle; (void)indices; (void)init_values; (void)length; // nothing to report: the count is zero
}

const char *rockamdGetLastError(void) { return g_last_error.c_str(); }

} // extern "C"
