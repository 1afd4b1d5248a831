// Measurement helpers exported beside the C ABI (include/rocmlir_amd_bench.h): HIP-event timing of a handle's
// kernel and the MFMA issue-rate probe.
#include "rock_host.h"
#include "../../include/rocmlir_amd_bench.h"

using namespace rockhost;

extern "C" {

int rockamdBenchmark(MiirHandle handle, void *const *pointers, int num_pointers, void *stream,
                     int warmup, int iters, float *avg_ms) {
  auto *h = static_cast<Handle *>(handle);
  if (!check_launch_args(h, pointers, num_pointers) || iters <= 0 || !avg_ms)
    return (int)hipErrorInvalidValue;
  hipFunction_t fn;
  int rc = get_function(h, &fn);
  if (rc != 0)
    return rc;
  hipStream_t s = (hipStream_t)stream;
  for (int i = 0; i < warmup && rc == 0; ++i)
    rc = launch_once(h, fn, pointers, s);
  if (rc != 0)
    return rc;
  hipEvent_t e0, e1;
  if ((rc = (int)hipEventCreate(&e0)) != 0)
    return rc;
  if ((rc = (int)hipEventCreate(&e1)) != 0) {
    hipEventDestroy(e0);
    return rc;
  }
  rc = (int)hipEventRecord(e0, s);
  for (int i = 0; i < iters && rc == 0; ++i)
    rc = launch_once(h, fn, pointers, s);
  if (rc == 0)
    rc = (int)hipEventRecord(e1, s);
  if (rc == 0)
    rc = (int)hipEventSynchronize(e1);
  float ms = 0.0f;
  if (rc == 0)
    rc = (int)hipEventElapsedTime(&ms, e0, e1);
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  if (rc != 0) {
    set_error(std::string("benchmark failed: ") + hipGetErrorString((hipError_t)rc));
    return rc;
  }
  *avg_ms = ms / (float)iters;
  return 0;
}

int rockamdMeasureMfmaRate(int dtype, int random_data, void *stream, double *tera_ops) {
  static const char *names[] = {"f32", "f16", "bf16", "i8", "fp8"};
  // multiply-accumulates of one 32x32xK instruction per operand type
  static const double macs[] = {32 * 32 * 2 * 4.0, 32 * 32 * 16.0, 32 * 32 * 16.0, 32 * 32 * 32.0,
                                32 * 32 * 64.0};
  if (dtype < 0 || dtype > ROCK_FP8 || !tera_ops) {
    set_error("rate probe: operand type must be f32, f16, bf16, i8 or fp8");
    return (int)hipErrorInvalidValue;
  }
  const std::string kname = std::string("rock_probe_mfma_") + names[dtype];
  const Blob *blob = find_blob(kname);
  if (!blob)
    return (int)hipErrorInvalidValue;
  hipModule_t mod;
  if (int rc = load_module(blob, &mod))
    return rc;
  hipError_t e;
  hipFunction_t fn;
  e = hipModuleGetFunction(&fn, mod, kname.c_str());
  if (e != hipSuccess)
    return (int)e;
  const int blocks = kNumCU * 4, threads = 256, iters = 40000;
  float *out = nullptr;
  e = hipMalloc((void **)&out, (size_t)blocks * threads * sizeof(float));
  if (e != hipSuccess)
    return (int)e;
  hipStream_t s = (hipStream_t)stream;
  int it = iters, rnd = random_data;
  void *args[] = {&out, &it, &rnd};
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  int rc = (int)hipModuleLaunchKernel(fn, blocks, 1, 1, threads, 1, 1, 0, s, args, nullptr); // warm-up
  if (rc == 0) rc = (int)hipEventRecord(e0, s);
  if (rc == 0) rc = (int)hipModuleLaunchKernel(fn, blocks, 1, 1, threads, 1, 1, 0, s, args, nullptr);
  if (rc == 0) rc = (int)hipEventRecord(e1, s);
  if (rc == 0) rc = (int)hipEventSynchronize(e1);
  float ms = 0.0f;
  if (rc == 0) rc = (int)hipEventElapsedTime(&ms, e0, e1);
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  hipFree(out);
  if (rc != 0) {
    set_error(std::string("rate probe failed: ") + hipGetErrorString((hipError_t)rc));
    return rc;
  }
  // 4 instructions per iteration per wave, 4 waves per block
  double ops = 2.0 * macs[dtype] * 4.0 * iters * 4.0 * blocks;
  *tera_ops = ops / (ms * 1e-3) / 1e12;
  return 0;
}

} // extern "C"
