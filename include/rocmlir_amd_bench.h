/* Measurement helpers of librocmlir_amd.so: what the benchmark and the tuner use to time kernels.  They are
 * exported from the same library as the C ABI of rocmlir_amd.h but are no part of the drop-in boundary: a client
 * of the reference's Miir interface needs none of them.  The reference times kernels from its Python scripts
 * through rocprof (mlir/utils/performance/perfRunner.py:131-141, 926-938). */
#ifndef ROCMLIR_AMD_BENCH_H
#define ROCMLIR_AMD_BENCH_H

#include "rocmlir_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Timed loop with HIP events on `stream`: `warmup` untimed launches, then
 * `iters` launches between one start/stop event pair; writes the average
 * milliseconds per launch.  Synchronises the stream. */
ROCMLIR_AMD_API int rockamdBenchmark(MiirHandle handle, void *const *pointers, int num_pointers,
                     void *stream, int warmup, int iters, float *avg_ms);

/* Matrix-core issue-rate probe on the current device: runs a register-only
 * chain of 32x32 MFMAs of the given operand type (a RockDType value: f32, f16,
 * bf16, i8 or fp8) and writes the sustained rate in tera-operations per
 * second.  `random_data` != 0 gives the operands hashed bit patterns instead
 * of constants; the gap between the two is the clock the part gives up to
 * power on real data.  The reference has no counterpart (its perf scripts
 * compare against rocBLAS instead, mlir/utils/performance/perfRunner.py);
 * the benchmark reports it next to every roofline fraction. */
ROCMLIR_AMD_API int rockamdMeasureMfmaRate(int dtype, int random_data, void *stream,
                                           double *tera_ops);

#ifdef __cplusplus
}
#endif

#endif /* ROCMLIR_AMD_BENCH_H */
