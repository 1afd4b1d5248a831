/*
 * rocmlir_amd.h -- C ABI of librocmlir_amd.so: MI355X (gfx950) kernels for the
 * Rock-dialect contraction ops (GEMM, forward convolution, fused attention,
 * quantised-GEMM epilogue), handed back as launchable HIP code objects.
 *
 * The first block is a drop-in for the reference's kernel-generator library
 * (mlir/tools/rocmlir-lib/Miir.h:16-101): same names, same argument meaning,
 * same NULL / status error behaviour, same two-call buffer protocol.  The
 * second block carries what MIGraphX reads through the MLIR C API
 * (mlir/include/mlir-c/Dialect/MIGraphX.h:27-78, mlir-c/Dialect/Rock.h:22-167)
 * for the same kernels: name, block/grid, argument list, perf-config string,
 * tuning problem key.  The third block is a convenience launcher so that a
 * host without its own hipModule plumbing (tests, benchmarks, a ctypes or
 * cgo binding) can run what it was handed.
 *
 * All entry points are plain C, take only pointers, sizes and scalars, never
 * throw, and may be called from several threads; a handle must not be used
 * from two threads at once.
 */
#ifndef ROCMLIR_AMD_H
#define ROCMLIR_AMD_H

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define ROCMLIR_AMD_API __attribute__((visibility("default")))
#else
#define ROCMLIR_AMD_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* Miir.h:18 -- kernel ABI generation: bare pointers, one per tensor. */
#define MIIR_VERSION_FLAT 6
/* This library's own revision of the extension block below. */
#define ROCMLIR_AMD_API_VERSION 1

/* Miir.h:20-26 */
enum MiirStatus {
  MIIR_SUCCESS = 0,
  MIIR_INVALID_PARAM,
  MIIR_INVALID_MODULE,
  MIIR_BUILD_FAILURE
};
typedef enum MiirStatus MiirStatus;

/* Miir.h:30 */
typedef void *MiirHandle;

/* ---------------------------------------------------------------------------
 * 1. Miir drop-in
 * ------------------------------------------------------------------------- */

/* Miir.h:50 (impl rocmlir-lib.cpp:117-154).  `options` is a whitespace
 * separated "--key value" list.  Convolution keys are the reference's
 * (ConvGenerator.cpp:492-661): operation {conv|conv_bwd_data|conv_bwd_weight}
 * (the gradients take f32, f16 or bf16, the forward problem's keys and pointer
 * order, and usually several kernels: see rockamdGetPointerMap), arch, num_cu, kernel_id,
 * kernel_name, perf_config, in_type/fil_type/out_type, in_layout/fil_layout/
 * out_layout, batchsize, groupsize, in_channels, out_channels, in_h, in_w,
 * out_h, out_w, fil_h, fil_w, dilation_{h,w}, conv_stride_{h,w},
 * padding_{h,w}.  With in_d / fil_d (and out_d, dilation_d, conv_stride_d,
 * padding_d; rocmlir-gen.cpp:171-294) the convolution, forward or either
 * gradient, runs over three spatial dimensions and the layouts have six
 * letters (ngc012 / gkc012 / ngk012, h w d and y x z accepted for 0 1 2):
 * several kernels over a workspace, same pointer order.  `--operation gemm` and `--operation attention` take the
 * reference's rocmlir-gen flag names (rocmlir-gen.cpp:90-561): t,
 * out_datatype, g, m, k, n, transA, transB, transC; g, seq_len_q, seq_len_k,
 * head_dim_qk, head_dim_v, transQ, transK, transV, transO, with-attn-bias,
 * with-attn-scale (pointer order Q, K, V, [scale tensor], bias slot, O);
 * attention types f16, bf16, f32, and i8 = int8 Q and K with f16 V / O, the
 * scores dequantised as (acc - zero_point) * scale.  One fused kernel covers
 * the 16-bit types up to head dimension 256 and i8 up to 128 (beyond 128, and
 * for i8, over tensors contiguous along the head dimension: transK, no other
 * transpose); f32, larger head dimensions and "-fused false" run as three
 * kernels over a score workspace.
 * Epilogue keys (all optional): scale, zero_point, quant_scale,
 * out_zero_point, bias, relu; and the element-wise operations MIGraphX fuses
 * behind a contraction (MIGraphXToTosa.cpp:1009-1016, 1089-1100, 1283-1295):
 * activation {relu|clip|sigmoid|tanh|erf|gelu|exp} with clip_min / clip_max
 * for clip, residual {add|mul} for a second tensor of the output's type and
 * layout.  Order: scale and zero point, bias, residual, activation,
 * narrowing.  Plan switches, all {true|false}, default true:
 * layout_conversion (conversion kernels in front of the vector contraction
 * kernel instead of the element-wise kernel), pointwise_as_gemm (1x1
 * convolutions as a batched GEMM over the tensors as they lie),
 * bwd_weight_gemm (the filter gradient of a one-group convolution as one
 * K-major GEMM plus the reduction of its pixel splits), window_resident (a
 * 16-bit or int8 stride-1 convolution whose tiles fill on the kernel that keeps the
 * input window in LDS, behind a conversion of the filter), split_k (a GEMM,
 * forward convolution or unit-stride input gradient with few output tiles and
 * a long reduction split over blocks, f32 (int8 operands: int32) partial sums
 * in the workspace, a reduction kernel behind the contraction; identity
 * epilogue only), tap_rows (a convolution over pixels of a few channels, without
 * padding or dilation along w, reads a row of filter taps as one run of
 * neighbouring pixels: conversions of both tensors, then a "_runs" kernel),
 * merge_phases (the input gradient of a strided layer whose phases times
 * channels fit 64 output columns: all phases in one convolution over the union
 * of their windows, a conversion kernel puts the positions together),
 * fused (attention, above).  A single leading dash and "key=value"
 * are accepted as well.  rocmlir-gen's scheduling and instruction-set toggles
 * (reverse_grid, mfma, wmma, dot, x2) are accepted and ignored, and so is
 * kernel_name: the code objects are built ahead of time and their kernel
 * symbols are fixed (rockamdGetKernelName tells the symbol to launch); flags that
 * would change the result and have no kernel here are refused: "store-method"
 * other than set (pass the addend as "residual add"), "force-f8-types" other
 * than arch / ocp.  Returns NULL on any parse, validation or support failure,
 * as the reference does. */
ROCMLIR_AMD_API MiirHandle miirCreateHandle(const char *options);

/* Miir.h:56 -- number of kernels the operation needs (1 for most problems; 2
 * for a GEMM or filter gradient split along its reduction; up to 3 for a
 * forward convolution behind layout conversions and for attention run
 * unfused; more for the backward and 3-D convolution plans, see
 * rockamdGetPointerMap); -1 for a NULL handle. */
ROCMLIR_AMD_API int miirGetKernelCount(MiirHandle handle);

/* Miir.h:65 -- workspace bytes shared by the kernels of the problem (0 for
 * single-kernel problems); -1 for a NULL handle or a size beyond int. */
ROCMLIR_AMD_API int miirGetWorkspaceSize(MiirHandle handle);

/* The same as a size_t ((size_t)-1 for a NULL handle): the score workspace of
 * attention run as three kernels can exceed what Miir.h:65's int holds.  No
 * counterpart in the reference. */
ROCMLIR_AMD_API size_t rockamdGetWorkspaceSize64(MiirHandle handle);

/* Miir.h:70 -- resolves the perf config (table lookup); needed before
 * miirGetExecutionDims, as in the reference flow. */
ROCMLIR_AMD_API MiirStatus miirLowerTuningParams(MiirHandle handle);

/* Miir.h:75 -- binds the code object for the selected kernel. */
ROCMLIR_AMD_API MiirStatus miirLowerBin(MiirHandle handle);

/* Miir.h:88 -- two-call protocol: buffer == NULL writes the size, otherwise
 * copies the gfx950 ELF code object into caller memory. */
ROCMLIR_AMD_API MiirStatus miirBufferGet(MiirHandle handle, char *buffer, size_t *size);

/* Miir.h:96 -- 1-D launch: global = grid * block work-items, local = block. */
ROCMLIR_AMD_API MiirStatus miirGetExecutionDims(MiirHandle handle, size_t *global_size,
                                size_t *local_size);

/* Miir.h:101 */
ROCMLIR_AMD_API MiirStatus miirDestroyHandle(MiirHandle handle);

/* ---------------------------------------------------------------------------
 * 2. Kernel description (what mlirGetKernelInfo / mlirGetKernelAttrs /
 *    mlirRockTuning* return in the reference)
 * ------------------------------------------------------------------------- */

/* Kernel symbol inside the code object (mlirGetKernelInfo's name,
 * MIGraphX.cpp:54-90).  Two-call protocol on `size` (includes the NUL). */
ROCMLIR_AMD_API MiirStatus rockamdGetKernelName(MiirHandle handle, char *buffer, size_t *size);

/* {block_size, grid_size} as mlirGetKernelAttrs returns them
 * (MIGraphX.cpp:93-110). */
ROCMLIR_AMD_API MiirStatus rockamdGetKernelAttrs(MiirHandle handle, uint32_t attrs[2]);

/* Kernel argument list: `num_pointers` bare device pointers in op order
 * (GEMM: A, B, C, aux, residual; conv: filter, input, output, aux, residual;
 * attention: Q, K, V, aux, O -- aux is the bias vector / pre-softmax bias
 * tensor, residual the tensor of "--residual"; NULL when unused), followed by
 * ONE by-value parameter block of `*params_size` bytes.  What the CALLER
 * passes to rockamdLaunch can be shorter: a problem without "--residual"
 * passes four pointers and the library fills the fifth with NULL
 * (rockamdGetPointerMap reports it as source -1).
 * Two-call protocol: params == NULL writes the size only.  The reference
 * bakes shapes into the kernel and passes pointers only (Pipelines.cpp:
 * 246-248); this block is the documented extension that replaces that. */
ROCMLIR_AMD_API MiirStatus rockamdGetKernelArgs(MiirHandle handle, int *num_pointers,
                                void *params, size_t *params_size);

/* The caller's pointer list described, one entry per pointer rockamdLaunch
 * takes (index < caller_pointers of rockamdGetPointerMap): element type
 * (RockDType value of kernel_params.h: 0 f32, 1 f16, 2 bf16, 3 i8, 4 fp8,
 * 5 bf8, 6 i32; -1 = bytes, the workspace), rank (<= 6) and dimensions in
 * storage order, outermost first -- what mlirGetKernelInfo reports per
 * argument (MIGraphX.cpp:54-90).  Any of the out-pointers may be NULL. */
ROCMLIR_AMD_API MiirStatus rockamdGetArgumentInfo(MiirHandle handle, int index, int *dtype, int *rank,
                                                  int64_t *dims);

/* The same as one question: bytes[i] is what the caller holds behind pointer i
 * of the list it is about to pass to rockamdLaunch (0 for a pointer it passes
 * as NULL).  MIIR_SUCCESS when every non-empty one is at least as large as the
 * kernel list addresses; otherwise MIIR_INVALID_PARAM with the argument and
 * the two sizes in rockamdGetLastError().  The kernels take bare pointers and
 * cannot check this themselves.  No counterpart in the reference, whose
 * clients pass memrefs that carry their sizes. */
ROCMLIR_AMD_API MiirStatus rockamdCheckArgumentSizes(MiirHandle handle, const size_t *bytes, int num_pointers);

/* perf-config string of the selected kernel in the reference's grammar
 * ("v2:MPB,NPB,KpackPB,MPW,MnPerXdl,Kpack,splitK,forceUnroll,1" or
 * "attn:v1:...", RockAttrDefs.td:241-329).  Copies what fits, always
 * terminates the buffer and returns the full length like
 * mlirRockTuningParamToString (Rock.h:60-75). */
ROCMLIR_AMD_API size_t rockamdGetPerfConfig(MiirHandle handle, char *buffer, size_t buffer_size);

/* Tuning problem key, "<arch>\t<numCU>\t<problem>" in the reference's format
 * (RockTuningImpl.cpp:550-871; mlirRockTuningGetKey, Rock.h:120-130).
 * Returns the full length, or (size_t)-1 on failure. */
ROCMLIR_AMD_API size_t rockamdGetProblemKey(MiirHandle handle, char *buffer, size_t buffer_size);

/* Multi-kernel problems.  As in the reference (rocmlir-lib.cpp:150-199: one
 * handle per "--kernel_id i", i < miirGetKernelCount, all kernels sharing
 * miirGetWorkspaceSize bytes of scratch), a problem may lower to several
 * kernels: a convolution whose filter or input is not channel-contiguous
 * (gkcyx / ngchw, the reference's default layouts) is run as one layout-
 * conversion kernel per such tensor followed by the vector contraction kernel
 * ("--layout_conversion false" keeps the single element-wise kernel).  Every
 * kernel of the problem is launched, in kernel_id order on one stream, with
 * the SAME caller list: the problem's pointers followed by the workspace
 * pointer.  This call says how many pointers the caller list has, how many
 * the kernel itself takes, and for each of those which caller pointer it is
 * (source[i]) plus a byte offset; rockamdLaunch applies the map itself.
 * source[i] == -1 means NULL (the residual slot of a problem without one).
 * With "--residual" the caller list is A, B, C, aux, residual[, workspace].
 * A convolution with a 1x1 filter, unit stride, no padding, one group and no
 * bias over NCHW tensors needs no conversion: it runs as ONE batched GEMM
 * kernel (filter x image, the image stored K-major). */
ROCMLIR_AMD_API MiirStatus rockamdGetPointerMap(MiirHandle handle, int *caller_pointers, int *kernel_pointers,
                                                int32_t *source, int64_t *offset);

/* Per-channel (broadcast-vector) quantisation, the form the reference lowers when the scale and zero point
 * of migraphx.dequantizelinear / quantizelinear are tensors with one value per output channel
 * (MIGraphXToTosa.cpp:874-982; mlir/test/fusion/resnet50-e2e/mixr-resnet-fusion-case-1-quantization.mlir:8-9).
 * GEMM and forward 2-D convolution take the options "--scale_vector true", "--zero_point_vector i32|i8",
 * "--quant_scale_vector true", "--out_zero_point_vector i32|i8": element n of the vector replaces the scalar
 * of the same name for output channel n (GEMM: column n of C; convolution: channel g * K + k).  The vectors
 * are further tensors of the CALLER list, in the order above, behind the problem's own pointers (A, B, C,
 * aux[, residual]) and in front of the workspace.  They are not kernel pointers: the contraction kernel reads
 * their addresses from pointer fields of its parameter block.  For a client that launches the code object
 * itself this call lists, for the handle's kernel, the byte offset inside the parameter block
 * (rockamdGetKernelArgs) at which caller pointer source[i] has to be written before the launch; *count is 0
 * for kernels that read no vector (the other kernels of a plan, every problem without vectors).  Either
 * array may be NULL; at most four entries. */
ROCMLIR_AMD_API MiirStatus rockamdGetParamPointers(MiirHandle handle, int *count, int32_t *param_offset,
                                                   int32_t *source);

/* Epilogue scalars can be changed after creation (they live in the by-value
 * parameter block; fetch it again after a change).  Formulas:
 * MIGraphXToTosa.cpp:874-982.  No counterpart entry point in the reference,
 * where these are IR constants. */
ROCMLIR_AMD_API MiirStatus rockamdSetScale(MiirHandle handle, float scale);
ROCMLIR_AMD_API MiirStatus rockamdSetZeroPoint(MiirHandle handle, int32_t zero_point);

/* ---------------------------------------------------------------------------
 * 2b. Tuning surface (mlir-c/Dialect/Rock.h:39-148; implementation
 *     mlir/lib/Dialect/Rock/Tuning/RockTuningImpl.cpp:461-548,902-1015).
 *     The reference enumerates a grid of block/wave tile sizes; here the
 *     space of a problem is the list of hand-written kernels it can run on,
 *     each named by a perf_config string in the reference's "v2:" grammar.
 * ------------------------------------------------------------------------- */
typedef void *RockamdTuningSpace;
typedef void *RockamdTuningTable;

/* RocmlirTuningParamSetKind (RockEnums.h:19-23).  Quick: the built-in table's
 * choice and its two likeliest alternatives; Full: one entry per kernel the
 * problem can run on; Exhaustive: Full, and every tile once more as its twin
 * with the rolled epilogue (eighth field, forceUnroll, 0). */
enum { ROCKAMD_TUNING_QUICK = 0, ROCKAMD_TUNING_FULL = 1, ROCKAMD_TUNING_EXHAUSTIVE = 2 };
/* RocmlirSplitKSelectionLikelihood (RockEnums.h:26) */
enum { ROCKAMD_SPLITK_NEVER = 0, ROCKAMD_SPLITK_MAYBE = 1, ROCKAMD_SPLITK_ALWAYS = 2 };

/* mlirRockTuningSpaceCreate / mlirRockTuningGetNumParams /
 * mlirRockTuningParamGet + mlirRockTuningParamToString / mlirRockTuningSpaceDestroy
 * (Rock.h:39-84).  Entry 0 is the kernel the built-in table picks.  GEMM and
 * convolution entries are "v2:" strings, attention entries "attn:v1:" strings
 * (RockAttrDefs.td:241-329); both are accepted back by "--perf_config" and
 * rockamdTuningSetFromStr.  ToString copies what fits, always terminates the
 * buffer and returns the full length ((size_t)-1 for a bad position): a
 * result >= buffer_size means the text was cut. */
ROCMLIR_AMD_API RockamdTuningSpace rockamdTuningSpaceCreate(MiirHandle handle, int kind);
ROCMLIR_AMD_API unsigned rockamdTuningGetNumParams(RockamdTuningSpace space);
ROCMLIR_AMD_API size_t rockamdTuningParamToString(RockamdTuningSpace space, unsigned pos, char *buffer,
                                                  size_t buffer_size);
ROCMLIR_AMD_API void rockamdTuningSpaceDestroy(RockamdTuningSpace space);

/* mlirRockTuningSetFromStr (Rock.h:90-92): re-resolves the handle's kernel
 * under the given perf_config; a string that names no applicable kernel falls
 * back to the table (AffixTuningParameters.cpp:129-141).  Returns 1 on
 * success; fetch the code object, launch dimensions and parameter block again. */
ROCMLIR_AMD_API int rockamdTuningSetFromStr(MiirHandle handle, const char *perf_config);

/* mlirRockTuningTableCreate / Destroy / mlirRockTuningUpdateTable /
 * mlirRockTuningSetFromTable (Rock.h:94-117): an in-memory map from problem
 * key (rockamdGetProblemKey) to the best perf_config seen.  Update returns 1
 * if the entry was stored, 0 if a better-performing one exists; SetFromTable
 * returns 1 if the problem was found and applied. */
ROCMLIR_AMD_API RockamdTuningTable rockamdTuningTableCreate(void);
ROCMLIR_AMD_API void rockamdTuningTableDestroy(RockamdTuningTable table);
ROCMLIR_AMD_API int rockamdTuningUpdateTable(RockamdTuningTable table, const char *problem_key,
                                             const char *perf_config, float time);
ROCMLIR_AMD_API int rockamdTuningSetFromTable(RockamdTuningTable table, MiirHandle handle);

/* mlirIsModuleFusible (Rock.h:145-147, RockTuningImpl.cpp:1010-1015): may the
 * handle's element-wise tail (scale, bias, residual, activation) stay fused
 * when the problem runs under `perf_config`?  The reference says no when the
 * string asks for a split reduction, whose partial sums meet through atomic
 * adds; here a requested split sums its partial tiles inside the block before
 * the epilogue, so the answer is 1 for every string the problem resolves
 * under and 0 only for a NULL handle or string. */
ROCMLIR_AMD_API int rockamdIsFusible(MiirHandle handle, const char *perf_config);

/* mlirGetNumPrefillArgs / mlirGetPrefillArgsInfo (Rock.h:149-158): arguments
 * whose memory must hold an initial value before the launch.  The reference
 * needs a zero-filled output for its atomic split-K; no kernel of this
 * library accumulates into memory it has not written (split reductions go
 * through a workspace and a reduction kernel, the zero fill of the strided
 * backward-data phases is a kernel of the problem's own list), so the count
 * is 0 and the info call writes nothing. */
ROCMLIR_AMD_API size_t rockamdGetNumPrefillArgs(MiirHandle handle);
ROCMLIR_AMD_API void rockamdGetPrefillArgsInfo(MiirHandle handle, size_t *indices, float *init_values,
                                               size_t length);

/* mlirIsSplitKFaster (Rock.h:136-142, RockTuningImpl.cpp:962-1008), answered
 * for this library's split-K kernel (K divided over the waves of one block):
 * ALWAYS when the built-in table itself would choose it (64x64 tiles would
 * occupy at most half the CUs and K is at least 1 KiB), MAYBE while the tile
 * count does not exceed the CUs, NEVER otherwise.  element_size in bytes. */
ROCMLIR_AMD_API int rockamdIsSplitKFaster(int64_t g, int64_t m, int64_t n, int64_t k, int64_t num_cu,
                                          int element_size);

/* ---------------------------------------------------------------------------
 * 3. Launch helpers (the client side of rocmlir-tuning-driver.cpp:131-185)
 * ------------------------------------------------------------------------- */

/* Loads the handle's code object on the current device (cached) and enqueues
 * one launch on `stream` (a hipStream_t, NULL = default stream).  `pointers`
 * holds exactly the pointer arguments described above.  Returns 0 or a
 * hipError_t value; never synchronises. */
ROCMLIR_AMD_API int rockamdLaunch(MiirHandle handle, void *const *pointers, int num_pointers,
                  void *stream);

/* rockamdLaunch for callers that cannot allocate device memory: code under HIP
 * graph capture, serving loops and harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  A problem of several kernels
 * (miirGetKernelCount > 1) passes intermediate results through a workspace
 * that rockamdLaunch's caller allocates and passes last; this entry point
 * takes the problem's own pointers only (one fewer than rockamdLaunch when the
 * problem has a workspace) and uses an array of
 * ROCKAMD_STATIC_WORKSPACE_BYTES bytes in the library's own device image
 * instead.  It calls no allocating routine, except that the first call for a
 * handle on a device loads the handle's code object and resolves the array's
 * address: make that call outside a capture.  A problem whose workspace is
 * larger fails with hipErrorInvalidValue and a message in
 * rockamdGetLastError; nothing is launched.  Each GPU holds one such array
 * until the process ends and all calls on that GPU share it: launch the
 * kernels of one problem in kernel_id order on one stream, and do not let two
 * problems with workspaces overlap in time on one GPU (they race on it).  A
 * problem without a workspace behaves exactly as under rockamdLaunch. */
#define ROCKAMD_STATIC_WORKSPACE_BYTES ((size_t)64 << 20)
ROCMLIR_AMD_API int rockamdLaunchStaticWorkspace(MiirHandle handle, void *const *pointers, int num_pointers,
                                                 void *stream);

/* (The measurement helpers -- rockamdBenchmark, rockamdMeasureMfmaRate -- are declared in rocmlir_amd_bench.h.) */

/* Text of the last failure on the calling thread ("" if none). */
ROCMLIR_AMD_API const char *rockamdGetLastError(void);

#ifdef __cplusplus
}
#endif
#endif /* ROCMLIR_AMD_H */
