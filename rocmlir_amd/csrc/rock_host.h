// Internal declarations of librocmlir_amd.so's host side, shared by its
// translation units (none of this is exported; the C ABI is include/rocmlir_amd.h).
//
// The host side does problem-string parsing and validation, keeps the perf-config table and the problem keys,
// hands out code objects and launches them.  It stands where the reference has ConvGenerator::parseConvConfig /
// isApplicable (mlir/lib/Dialect/Rock/Generator/ConvGenerator.cpp:136-248,
// 487-749), the op verifiers (mlir/lib/Dialect/Rock/IR/RockDialect.cpp:509-568,
// 808-893,2071-2106), the tuning heuristics and problem keys
// (mlir/lib/Dialect/Rock/Tuning/GridwiseGemmParams.cpp, RockTuningImpl.cpp:
// 550-871) and the Miir entry points (mlir/tools/rocmlir-lib/rocmlir-lib.cpp:
// 117-316).  There is no compiler behind it: kernels are hand-written HIP,
// compiled ahead of time for gfx950 and embedded in this library.
#pragma once

#include "../../include/rocmlir_amd.h"
#include "kernel_params.h"
#include "rock_internal.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

namespace rockhost {

// ---- error text (per thread): rock_options.cpp --------------------------------
extern thread_local std::string g_last_error;
void set_error(const std::string &msg);

// ---- embedded code objects: rock_options.cpp -----------------------------------
struct Blob {
  const char *name; // the kernel's symbol
  const char *start;
  const char *end;
};
const Blob *find_blob(const std::string &kernel_name);

// ---- option strings: rock_options.cpp --------------------------------------------
using OptMap = std::map<std::string, std::string>;
bool parse_options(const char *text, OptMap &out);
bool get_int(const OptMap &m, const std::string &k, int64_t &v);
int64_t int_or(const OptMap &m, const std::string &k, int64_t dflt);
bool bool_or(const OptMap &m, const std::string &k, bool dflt);
bool get_float(const OptMap &m, const std::string &k, float &v);
std::string str_or(const OptMap &m, const std::string &k, const std::string &d);

// ---- route switches ---------------------------------------------------------------
// Every plan beyond "one kernel reads the tensors where they lie" can be switched off by the caller, by the
// tuner (to time a problem both ways) or by a test (to reach the plain kernel): one option each, all on by
// default, read in one place.  The reference has no such switches -- its generated kernel is the only route;
// the nearest thing is the splitK field of its perf_config, which requested_block_splits() reads.
struct RoutePolicy {
  bool layout_conversion; // conversion kernels in front of / behind a contraction (padded or re-laid-out copies)
  bool split_k;           // a long reduction divided over blocks, partial sums added by a reduction kernel
  bool window_resident;   // 3x3-style forward convolutions on the kernel that keeps the input window in LDS
  bool pointwise_as_gemm; // 1x1 unit-stride convolutions run as plain GEMMs
  bool merge_phases;      // strided input gradient: the stride phases in one convolution
  bool bwd_weight_gemm;   // filter gradient as a GEMM over channels-last copies
  bool tap_rows;          // few-channel first layers over rows of taps
  bool fused;             // attention on the fused kernels (off: GEMM, row softmax, GEMM)
  int64_t score_workspace_limit; // bytes of attention scores per chunk of the three-kernel form; 0: the default
  explicit RoutePolicy(const OptMap &o);
};

// ---- element types ----------------------------------------------------------------
int parse_dtype(std::string s);
const char *dtype_name(int t);
int dtype_size(int t);
bool is_float_in(int t);
int operand_code(int a, int b);
const char *operand_name(int code);

// --------------------------------------------------------------------------
// tile variants: the "small perf-config table"
// --------------------------------------------------------------------------
struct Tile {
  const char *suffix; // kernel name suffix
  int bm, bn, waves_m, waves_n;
  int blocks_per_cu;  // co-resident blocks (LDS bound)
  float efficiency;   // relative per-tile MFMA efficiency used by the heuristic
  bool gemm, conv;
};
inline const Tile kFastTiles[] = {
    // efficiencies: measured f16 4096^3 throughput of each tile relative to 256x256
    {"_256x256_fast", 256, 256, 2, 4, 1, 1.00f, true, false},
    {"_256x128_fast", 256, 128, 4, 2, 1, 0.82f, true, true},
    {"_128x128_fast", 128, 128, 2, 2, 2, 0.75f, true, true},
    {"_64x64_fast", 64, 64, 2, 2, 4, 0.46f, true, true},
};
inline const Tile kGenericTile = {"_64x64_generic", 64, 64, 2, 2, 4, 0.1f, true, true};
// 32x32 output tile, K split over the four waves of the block (GEMM fast path only)
inline const Tile kSplitKTile = {"_32x32_splitk", 32, 32, 1, 4, 2, 0.3f, true, false};
constexpr int kNumCU = 256; // MI355X
constexpr int kDirectTilePixels = 224;          // conv_direct.h: 7 blocks of 32 output pixels
constexpr int64_t kDirectWindowBytes = 80 * 1024; // conv_direct.h: the window's share of LDS (two blocks per CU)
constexpr int kNumXCD = 8;

inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }
inline int64_t align256(int64_t bytes) { return (bytes + 255) / 256 * 256; }
inline int64_t floor_div(int64_t a, int64_t b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

// --------------------------------------------------------------------------
// problems
// --------------------------------------------------------------------------
enum OpKind { OP_GEMM, OP_CONV, OP_ATTENTION, OP_RELAYOUT };

struct Handle {
  OpKind op;
  std::string arch = "gfx950";
  int num_cu = kNumCU;
  int kernel_id = 0;
  // resolved kernel
  std::string kernel_name;
  const Blob *blob = nullptr;
  uint32_t block_size = 0, grid_size = 0;
  int num_pointers = 0;
  std::vector<char> params; // by-value parameter block
  std::string perf_config;
  std::string problem_key;
  bool tuned = false, lowered = false;
  bool moved_for_scale_sign = false; // attention: rockamdSetScale took the handle off the plain fused kernel
  OptMap options; // the parsed problem, kept so that a perf_config can be applied later
  // multi-kernel problems (layout conversion + contraction): every kernel of
  // the problem is launched with the same caller pointer list, the problem's
  // tensors followed by one workspace pointer; ptr_map says where each of
  // THIS kernel's pointers comes from.  Single-kernel problems: identity.
  int kernel_count = 1;
  size_t workspace_bytes = 0;
  int caller_pointers = 0; // 0 = same as num_pointers
  struct PtrSrc {
    int source;     // index into the caller's list
    int64_t offset; // bytes added to it
  };
  std::vector<PtrSrc> ptr_map;
  // the caller's pointer list described: element type (RockDType, -1 = bytes)
  // and dimensions in storage order, outermost first
  struct ArgInfo {
    int dtype;
    std::vector<int64_t> dims;
  };
  std::vector<ArgInfo> args;
  // Pointers that ride INSIDE the parameter block (the per-channel quantisation vectors of RockEpilogue):
  // at launch the caller pointer `source` is written at byte `offset` of the block
  struct ParamPtr {
    int offset, source;
  };
  std::vector<ParamPtr> param_ptrs;
  // typed views of `params`
  RockEpilogue *epi = nullptr;
  // launch cache: device -> function
  std::map<int, hipFunction_t> functions;
};

// ---- epilogue and perf_config grammar: rock_options.cpp ------------------------------
bool parse_epilogue(const OptMap &o, int in_a, int out_dtype, RockEpilogue &e);
int channel_vector_flags(const OptMap &o);
void default_epilogue(RockEpilogue &e, int out_dtype);
int64_t perf_field(const OptMap &o, int index, int64_t dflt);
std::string perf_string(const Tile &t, int es, const OptMap *o = nullptr);
std::string forced_tile(const OptMap &o);
bool requested_tile_is(const OptMap &o, int bm, int bn);
int64_t requested_block_splits(const OptMap &o);
std::string with_block_splits(const std::string &pc, int64_t S);

// ---- GEMM planning: plan_gemm.cpp ------------------------------------------------------
const Tile *pick_tile(int64_t M, int64_t N, int G, bool conv, const std::string &force, bool k_major = false);
void apply_tile_grid(const Tile &t, int64_t M, int64_t N, int G, int &tiles_m, int &tiles_n, int &group_m,
                     int &xcd_remap, uint32_t &block, uint32_t &grid);
const char *rich_suffix(const RockEpilogue &e, bool tiled_kernel, const OptMap &o);
void set_contraction_pointers(Handle *h, const RockEpilogue &e);
bool plan_gemm_kernel(Handle *h, RockGemmParams &p, int code, int es, const OptMap &o, bool k_padded = false);
Handle *make_gemm(const OptMap &o);

// ---- conversion and utility kernels: plan_relayout.cpp -------------------------------------
RockFastDiv fast_div_of(int64_t d);
bool fill_relayout_handle(Handle *h, const int64_t size[5], const int64_t src_size[5],
                          const int64_t src_stride[5], int es, const int64_t *dst_stride = nullptr);
Handle *utility_fill_handle(int64_t bytes);
// A conversion kernel between two views of one tensor of more than five
// dimensions, listed in the destination's order (the last one contiguous
// there): unit dimensions go, neighbours that lie back to back on both sides
// fold, and what is left has to fit the kernel's five.
struct ViewDim { int64_t size, src_size, ss, ds; };
bool relayout_handle_nd(Handle *h, std::vector<ViewDim> dims, int es, const char *what);

// ---- convolution planning: plan_conv.cpp, plan_conv_bwd_data.cpp, plan_conv_bwd_weight.cpp, plan_conv3d.cpp ----
bool canon_layout(std::string s, char channel, const char *want, std::string &out);
void layout_strides(const std::string &layout, const std::string &letters, const int64_t *sizes, int64_t *strides);
std::string key_layout(const std::string &layout, bool filter);
// a 2-D convolution as its option list poses it, every direction
struct ConvProblem {
  int ti; // element type of all three tensors
  std::string fl, il, ol;
  int64_t n, g, c, k, hi, wi, y, x, ho, wo, sh, sw, ph, pw, dh, dw; // ph, pw: the top / left padding
  // bottom / right padding: it only enters through ho and wo (the kernels treat every read outside the tensor as
  // zero), but the routes that read the tensors "as they lie" need both sides to be zero
  int64_t ph_r = 0, pw_r = 0;
  bool unpadded() const { return ph == 0 && pw == 0 && ph_r == 0 && pw_r == 0; }
  int64_t fs[5], is[5], os[5]; // element strides in letter order gkcyx / ngchw / ngkhw
  // filter gradient only: the output gradient is a copy whose k channels were padded with zeros up to a whole
  // 16-byte chunk; only the first k_valid rows of the gradient exist in the caller's tensor (0: all k)
  int64_t k_valid = 0;
};
bool conv_view_fast(const RockConvParams &q, int es);
bool select_view_conv_kernel(Handle *h, RockConvParams &p, int ti, const OptMap &o);
std::string conv_problem_key(const Handle *h, const OptMap &o, const ConvProblem &cp, int direction);
Handle *conv_handle_from_view(const RockConvParams &q, int ti, const OptMap &o);
// The window-resident kernel (conv_direct.h) on a convolution given as a view
// (p: sizes, strides of input and output, unit stride and dilation assumed
// checked here).  It needs: a filter of more than one tap, equal padding on
// both sides (the caller says so), a channel run that is a power of two of
// 128..1024 bytes, whole 32-channel blocks of output channels, output rows
// that fit the tile's pixels, and a window of TH + Y - 1 padded rows (Y - 1
// more when tiles straddle two images) within 80 KiB of LDS.  The filter
// reaches it repacked (fragment-major, every group padded to whole 128-channel
// tiles): `filter_bytes` of workspace.
struct WindowPlan {
  bool ok = false, by_itself = false;
  int64_t rows = 0, tiles_n = 0, filter_bytes = 0;
};
WindowPlan window_plan(const RockConvParams &p, int ti, bool equal_padding, const OptMap &o);
void apply_window_plan(Handle *h, RockConvParams &p, const WindowPlan &w, int ti, const OptMap &o);
Handle *make_conv(const OptMap &o);
Handle *make_conv_bwd_data(const OptMap &o, const ConvProblem &cp);
Handle *make_conv_bwd_weight(const OptMap &o, const ConvProblem &cp);
bool canon_layout3(std::string s, char channel, bool filter, std::string &out);
Handle *make_conv3d(const OptMap &o);

// ---- attention planning: plan_attention.cpp ---------------------------------------------------
// "attn:v1:MPB_G0,MPB_G1,NPB_G0,KpackPB,MPW,MnPerXdl,Kpack,forceUnroll"
// (RockAttrDefs.td:241-329; G0 M tiles seq_k, G1 M the head dimension, G0 N
// seq_q).  The hand-written kernels all take 64 keys x 128 queries per step;
// what a string selects is the head-dimension instantiation (MPB_G1 = 64 or
// 128), the element-wise kernel (KpackPB = 1) and, through forceUnroll, the
// order of work inside a key tile: 1 = the next tile's score MFMAs are issued
// ahead of this tile's softmax (only without bias / scale tensor and with a
// non-negative scale), 0 = scores, softmax, PV per tile.
struct AttnVariant {
  const char *kind; // kernel-name suffix
  int kpack_pb, force_unroll;
};
inline const AttnVariant kAttnVariants[] = {{"fast", 8, 1}, {"fast_bias", 8, 0}, {"generic", 1, 1}};
std::string attn_perf_string(const AttnVariant &v, int dmax);
bool parse_attn_perf(const std::string &pc, int &dmax, int &kpack_pb, int &force_unroll);
Handle *make_attention(const OptMap &o);

// ---- handles and tuning: rock_handle.cpp ---------------------------------------------------------
Handle *build_handle(const OptMap &o);
std::vector<std::string> tuning_candidates(const Handle &h, int kind);
struct TuningSpace {
  std::vector<std::string> params;
};

// problem key -> best perf_config seen and its time (mlirRockTuningUpdateTable keeps only the best)
struct TuningTable {
  std::map<std::string, std::pair<std::string, float>> best;
  std::mutex mutex; // several tuning threads may share one table (RockTuningImpl.cpp:902-931 takes a RW lock)
};

// ---- launching: rock_launch.cpp ----------------------------------------------------------------------
int load_module(const Blob *blob, hipModule_t *module); // one hipModule per (device, code object)
int get_function(Handle *h, hipFunction_t *fn);
int launch_once(Handle *h, hipFunction_t fn, void *const *pointers, hipStream_t stream);
bool check_launch_args(Handle *h, void *const *pointers, int num_pointers);

} // namespace rockhost
