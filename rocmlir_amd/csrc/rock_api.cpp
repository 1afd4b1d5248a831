// Host side of librocmlir_amd.so: problem-string parsing and validation,
// perf-config table, problem keys, code-object hand-out and a launch helper.
//
// It stands where the reference has ConvGenerator::parseConvConfig /
// isApplicable (mlir/lib/Dialect/Rock/Generator/ConvGenerator.cpp:136-248,
// 487-749), the op verifiers (mlir/lib/Dialect/Rock/IR/RockDialect.cpp:509-568,
// 808-893,2071-2106), the tuning heuristics and problem keys
// (mlir/lib/Dialect/Rock/Tuning/GridwiseGemmParams.cpp, RockTuningImpl.cpp:
// 550-871) and the Miir entry points (mlir/tools/rocmlir-lib/rocmlir-lib.cpp:
// 117-316).  There is no compiler behind it: kernels are hand-written HIP,
// compiled ahead of time for gfx950 and embedded in this library.
#include "../../include/rocmlir_amd.h"
#include "kernel_params.h"
#include "rock_internal.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

namespace {

// --------------------------------------------------------------------------
// error text (per thread)
// --------------------------------------------------------------------------
thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }

// --------------------------------------------------------------------------
// embedded gfx950 code objects, one per kernel and named after it (blobs.S;
// blobs.inc is the list the build generates).  The reference hands out one
// kernel per code object (rocmlir-lib.cpp:292-316); so does miirBufferGet.
// --------------------------------------------------------------------------
#define ROCK_BLOB(n)                                                           \
  extern "C" const char rock_hsaco_##n##_start[];                              \
  extern "C" const char rock_hsaco_##n##_end[];
#include "blobs.inc"
#undef ROCK_BLOB

struct Blob {
  const char *name; // the kernel's symbol
  const char *start;
  const char *end;
};
const Blob kBlobs[] = {
#define ROCK_BLOB(n) {#n, rock_hsaco_##n##_start, rock_hsaco_##n##_end},
#include "blobs.inc"
#undef ROCK_BLOB
};

const Blob *find_blob(const std::string &kernel_name) {
  static const std::map<std::string, const Blob *> index = [] {
    std::map<std::string, const Blob *> m;
    for (const Blob &b : kBlobs)
      m[b.name] = &b;
    return m;
  }();
  auto it = index.find(kernel_name);
  return it == index.end() ? nullptr : it->second;
}

// --------------------------------------------------------------------------
// option parsing: "--key value", "-key value", "--key=value"
// (ConvGenerator.cpp:82-98 tokeniser, widened to rocmlir-gen's spellings)
// --------------------------------------------------------------------------
using OptMap = std::map<std::string, std::string>;

bool parse_options(const char *text, OptMap &out) {
  if (!text)
    return false;
  std::istringstream iss(text);
  std::string tok, key;
  while (iss >> tok) {
    bool is_key = tok.size() > 1 && tok[0] == '-' &&
                  !(std::isdigit((unsigned char)tok[1]) || tok[1] == '.');
    if (is_key) {
      if (!key.empty())
        out[key] = "true"; // flag without a value
      size_t p = tok.find_first_not_of('-');
      if (p == std::string::npos)
        return false;
      key = tok.substr(p);
      size_t eq = key.find('=');
      if (eq != std::string::npos) {
        out[key.substr(0, eq)] = key.substr(eq + 1);
        key.clear();
      }
    } else {
      if (key.empty())
        continue; // stray value: ignored as the reference does
      out[key] = tok;
      key.clear();
    }
  }
  if (!key.empty())
    out[key] = "true";
  return true;
}

bool get_int(const OptMap &m, const std::string &k, int64_t &v) {
  auto it = m.find(k);
  if (it == m.end())
    return false;
  char *end = nullptr;
  long long r = std::strtoll(it->second.c_str(), &end, 10);
  if (end == it->second.c_str() || *end != '\0')
    return false;
  v = r;
  return true;
}
int64_t int_or(const OptMap &m, const std::string &k, int64_t dflt) {
  int64_t v;
  return get_int(m, k, v) ? v : dflt;
}
bool bool_or(const OptMap &m, const std::string &k, bool dflt) {
  auto it = m.find(k);
  if (it == m.end())
    return dflt;
  const std::string &s = it->second;
  return s == "true" || s == "1" || s == "True";
}
bool get_float(const OptMap &m, const std::string &k, float &v) {
  auto it = m.find(k);
  if (it == m.end())
    return false;
  char *end = nullptr;
  double r = std::strtod(it->second.c_str(), &end);
  if (end == it->second.c_str() || *end != '\0')
    return false;
  v = (float)r;
  return true;
}
std::string str_or(const OptMap &m, const std::string &k, const std::string &d) {
  auto it = m.find(k);
  return it == m.end() ? d : it->second;
}

// --------------------------------------------------------------------------
// element types
// --------------------------------------------------------------------------
int parse_dtype(std::string s) {
  // Miir spellings (ConvGenerator.cpp:569-590) and MLIR names; on gfx950 the
  // short 8-bit float names mean the OCP formats (rocmlir-gen.cpp:3709-3729).
  if (s == "f32" || s == "fp32") return ROCK_F32;
  if (s == "f16" || s == "fp16") return ROCK_F16;
  if (s == "bf16") return ROCK_BF16;
  if (s == "i8" || s == "int8") return ROCK_I8;
  if (s == "fp8" || s == "f8E4M3FN") return ROCK_FP8;
  if (s == "bf8" || s == "f8E5M2") return ROCK_BF8;
  if (s == "i32" || s == "int32") return ROCK_I32;
  return -1;
}
const char *dtype_name(int t) {
  static const char *n[] = {"f32", "f16", "bf16", "i8", "fp8", "bf8", "i32"};
  return (t >= 0 && t < ROCK_DTYPE_COUNT) ? n[t] : "?";
}
int dtype_size(int t) {
  switch (t) {
  case ROCK_F32: case ROCK_I32: return 4;
  case ROCK_F16: case ROCK_BF16: return 2;
  default: return 1;
  }
}
bool is_float_in(int t) { return t != ROCK_I8 && t != ROCK_I32; }

// internal operand-pair code (mfma_gfx950.h): the public codes plus the two
// mixed 8-bit float pairs; -1 if the pair has no kernel
int operand_code(int a, int b) {
  if (a == b && a != ROCK_I32)
    return a;
  if (a == ROCK_FP8 && b == ROCK_BF8) return 7;
  if (a == ROCK_BF8 && b == ROCK_FP8) return 8;
  return -1;
}
const char *operand_name(int code) {
  static const char *n[] = {"f32", "f16", "bf16", "i8", "fp8", "bf8", "", "fp8_bf8", "bf8_fp8"};
  return n[code];
}

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
const Tile kFastTiles[] = {
    // efficiencies: measured f16 4096^3 throughput of each tile relative to 256x256
    {"_256x256_fast", 256, 256, 2, 4, 1, 1.00f, true, false},
    {"_256x128_fast", 256, 128, 4, 2, 1, 0.82f, true, true},
    {"_128x128_fast", 128, 128, 2, 2, 2, 0.75f, true, true},
    {"_64x64_fast", 64, 64, 2, 2, 4, 0.46f, true, true},
};
const Tile kGenericTile = {"_64x64_generic", 64, 64, 2, 2, 4, 0.1f, true, true};
// 32x32 output tile, K split over the four waves of the block (GEMM fast path only)
const Tile kSplitKTile = {"_32x32_splitk", 32, 32, 1, 4, 2, 0.3f, true, false};
constexpr int kNumCU = 256; // MI355X
constexpr int kDirectTilePixels = 224;          // conv_direct.h: 7 blocks of 32 output pixels
constexpr int64_t kDirectWindowBytes = 80 * 1024; // conv_direct.h: the window's share of LDS (two blocks per CU)
constexpr int kNumXCD = 8;

int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

// pick the tile that minimises rounds * tile_area / efficiency
// `k_major`: the problem has a K-major operand; those kernels exist for the square tiles only
const Tile *pick_tile(int64_t M, int64_t N, int G, bool conv, const std::string &force, bool k_major = false) {
  const Tile *best = nullptr;
  double best_cost = 0;
  for (const Tile &t : kFastTiles) {
    if (conv ? !t.conv : !t.gemm)
      continue;
    if (k_major && t.bm != t.bn)
      continue;
    if (!force.empty()) {
      if (force == std::to_string(t.bm) + "x" + std::to_string(t.bn))
        return &t;
      continue;
    }
    int64_t tiles = (int64_t)ceil_div(M, t.bm) * ceil_div(N, t.bn) * G;
    // co-resident blocks share one CU's matrix cores, so what counts is the
    // largest number of tiles any CU has to work through
    int64_t per_cu = (tiles + kNumCU - 1) / kNumCU;
    // The 256x128 tile's figure comes from GEMMs.  As an implicit-GEMM
    // convolution tile it lost to 128x128 on every problem of the reference's
    // convolution list where this model had preferred it (13 of 40, by 4-30 %):
    // one resident block per CU leaves the im2col address work of its loader
    // waves with nothing to hide behind.
    const double efficiency = (conv && t.bm == 256) ? 0.62 : t.efficiency;
    double cost = (double)per_cu * t.bm * t.bn / efficiency;
    // a compute unit with a single four-wave block resident (one wave per
    // SIMD) cannot keep its matrix pipes busy: nothing overlaps a wave's LDS
    // reads and barriers
    const int64_t resident = std::min<int64_t>(per_cu, t.blocks_per_cu);
    if (resident * t.waves_m * t.waves_n < 8)
      cost /= 0.7;
    if (!best || cost < best_cost) {
      best = &t;
      best_cost = cost;
    }
  }
  return best;
}

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

bool parse_epilogue(const OptMap &o, int in_a, int out_dtype, RockEpilogue &e) {
  e.scale = 1.0f;
  e.inv_quant_scale = 1.0f;
  e.zero_point = 0;
  e.out_zero_point = 0;
  e.has_bias = bool_or(o, "bias", false) ? 1 : 0;
  e.out_dtype = out_dtype;
  // element-wise tail: "-activation relu|clip|sigmoid|tanh|erf|gelu|exp"
  // ("-relu true" is the older spelling), "-clip_min/-clip_max" for clip,
  // "-residual add|mul" for a second tensor shaped like the output
  e.activation = bool_or(o, "relu", false) ? ROCK_ACT_RELU : ROCK_ACT_NONE;
  e.act_lo = 0.0f;
  e.act_hi = 0.0f;
  {
    static const std::pair<const char *, int> kActs[] = {
        {"none", ROCK_ACT_NONE}, {"relu", ROCK_ACT_RELU}, {"clip", ROCK_ACT_CLIP}, {"sigmoid", ROCK_ACT_SIGMOID},
        {"tanh", ROCK_ACT_TANH}, {"erf", ROCK_ACT_ERF},   {"gelu", ROCK_ACT_GELU}, {"exp", ROCK_ACT_EXP}};
    const std::string act = str_or(o, "activation", "");
    bool known = act.empty();
    for (const auto &a : kActs)
      if (act == a.first) {
        e.activation = a.second;
        known = true;
      }
    if (!known)
      return false;
    e.act_lo = -INFINITY;
    e.act_hi = INFINITY;
    if (e.activation == ROCK_ACT_RELU)
      e.act_lo = 0.0f;
    if (e.activation == ROCK_ACT_CLIP) {
      if (!get_float(o, "clip_min", e.act_lo) || !get_float(o, "clip_max", e.act_hi) || e.act_lo > e.act_hi)
        return false;
    }
    const std::string res = str_or(o, "residual", "none");
    if (res != "none" && res != "add" && res != "mul")
      return false;
    e.residual_op = res == "add" ? ROCK_RES_ADD : res == "mul" ? ROCK_RES_MUL : ROCK_RES_NONE;
    // integers leaving as integers take no float step
    if (out_dtype == ROCK_I32 && e.activation != ROCK_ACT_NONE)
      return false;
  }
  get_float(o, "scale", e.scale);
  float qs;
  if (get_float(o, "quant_scale", qs)) {
    if (qs == 0.0f)
      return false;
    e.inv_quant_scale = 1.0f / qs;
  }
  e.zero_point = (int32_t)int_or(o, "zero_point", 0);
  e.out_zero_point = (int32_t)int_or(o, "out_zero_point", 0);
  // Per-channel vectors in place of the four scalars above: "-scale_vector true", "-zero_point_vector i32|i8",
  // "-quant_scale_vector true", "-out_zero_point_vector i32|i8" (one element per output channel, passed as
  // further tensors behind the problem's own; MIGraphXToTosa.cpp:874-982 broadcasts such tensors)
  e.chan_flags = 0;
  {
    auto vec = [&](const char *key, int bit, int i8_bit) {
      const std::string v = str_or(o, key, "false");
      if (v == "false" || v == "0")
        return true;
      if (v == "i8" && i8_bit)
        e.chan_flags |= bit | i8_bit;
      else if (v == "true" || v == "1" || v == "i32" || (v == "f32" && !i8_bit))
        e.chan_flags |= bit;
      else
        return false;
      return true;
    };
    if (!vec("scale_vector", ROCK_CHAN_SCALE, 0) || !vec("zero_point_vector", ROCK_CHAN_ZP, ROCK_CHAN_ZP_I8) ||
        !vec("quant_scale_vector", ROCK_CHAN_QUANT_SCALE, 0) ||
        !vec("out_zero_point_vector", ROCK_CHAN_OUT_ZP, ROCK_CHAN_OUT_ZP_I8))
      return false;
    // the dequantisation vectors need the float step, a zero point an integer accumulator, the
    // quantisation vectors an int8 result
    if ((e.chan_flags & (ROCK_CHAN_SCALE | ROCK_CHAN_ZP)) && out_dtype == ROCK_I32)
      return false;
    if ((e.chan_flags & ROCK_CHAN_ZP) && is_float_in(in_a))
      return false;
    if ((e.chan_flags & (ROCK_CHAN_QUANT_SCALE | ROCK_CHAN_OUT_ZP)) && out_dtype != ROCK_I8)
      return false;
  }
  // legality (RockDialect.cpp:539-568): float in -> float out, int in -> int
  // out; the fused quantisation epilogue additionally lets an int8 problem
  // leave as a float (dequantizelinear) and a float problem leave as int8
  // (quantizelinear).
  if (is_float_in(in_a) && out_dtype == ROCK_I32)
    return false;
  return true;
}

// RockChannelVector bits of the per-channel quantisation vectors a problem asks for (the keys parse_epilogue reads)
int channel_vector_flags(const OptMap &o) {
  int flags = 0;
  auto vec = [&](const char *key, int bit, int i8_bit) {
    const std::string v = str_or(o, key, "false");
    if (v != "false" && v != "0")
      flags |= bit | (v == "i8" ? i8_bit : 0);
  };
  vec("scale_vector", ROCK_CHAN_SCALE, 0);
  vec("zero_point_vector", ROCK_CHAN_ZP, ROCK_CHAN_ZP_I8);
  vec("quant_scale_vector", ROCK_CHAN_QUANT_SCALE, 0);
  vec("out_zero_point_vector", ROCK_CHAN_OUT_ZP, ROCK_CHAN_OUT_ZP_I8);
  return flags;
}

void apply_tile_grid(const Tile &t, int64_t M, int64_t N, int G, int &tiles_m, int &tiles_n,
                     int &group_m, int &xcd_remap, uint32_t &block, uint32_t &grid) {
  tiles_m = ceil_div(M, t.bm);
  tiles_n = ceil_div(N, t.bn);
  group_m = std::min(tiles_m, t.bm >= 256 ? 4 : 8);
  int64_t total = (int64_t)tiles_m * tiles_n * G;
  xcd_remap = total >= 2 * kNumXCD ? 1 : 0;
  block = (uint32_t)(t.waves_m * t.waves_n * 64);
  grid = (uint32_t)total;
}

// field `index` (0-based) of "--perf_config [v2:]a,b,c,...", or dflt
int64_t perf_field(const OptMap &o, int index, int64_t dflt) {
  std::string pc = str_or(o, "perf_config", "");
  if (pc.rfind("v2:", 0) == 0)
    pc = pc.substr(3);
  else if (pc.find(':') != std::string::npos)
    return dflt; // another grammar (attn:v1:...)
  std::istringstream iss(pc);
  std::string part;
  for (int i = 0; std::getline(iss, part, ','); ++i)
    if (i == index) {
      char *end = nullptr;
      long long v = std::strtoll(part.c_str(), &end, 10);
      return (end != part.c_str() && *end == '\0') ? v : dflt;
    }
  return dflt;
}

std::string perf_string(const Tile &t, int es, const OptMap *o = nullptr) {
  // v2:MPB,NPB,KpackPB,MPW,MnPerXdl,Kpack,splitK,forceUnroll,1
  // forceUnroll: 1 = the kernel whose epilogue is unrolled over its
  // accumulators wherever the problem's epilogue allows it, 0 = the "_e" twin
  // with the rolled epilogue whatever the epilogue (see rich_suffix)
  int kpack = 16 / es;
  int kpack_per_block = 128 / 16; // 128 K bytes per stage row, 16-byte chunks
  char buf[96];
  std::snprintf(buf, sizeof buf, "v2:%d,%d,%d,%d,%d,%d,1,%d,1", t.bm, t.bn, kpack_per_block,
                t.bm / t.waves_m, 16, kpack, (o && perf_field(*o, 7, 1) == 0) ? 0 : 1);
  return buf;
}

// "--perf_config v2:MPB,NPB,..." selects a tile by its block sizes; anything
// that does not name an available tile falls back to the table, like the
// reference's tuningFallback (AffixTuningParameters.cpp:129-141).
std::string forced_tile(const OptMap &o) {
  std::string pc = str_or(o, "perf_config", "");
  if (pc.rfind("v2:", 0) == 0)
    pc = pc.substr(3);
  int a = 0, b = 0;
  if (std::sscanf(pc.c_str(), "%d,%d", &a, &b) == 2) {
    for (const Tile &t : kFastTiles)
      if (t.bm == a && t.bn == b)
        return std::to_string(a) + "x" + std::to_string(b);
  }
  return "";
}

// true when "--perf_config [v2:]MPB,NPB,..." names exactly this block tile
// (the first two fields; later fields of a reference-style string, such as
// MPerWave = 32, must not match)
bool requested_tile_is(const OptMap &o, int bm, int bn) {
  std::string pc = str_or(o, "perf_config", "");
  if (pc.rfind("v2:", 0) == 0)
    pc = pc.substr(3);
  int a = 0, b = 0;
  return std::sscanf(pc.c_str(), "%d,%d", &a, &b) == 2 && a == bm && b == bn;
}

// A reduction split over blocks (S shares of K into f32 partial sums, added by
// rock_reduce_splits) rides in the 7th field of the string, splitK in the
// reference's grammar (RockAttrDefs.td:241-251), so that the perf_config a
// split plan reports leads back to the same plan.  The 32x32 kernel that divides K
// over the four waves of a block has always reported 4 there: its field is 4 * S.
// -1: no perf_config given, the table decides.
int64_t requested_block_splits(const OptMap &o) {
  if (!o.count("perf_config"))
    return -1;
  const int64_t field = std::max<int64_t>(1, perf_field(o, 6, 1));
  return requested_tile_is(o, 32, 32) ? std::max<int64_t>(1, field / 4) : field;
}

std::string with_block_splits(const std::string &pc, int64_t S) {
  if (S <= 1 || pc.rfind("v2:", 0) != 0)
    return pc;
  std::vector<std::string> f;
  std::istringstream iss(pc.substr(3));
  for (std::string part; std::getline(iss, part, ',');)
    f.push_back(part);
  if (f.size() < 7)
    return pc;
  const bool wave_split = f[0] == "32" && f[1] == "32";
  f[6] = std::to_string(wave_split ? 4 * S : S);
  std::string out = "v2:";
  for (size_t i = 0; i < f.size(); ++i)
    out += (i ? "," : "") + f[i];
  return out;
}

void default_epilogue(RockEpilogue &e, int out_dtype) {
  std::memset(&e, 0, sizeof e);
  e.scale = 1.0f;
  e.inv_quant_scale = 1.0f;
  e.out_dtype = out_dtype;
  e.act_lo = -INFINITY;
  e.act_hi = INFINITY;
}

int64_t align256(int64_t bytes) { return (bytes + 255) / 256 * 256; }

// The tiled kernels exist twice: with the plain epilogue unrolled over their
// accumulators, and ("_e") with the rolled epilogue that a residual tensor or a
// transcendental activation needs.  The element-wise kernels handle both in
// one.
const char *rich_suffix(const RockEpilogue &e, bool tiled_kernel, const OptMap &o) {
  // "-rolled_epilogue true", or a perf_config whose eighth field (forceUnroll)
  // is 0, asks for the twin regardless (it handles every epilogue)
  // (so do the per-channel quantisation vectors: the plain kernels are compiled without them)
  return tiled_kernel && (e.residual_op != ROCK_RES_NONE || e.activation > ROCK_ACT_CLIP || e.chan_flags != 0 ||
                          bool_or(o, "rolled_epilogue", false) || perf_field(o, 7, 1) == 0) ? "_e" : "";
}

// The contraction kernels take five pointers: two operands, the output, the
// per-channel bias and the residual tensor.  A caller passes the residual
// only when the problem names one; otherwise the library fills that slot
// with NULL.
void set_contraction_pointers(Handle *h, const RockEpilogue &e) {
  h->num_pointers = 5;
  if (e.residual_op) {
    h->caller_pointers = 0; // all five, in order
    h->ptr_map.clear();
  } else {
    h->caller_pointers = 4;
    h->ptr_map = {{0, 0}, {1, 0}, {2, 0}, {3, 0}, {-1, 0}};
  }
}

// Chooses the kernel, tile and grid for a GEMM whose sizes and strides are
// already in p.  Returns false when only the element-wise kernel fits.
// `k_padded`: the caller guarantees that every K-contiguous operand row is
// zero-filled from K up to the next whole 16-byte chunk (copies made by the
// conversion plan), so K itself need not be a whole number of chunks.
bool plan_gemm_kernel(Handle *h, RockGemmParams &p, int code, int es, const OptMap &o, bool k_padded = false) {
  const int64_t M = p.M, N = p.N, K = p.K, G = p.G;
  // vector path: K-contiguous rows of whole 16-byte chunks, and every byte
  // offset inside one block tile (256 rows at most) below 2^31 for the buffer
  // descriptors of the direct-to-LDS loads
  const int64_t kMaxOff = (int64_t)1 << 31;
  auto al16 = [&](int64_t elems) { return (elems * es) % 16 == 0; };
  // each operand either K-contiguous (rows of whole chunks) or K-major (its
  // M / N index contiguous, k-rows of whole chunks: the transposing-read path)
  const bool k_ok = al16(K) || k_padded;
  const bool a_rows = p.a_ks == 1 && al16(p.a_ms) && k_ok && al16(p.a_gs) && 256 * p.a_ms * es + K * es < kMaxOff;
  const bool b_rows = p.b_ks == 1 && al16(p.b_ns) && k_ok && al16(p.b_gs) && 256 * p.b_ns * es + K * es < kMaxOff;
  const bool a_cols = p.a_ms == 1 && al16(p.a_ks) && al16(M) && al16(p.a_gs) && K * p.a_ks * es + 256 * es < kMaxOff;
  const bool b_cols = p.b_ns == 1 && al16(p.b_ks) && al16(N) && al16(p.b_gs) && K * p.b_ks * es + 256 * es < kMaxOff;
  const bool fast = a_rows && b_rows;
  // storage suffix of the K-major variants: n = as the reference stores it by default
  const char *storage = nullptr;
  if (!fast && (a_rows || a_cols) && (b_rows || b_cols))
    storage = a_rows ? "_nn" : b_rows ? "_tt" : "_tn";
  const bool tiled = fast || storage;
  const Tile *tile = tiled ? pick_tile(M, N, p.G, false, forced_tile(o), storage != nullptr) : nullptr;
  if (!tile)
    tile = tiled ? pick_tile(M, N, p.G, false, "", storage != nullptr) : &kGenericTile;
  // Too few 64x64 tiles to occupy half the CUs and a K long enough to split:
  // one 32x32 tile per block with the K range divided over its waves (the
  // reference's answer to the same situation is split-K with atomics,
  // RockTuningImpl.cpp:962-1008).
  const bool forced = !forced_tile(o).empty();
  const int64_t tiles64 = (int64_t)ceil_div(M, 64) * ceil_div(N, 64) * G;
  int split_k = 1;
  if (fast && !forced && tiles64 * 2 <= kNumCU && K * es >= 16 * 64) {
    tile = &kSplitKTile;
    split_k = 4;
  }
  if (fast && requested_tile_is(o, kSplitKTile.bm, kSplitKTile.bn)) {
    tile = &kSplitKTile; // "-perf_config v2:32,32,..." asks for it explicitly
    split_k = 4;
  }
  apply_tile_grid(*tile, M, N, p.G, p.tiles_m, p.tiles_n, p.group_m, p.xcd_remap,
                  h->block_size, h->grid_size);
  if (split_k > 1)
    h->block_size = 256;
  h->kernel_name = std::string("rock_gemm_") + operand_name(code) + tile->suffix + (storage ? storage : "") +
                   rich_suffix(p.epi, tiled, o);
  set_contraction_pointers(h, p.epi);
  h->perf_config = perf_string(*tile, es, &o);
  if (split_k > 1) { // the reference's grammar has a splitK field (7th)
    char buf[96];
    std::snprintf(buf, sizeof buf, "v2:32,32,4,32,32,%d,%d,1,1", 16 / es, split_k);
    h->perf_config = buf;
  }
  return tiled;
}

// ---- attention kernel variants and their perf_config strings ---------------
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
const AttnVariant kAttnVariants[] = {{"fast", 8, 1}, {"fast_bias", 8, 0}, {"generic", 1, 1}};

std::string attn_perf_string(const AttnVariant &v, int dmax) {
  char buf[96];
  std::snprintf(buf, sizeof buf, "attn:v1:64,%d,128,%d,32,32,%d,%d", dmax, v.kpack_pb, v.kpack_pb == 1 ? 1 : 8,
                v.force_unroll);
  return buf;
}

// Parses "attn:v1:..." (eight fields); false when the string is another grammar or malformed.
bool parse_attn_perf(const std::string &pc, int &dmax, int &kpack_pb, int &force_unroll) {
  if (pc.rfind("attn:v1:", 0) != 0)
    return false;
  int f[8];
  if (std::sscanf(pc.c_str() + 8, "%d,%d,%d,%d,%d,%d,%d,%d", &f[0], &f[1], &f[2], &f[3], &f[4], &f[5], &f[6], &f[7]) != 8)
    return false;
  dmax = f[1];
  kpack_pb = f[3];
  force_unroll = f[7];
  return true;
}

bool fill_relayout_handle(Handle *h, const int64_t size[5], const int64_t src_size[5],
                          const int64_t src_stride[5], int es, const int64_t *dst_stride = nullptr);

// ---- GEMM -----------------------------------------------------------------
Handle *make_gemm(const OptMap &o) {
  std::string t = str_or(o, "t", "f32");
  int ta, tb;
  size_t us = t.find('_');
  if (us != std::string::npos) {
    ta = parse_dtype(t.substr(0, us));
    tb = parse_dtype(t.substr(us + 1));
  } else {
    ta = tb = parse_dtype(t);
  }
  if (ta < 0 || tb < 0 || ta == ROCK_I32 || tb == ROCK_I32) {
    set_error("gemm: unknown data type '" + t + "'");
    return nullptr;
  }
  int code = operand_code(ta, tb);
  if (code < 0) {
    set_error("gemm: unsupported operand type pair '" + t + "'");
    return nullptr;
  }
  // default output type: i8 -> i32, 8-bit floats -> f32, else the input type
  // (rocmlir-gen.cpp:432-458)
  int dflt_out = ta == ROCK_I8 ? ROCK_I32 : (ta == ROCK_FP8 || ta == ROCK_BF8) ? ROCK_F32 : ta;
  std::string outs = str_or(o, "out_datatype", str_or(o, "c_dtype", ""));
  int tc = outs.empty() ? dflt_out : parse_dtype(outs);
  if (tc < 0) {
    set_error("gemm: unknown output type '" + outs + "'");
    return nullptr;
  }
  int64_t G = int_or(o, "g", 1), M, N, K;
  if (!get_int(o, "m", M) || !get_int(o, "n", N) || !get_int(o, "k", K) || G <= 0 || M <= 0 ||
      N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || G > INT32_MAX) {
    set_error("gemm: -m, -n, -k (and -g) must be given and positive");
    return nullptr;
  }
  bool tA = bool_or(o, "transA", false), tB = bool_or(o, "transB", false),
       tC = bool_or(o, "transC", false);

  auto *h = new Handle;
  h->op = OP_GEMM;
  h->params.assign(sizeof(RockGemmParams), 0);
  auto &p = *reinterpret_cast<RockGemmParams *>(h->params.data());
  h->epi = &p.epi;
  if (!parse_epilogue(o, ta, tc, p.epi)) {
    set_error("gemm: illegal input/output type combination or epilogue");
    delete h;
    return nullptr;
  }
  // storage (rocmlir-gen.cpp:2058-2080): A [G,M,K] (transA: [G,K,M]),
  // B [G,K,N] (transB: [G,N,K]), C [G,M,N] (transC: [G,N,M])
  p.G = (int)G; p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.a_gs = M * K; p.a_ms = tA ? 1 : K; p.a_ks = tA ? M : 1;
  p.b_gs = K * N; p.b_ks = tB ? 1 : N; p.b_ns = tB ? K : 1;
  p.c_gs = M * N; p.c_ms = tC ? 1 : N; p.c_ns = tC ? M : 1;

  bool vector_kernel = plan_gemm_kernel(h, p, code, dtype_size(ta), o);
  // Padded copies.  An operand whose rows are not whole, aligned 16-byte chunks
  // (an odd K, N = 60 under the default [K, N] storage) would leave the whole
  // problem on the element-wise kernel.  Instead each such operand is first
  // copied K-contiguous into the workspace by one conversion kernel, its rows
  // zero-filled up to whole chunks, and the vector kernel reads the copies; the
  // output is written as the caller laid it out.  The reference pads to block
  // multiples inside its generated kernel and stays on the MFMA schedule
  // (GridwiseGemmParams.cpp:91-103); this is the same through the multi-kernel
  // protocol the library already speaks.
  if (!vector_kernel && bool_or(o, "layout_conversion", true)) {
    const int es = dtype_size(ta);
    const int64_t ce = 16 / es, Kp = (K + ce - 1) / ce * ce;
    auto al = [&](int64_t elems) { return (elems * es) % 16 == 0; };
    // as plan_gemm_kernel reads them, with the K tail now allowed
    const bool a_keep = (p.a_ks == 1 && al(p.a_ms) && al(p.a_gs) && p.a_ms >= Kp) || (p.a_ms == 1 && al(p.a_ks) && al(M) && al(p.a_gs));
    const bool b_keep = (p.b_ks == 1 && al(p.b_ns) && al(p.b_gs) && p.b_ns >= Kp) || (p.b_ns == 1 && al(p.b_ks) && al(N) && al(p.b_gs));
    // a kept K-contiguous operand must have zeros behind an odd K as well: only copies do
    const bool need_a = !a_keep || (p.a_ks == 1 && Kp != K), need_b = !b_keep || (p.b_ks == 1 && Kp != K);
    const int64_t a_bytes = align256(G * M * Kp * es), b_bytes = align256(G * N * Kp * es);
    RockGemmParams q = p;
    if (need_a) { q.a_gs = M * Kp; q.a_ms = Kp; q.a_ks = 1; }
    if (need_b) { q.b_gs = N * Kp; q.b_ns = Kp; q.b_ks = 1; }
    Handle probe;
    probe.params.assign(sizeof q, 0);
    if ((need_a || need_b) && G * M * Kp <= INT32_MAX && G * N * Kp <= INT32_MAX &&
        plan_gemm_kernel(&probe, q, code, es, o, true)) {
      // one conversion kernel: of the operand that needs it, or of both in one launch
      const int n_copy = 1;
      const int ws = p.epi.residual_op ? 5 : 4; // A, B, C, bias, [residual,] workspace
      const int kid = (int)int_or(o, "kernel_id", 0);
      if (kid < 0 || kid > n_copy) {
        set_error("gemm: kernel_id out of range");
        delete h;
        return nullptr;
      }
      const int64_t off_a = 0, off_b = need_a ? a_bytes : 0;
      if (kid == 0) {
        auto fill = [&](Handle *dst, bool is_a) {
          const int64_t rows = is_a ? M : N;
          const int64_t size[5] = {1, 1, G, rows, Kp}, src_size[5] = {1, 1, G, rows, K};
          const int64_t stride[5] = {0, 0, is_a ? p.a_gs : p.b_gs, is_a ? p.a_ms : p.b_ns, is_a ? p.a_ks : p.b_ks};
          return fill_relayout_handle(dst, size, src_size, stride, es);
        };
        if (need_a && need_b) {
          Handle first, second;
          if (!fill(&first, true) || !fill(&second, false)) {
            delete h;
            return nullptr;
          }
          RockRelayoutPairParams pair;
          std::memset(&pair, 0, sizeof pair);
          std::memcpy(&pair.first, first.params.data(), sizeof pair.first);
          std::memcpy(&pair.second, second.params.data(), sizeof pair.second);
          pair.first_blocks = (int32_t)first.grid_size;
          h->op = OP_RELAYOUT;
          h->epi = nullptr;
          h->params.assign(sizeof pair, 0);
          std::memcpy(h->params.data(), &pair, sizeof pair);
          h->kernel_name = std::string("rock_relayout_pair_b") + std::to_string(es);
          h->block_size = 256;
          h->grid_size = first.grid_size + second.grid_size;
          h->num_pointers = 4;
          h->perf_config = "";
          h->ptr_map = {{0, 0}, {ws, off_a}, {1, 0}, {ws, off_b}};
        } else {
          if (!fill(h, need_a)) {
            delete h;
            return nullptr;
          }
          h->ptr_map = {{need_a ? 0 : 1, 0}, {ws, need_a ? off_a : off_b}};
        }
      } else {
        p = q;
        vector_kernel = plan_gemm_kernel(h, p, code, es, o, true);
        h->ptr_map = {{need_a ? ws : 0, need_a ? off_a : 0}, {need_b ? ws : 1, need_b ? off_b : 0}, {2, 0}, {3, 0},
                      {p.epi.residual_op ? 4 : -1, 0}};
      }
      { // every handle of the problem carries the problem's key
        std::ostringstream k;
        k << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << "-t " << operand_name(code)
          << " -out_datatype " << dtype_name(tc) << " -transA " << (tA ? "true" : "false")
          << " -transB " << (tB ? "true" : "false") << " -g " << G << " -m " << M << " -n " << N
          << " -k " << K;
        h->problem_key = k.str();
      }
      h->kernel_count = n_copy + 1;
      h->workspace_bytes = (size_t)((need_a ? a_bytes : 0) + (need_b ? b_bytes : 0));
      h->caller_pointers = ws + 1;
      return h;
    }
  }
  // problem key (RockTuningImpl.cpp:808-862)
  auto set_key = [&](Handle *hh) {
    std::ostringstream k;
    k << hh->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << "-t " << operand_name(code)
      << " -out_datatype " << dtype_name(tc) << " -transA " << (tA ? "true" : "false")
      << " -transB " << (tB ? "true" : "false") << " -g " << G << " -m " << M << " -n " << N
      << " -k " << K;
    hh->problem_key = k.str();
  };
  // Split of the reduction over blocks.  A single floating-point GEMM with few
  // output tiles and a long K leaves most of the chip idle; its K range is cut
  // into S batch entries writing f32 partial results into a workspace, which
  // the reduction kernel adds up in split order (the reference reaches the same
  // parallelism with atomic adds into a pre-filled C, RockTuningImpl.cpp:962-1008,
  // Rock.cpp:167-198).  Only with the identity epilogue, which commutes with the sum.
  {
    const int es = dtype_size(ta);
    const RockEpilogue &e = p.epi;
    const bool identity = e.scale == 1.0f && !e.has_bias && e.activation == ROCK_ACT_NONE && !e.chan_flags &&
                          e.residual_op == ROCK_RES_NONE && (tc == ROCK_F32 || tc == ROCK_F16 || tc == ROCK_BF16);
    // any vector storage, including the K-contiguous one for which the planner
    // has just chosen the split over the waves of a block: the sub-problems
    // are planned again below and may still take that kernel, now S times over
    const bool tiled = vector_kernel;
    const int64_t tiles64 = (int64_t)ceil_div(M, 64) * ceil_div(N, 64);
    // ... unless that kernel's 32x32 tiles already occupy half the chip by themselves
    const bool wave_split = h->kernel_name.find(kSplitKTile.suffix) != std::string::npos;
    // (measured: with K = 1024 the second kernel costs more than the split gives back; from K = 2048 on the
    // split over blocks wins even against the wave-split kernel with all its tiles resident -- M 640, N 768,
    // K 8192 f16: 21 us against 36 (NT, wave split) and 58 (NN, one block per tile))
    const bool long_k = K >= 2048;
    const bool wave_split_fills = wave_split && !long_k && (int64_t)ceil_div(M, 32) * ceil_div(N, 32) * 2 > kNumCU;
    int64_t S = 1;
    const int64_t s_req = requested_block_splits(o); // a perf_config names the split itself
    auto share_ok = [&](int64_t d) { return K % d == 0 && ((K / d) * es) % 64 == 0; };
    if (G == 1 && is_float_in(ta) && is_float_in(tb) && identity && tiled && bool_or(o, "split_k", true)) {
      if (s_req > 1 && share_ok(s_req))
        S = s_req;
      else if (s_req < 0 && !wave_split_fills && tiles64 * (long_k ? 2 : 4) <= kNumCU) {
        const int64_t want = std::min<int64_t>(2 * kNumCU / tiles64, K / 512);
        for (int64_t d = want; d >= 2; --d)
          if (share_ok(d)) {
            S = d;
            break;
          }
      }
    }
    if (S > 1) {
      const int kid = (int)int_or(o, "kernel_id", 0);
      if (kid < 0 || kid > 1) {
        set_error("gemm: kernel_id out of range");
        delete h;
        return nullptr;
      }
      const int64_t Ks = K / S, cstride_m = p.c_ms, cstride_n = p.c_ns;
      if (kid == 0) {
        p.G = (int)S; p.K = (int)Ks;
        p.a_gs = Ks * p.a_ks; p.b_gs = Ks * p.b_ks;
        p.c_gs = M * N; p.c_ms = N; p.c_ns = 1;
        default_epilogue(p.epi, ROCK_F32);
        plan_gemm_kernel(h, p, code, es, o);
        h->perf_config = with_block_splits(h->perf_config, S);
        h->ptr_map = {{0, 0}, {1, 0}, {4, 0}, {-1, 0}, {-1, 0}};
        set_key(h);
      } else {
        RockReduceParams r;
        std::memset(&r, 0, sizeof r);
        r.split_stride = M * N;
        r.size[0] = 1; r.size[1] = 1; r.size[2] = (int)M; r.size[3] = (int)N;
        r.dst_stride[2] = cstride_m; r.dst_stride[3] = cstride_n;
        r.splits = (int)S;
        r.out_dtype = tc;
        h->op = OP_RELAYOUT;
        h->epi = nullptr;
        h->params.assign(sizeof r, 0);
        std::memcpy(h->params.data(), &r, sizeof r);
        h->kernel_name = "rock_reduce_splits";
        h->block_size = 256;
        h->grid_size = (uint32_t)((M * N + 255) / 256);
        h->num_pointers = 2;
        h->perf_config = "";
        h->ptr_map = {{4, 0}, {2, 0}};
        h->problem_key = "reduction of the split partial sums";
      }
      h->kernel_count = 2;
      h->workspace_bytes = (size_t)align256(S * M * N * 4);
      h->caller_pointers = 5; // A, B, C, unused, workspace
      return h;
    }
  }
  {
    std::ostringstream k;
    k << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << "-t " << operand_name(code)
      << " -out_datatype " << dtype_name(tc) << " -transA " << (tA ? "true" : "false")
      << " -transB " << (tB ? "true" : "false") << " -g " << G << " -m " << M << " -n " << N
      << " -k " << K;
    h->problem_key = k.str();
  }
  return h;
}

// n / d for n < 2^31 as a multiplication and a shift (Granlund and Montgomery, "Division by invariant integers
// using multiplication", 1994, theorem 4.2 with 31-bit dividends): mul = ceil(2^(31 + l) / d), l = ceil(log2 d)
RockFastDiv fast_div_of(int64_t d) {
  int l = 0;
  while (((int64_t)1 << l) < d)
    ++l;
  const unsigned __int128 pow = (unsigned __int128)1 << (31 + l);
  return RockFastDiv{(uint32_t)((pow + (unsigned __int128)d - 1) / (unsigned __int128)d), (uint32_t)(31 + l)};
}

// Makes h a layout-conversion kernel: a 5-D tensor, dimensions listed in the
// destination's order (the last one contiguous there, the destination dense
// unless dst_stride says otherwise),
// read through src_stride and zero-filled beyond src_size.  Strides may be
// negative (a flipped filter); the caller adds the matching base offset to the
// source pointer.  Returns false with the error set when the tensor is too
// large for the kernel's 32-bit indices.
bool fill_relayout_handle(Handle *h, const int64_t size[5], const int64_t src_size[5],
                          const int64_t src_stride[5], int es, const int64_t *dst_stride) {
  RockRelayoutParams r;
  std::memset(&r, 0, sizeof r);
  struct Dim { int64_t size, src_size, ss, ds; };
  std::vector<Dim> dims;
  int64_t dst = 1;
  // dst_stride: a destination that is a slice of a larger dense tensor (last
  // dimension still contiguous, every stride a whole number of 16-byte chunks)
  for (int d = 4; d >= 0; --d) {
    dims.insert(dims.begin(), Dim{size[d], src_size[d], src_stride[d], dst_stride ? dst_stride[d] : dst});
    dst *= size[d];
  }
  // drop unit dimensions and fold neighbours that are laid out back to back
  // on both sides (h and w of an NCHW image) into one, so that the tiled
  // dimensions are as long as the layouts allow
  for (size_t d = 0; d + 1 < dims.size();) // the channel dimension stays last
    if (dims[d].size == 1)
      dims.erase(dims.begin() + d);
    else
      ++d;
  for (size_t d = 0; d + 1 < dims.size();) {
    const Dim &o = dims[d], &i = dims[d + 1];
    if (i.src_size == i.size && o.ss == i.size * i.ss && o.ds == i.size * i.ds &&
        o.size * i.size <= INT32_MAX) {
      dims[d] = Dim{o.size * i.size, o.src_size * i.size, i.ss, i.ds};
      dims.erase(dims.begin() + d + 1);
    } else {
      ++d;
    }
  }
  while (dims.size() < 5)
    dims.insert(dims.begin(), Dim{1, 1, 0, 0});
  for (int d = 0; d < 5; ++d) {
    r.size[d] = (int32_t)dims[d].size;
    r.src_size[d] = (int32_t)dims[d].src_size;
    r.src_stride[d] = dims[d].ss;
    r.dst_stride[d] = dims[d].ds;
  }
  r.dst_fast = 4;
  r.src_fast = 4;
  for (int d = 0; d < 5; ++d) // the source's contiguous dimension (ties: the longest)
    if (r.src_stride[d] == 1 && (r.src_stride[r.src_fast] != 1 || r.size[d] > r.size[r.src_fast]))
      r.src_fast = d;
  if (r.src_stride[r.src_fast] != 1) {
    // no unit-stride dimension (every other pixel of a row, a flipped filter):
    // tile along the one whose elements lie closest together
    for (int d = 0; d < 5; ++d)
      if (r.size[d] > 1 && r.src_stride[d] != 0 &&
          std::llabs(r.src_stride[d]) < std::llabs(r.src_stride[r.src_fast]))
        r.src_fast = d;
  }
  // runs along the shared contiguous dimension that are a power-of-two fraction of a 16-byte chunk, stored
  // back to back along dimension 3 (3 channels padded to 4 of 16 bits): a chunk holds several of them
  int positions_per_chunk = 1;
  {
    const int64_t run_bytes = (int64_t)r.size[4] * es;
    if (run_bytes < 16 && 16 % run_bytes == 0 && r.dst_stride[3] == r.size[4] && r.size[3] % (16 / run_bytes) == 0 &&
        (r.src_fast == 4 || r.src_fast == 3))
      positions_per_chunk = (int)(16 / run_bytes);
  }
  if (positions_per_chunk == 1 && r.src_fast == r.dst_fast && ((int64_t)r.size[4] * es) % 16 != 0) {
    // runs along the shared contiguous dimension that are not whole 16-byte
    // chunks (an output with 12 f16 channels): element-wise tiles over that
    // dimension and another one: of those long enough to fill a tile's rows
    // the one whose runs lie closest together in the source, else the longest
    r.src_fast = 3;
    for (int d = 0; d < 4; ++d)
      if (r.size[d] > r.size[r.src_fast])
        r.src_fast = d;
    for (int d = 0; d < 4; ++d)
      if (r.size[d] >= 32 && r.src_stride[d] != 0 &&
          (r.size[r.src_fast] < 32 || std::llabs(r.src_stride[d]) < std::llabs(r.src_stride[r.src_fast])))
        r.src_fast = d;
  }
  int64_t blocks = 1;
  int tile_s_of_plan = 1;
  // a destination run of one 16-byte chunk (a 3-channel image padded to 8):
  // one thread per chunk gathers its elements wherever the source keeps them;
  // consecutive threads take consecutive pixels
  const bool one_chunk = (int64_t)r.size[4] * es == 16 && r.src_fast == 3;
  if (r.src_fast == r.dst_fast || one_chunk || positions_per_chunk > 1) {
    // whole 16-byte chunks along the contiguous dimension (by construction of cp), or several runs a chunk
    r.mode = RELAYOUT_COPY;
    r.tile_d = positions_per_chunk;
    const int64_t chunks = positions_per_chunk > 1 ? (int64_t)r.size[2] * (r.size[3] / positions_per_chunk)
                                                   : (int64_t)r.size[2] * r.size[3] * (r.size[4] * es / 16);
    if (chunks > INT32_MAX) {
      set_error("conv: tensor too large for the layout-conversion kernel");
      return false;
    }
    blocks = (chunks + 255) / 256 * r.size[1] * r.size[0];
  } else {
    // short channel runs: narrow tiles, element-wise; otherwise tiles with
    // 16-byte accesses (relayout_body.h): 128-byte rows on both sides, reshaped
    // when either dimension is shorter than that
    const bool vec = r.size[r.dst_fast] > 16;
    r.mode = vec ? RELAYOUT_TRANSPOSE_VEC : RELAYOUT_TRANSPOSE;
    int tile_s;
    if (vec) {
      const int v = 16 / es, area = 256 * (es == 1 ? 4 : 2) * v, min_side = 2 * v;
      auto pow2_at_least = [](int64_t n) { int q = 1; while (q < n) q *= 2; return q; };
      int td = std::min(std::max(pow2_at_least(r.size[r.dst_fast]), min_side), 8 * v);
      int ts = area / td;
      if (r.size[r.src_fast] < ts) {
        ts = std::max(pow2_at_least(r.size[r.src_fast]), min_side);
        td = area / ts;
      }
      r.tile_d = td;
      tile_s = ts;
    } else {
      r.tile_d = r.size[r.dst_fast] <= 8 ? 8 : r.size[r.dst_fast] <= 16 ? 16 : 32;
      tile_s = 1024 / r.tile_d;
    }
    tile_s_of_plan = tile_s;
    for (int d = 0; d < 5; ++d) {
      if (d == r.src_fast)
        blocks *= (r.size[d] + tile_s - 1) / tile_s;
      else if (d == r.dst_fast)
        blocks *= (r.size[d] + r.tile_d - 1) / r.tile_d;
      else
        blocks *= r.size[d];
    }
  }
  if (blocks > INT32_MAX) {
    set_error("conv: tensor too large for the layout-conversion kernel");
    return false;
  }
  {
    // the divisors of the kernel's index decoding, in its order (kernel_params.h)
    int64_t divisor[5] = {1, 1, 1, 1, 1};
    if (r.mode == RELAYOUT_COPY) {
      const int64_t chunks4 = r.tile_d > 1 ? 1 : r.size[4] * es / 16, groups3 = r.size[3] / r.tile_d;
      divisor[0] = ((int64_t)r.size[2] * groups3 * chunks4 + 255) / 256;
      divisor[1] = r.size[1];
      divisor[2] = chunks4;
      divisor[3] = groups3;
    } else {
      const int sf = r.src_fast, df = r.dst_fast;
      r.ss_s = r.src_stride[sf]; r.ss_d = r.src_stride[df];
      r.ds_s = r.dst_stride[sf]; r.ds_d = r.dst_stride[df];
      r.size_s = r.size[sf]; r.size_d = r.size[df];
      r.src_s = r.src_size[sf]; r.src_d = r.src_size[df];
      r.tiles_s = (r.size[sf] + tile_s_of_plan - 1) / tile_s_of_plan;
      r.tiles_d = (r.size[df] + r.tile_d - 1) / r.tile_d;
      r.ts_shift = __builtin_ctz((unsigned)tile_s_of_plan);
      r.td_shift = __builtin_ctz((unsigned)r.tile_d);
      divisor[0] = r.tiles_s;
      divisor[1] = r.tiles_d;
      int n = 0;
      for (int d = 4; d >= 0; --d) {
        if (d == sf || d == df)
          continue;
        r.outer_size[n] = r.size[d];
        r.outer_src[n] = r.src_size[d];
        r.outer_ss[n] = r.src_stride[d];
        r.outer_ds[n] = r.dst_stride[d];
        divisor[2 + n] = r.size[d];
        ++n;
      }
    }
    for (int i = 0; i < 5; ++i)
      r.div[i] = fast_div_of(divisor[i]);
  }
  h->op = OP_RELAYOUT;
  h->epi = nullptr;
  h->params.assign(sizeof r, 0);
  std::memcpy(h->params.data(), &r, sizeof r);
  h->kernel_name = std::string("rock_relayout_b") + std::to_string(es);
  h->block_size = 256;
  h->grid_size = (uint32_t)blocks;
  h->num_pointers = 2;
  h->caller_pointers = 0;
  h->perf_config = "";
  return true;
}

// ---- convolution --------------------------------------------------------------
// letter-by-letter layout translation (ConvGenerator.cpp:641-647) widened to
// rocmlir-gen's lowercase spellings with optional g (rocmlir-gen.cpp:837-863)
bool canon_layout(std::string s, char channel, const char *want, std::string &out) {
  // want: "gkcyx" / "ngchw" / "ngkhw"; `channel` is the tensor's own channel
  // letter ('k' for filter/output second channel)
  for (auto &ch : s)
    ch = (char)std::tolower((unsigned char)ch);
  const bool filter = want[0] == 'g' && want[1] == 'k';
  std::string r;
  for (char ch : s) {
    char m = ch;
    if (ch == '0') m = filter ? 'y' : 'h';
    else if (ch == '1') m = filter ? 'x' : 'w';
    else if (filter && ch == 'h') m = 'y';
    else if (filter && ch == 'w') m = 'x';
    else if (filter && ch == 'n') m = 'k';
    else if (!filter && ch == 'y') m = 'h';
    else if (!filter && ch == 'x') m = 'w';
    else if (!filter && channel == 'k' && ch == 'c') m = 'k';
    r.push_back(m);
  }
  if (r.find('g') == std::string::npos) {
    if (filter) {
      r = "g" + r;
    } else {
      std::string c1(1, channel);
      if (r.size() >= 2 && r.substr(0, 2) == "n" + c1)
        r = "ng" + c1 + r.substr(2);
      else if (r[0] == 'n' && r.back() == channel)
        r = r.substr(0, r.size() - 1) + "g" + c1;
      else
        r = "g" + r;
    }
  }
  if (r.size() != 5)
    return false;
  std::string a = r, b = want;
  std::sort(a.begin(), a.end());
  std::sort(b.begin(), b.end());
  if (a != b)
    return false;
  out = r;
  return true;
}

void layout_strides(const std::string &layout, const std::string &letters, const int64_t *sizes,
                    int64_t *strides) {
  int64_t run = 1;
  for (int pos = (int)layout.size() - 1; pos >= 0; --pos) {
    size_t idx = letters.find(layout[pos]);
    strides[idx] = run;
    run *= sizes[idx];
  }
}

std::string key_layout(const std::string &layout, bool filter) {
  // problem-key letters (RockTuningImpl.cpp:708-731): k->N (filter), c->C,
  // g->G, n->N, output k->C, spatial -> 0,1
  std::string r;
  for (char ch : layout) {
    switch (ch) {
    case 'g': r.push_back('G'); break;
    case 'n': r.push_back('N'); break;
    case 'c': r.push_back('C'); break;
    case 'k': r.push_back(filter ? 'N' : 'C'); break;
    case 'y': case 'h': r.push_back('0'); break;
    case 'x': case 'w': r.push_back('1'); break;
    }
  }
  return r;
}

// ---- backward convolutions ------------------------------------------------------
// Both gradients are forward convolutions over re-labelled views of the
// problem's tensors, so they run on the forward kernels; what the views cannot
// express directly (channel-contiguous operands for the vector kernels,
// flipped filters, a reduction split over blocks) goes through the utility
// kernels and the multi-kernel protocol.  The reference lowers them through
// its own gridwise GEMM with dedicated coordinate transforms
// (ConvToGemm.cpp:530-1131) plus zero-init / converting-copy utility kernels
// (ConvGenerator.cpp:279-344, 434-480).
struct ConvProblem {
  int ti; // element type of all three tensors
  std::string fl, il, ol;
  int64_t n, g, c, k, hi, wi, y, x, ho, wo, sh, sw, ph, pw, dh, dw;
  int64_t fs[5], is[5], os[5]; // element strides in letter order gkcyx / ngchw / ngkhw
  // filter gradient only: the output gradient is a copy whose k channels were padded with zeros up to a whole
  // 16-byte chunk; only the first k_valid rows of the gradient exist in the caller's tensor (0: all k)
  int64_t k_valid = 0;
};

int64_t floor_div(int64_t a, int64_t b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

bool conv_view_fast(const RockConvParams &q, int es) {
  auto al = [&](int64_t elems) { return (elems * es) % 16 == 0; };
  const int64_t cc = q.c;
  return q.in_cs == 1 && al(cc) && al(q.in_ws) && al(q.in_hs) && al(q.in_ns) && al(q.in_gs) && q.fil_cs == 1 &&
         q.fil_xs == cc && q.fil_ys == (int64_t)q.x * cc && al(q.fil_ks) && al(q.fil_gs) &&
         ((int64_t)q.n * q.in_ns + (int64_t)q.hi * q.in_hs + (int64_t)q.wi * q.in_ws + cc) * es < ((int64_t)1 << 31) &&
         (256 * q.fil_ks + cc * q.y * q.x) * es < ((int64_t)1 << 31);
}

// Kernel, tile and grid for a forward convolution given entirely by its
// parameter block (sizes, strides, epilogue).  False when the sizes exceed the
// kernels' 32-bit indices.
bool select_view_conv_kernel(Handle *h, RockConvParams &p, int ti, const OptMap &o) {
  const int es = dtype_size(ti);
  const int64_t Mg = (int64_t)p.n * p.ho * p.wo, Kg = (int64_t)p.c * p.y * p.x;
  if (Mg > INT32_MAX || Kg > INT32_MAX) {
    set_error("conv: problem too large for 32-bit tile indices");
    return false;
  }
  p.M = (int)Mg; p.N = p.k; p.K = (int)Kg;
  const bool fast = conv_view_fast(p, es);
  p.k_order_yxc = (p.in_cs == 1) ? 1 : 0;
  p.rows_per_tile = 0;
  const Tile *tile = fast ? pick_tile(Mg, p.k, p.g, true, forced_tile(o)) : nullptr;
  if (!tile)
    tile = fast ? pick_tile(Mg, p.k, p.g, true, "") : &kGenericTile;
  apply_tile_grid(*tile, Mg, p.k, p.g, p.tiles_m, p.tiles_n, p.group_m, p.xcd_remap, h->block_size, h->grid_size);
  h->op = OP_CONV;
  h->kernel_name = std::string("rock_conv_") + dtype_name(ti) + tile->suffix;
  h->num_pointers = 5;
  h->perf_config = perf_string(*tile, es, &o);
  return true;
}

std::string conv_problem_key(const Handle *h, const OptMap &o, const ConvProblem &cp, int direction) {
  std::ostringstream key;
  const int ti = cp.ti;
  const char *opname = ti == ROCK_F32 ? "conv" : ti == ROCK_F16 ? "convfp16" : ti == ROCK_BF16 ? "convbfp16"
                     : ti == ROCK_I8 ? "convint8" : ti == ROCK_FP8 ? "convfp8_fp8" : "convbf8_bf8";
  key << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << opname << " -F " << direction << " -f "
      << key_layout(cp.fl, true) << " -I " << key_layout(cp.il, false) << " -O " << key_layout(cp.ol, false)
      << " -n " << cp.n << " -c " << cp.c << " -H " << cp.hi << " -W " << cp.wi << " -k " << cp.k << " -y "
      << cp.y << " -x " << cp.x << " -p " << cp.ph << " -q " << cp.pw << " -u " << cp.sh << " -v " << cp.sw
      << " -l " << cp.dh << " -j " << cp.dw << " -g " << cp.g;
  return key.str();
}

Handle *conv_handle_from_view(const RockConvParams &q, int ti, const OptMap &o) {
  auto *h = new Handle;
  h->params.assign(sizeof(RockConvParams), 0);
  auto &p = *reinterpret_cast<RockConvParams *>(h->params.data());
  p = q;
  h->epi = &p.epi;
  if (!select_view_conv_kernel(h, p, ti, o)) {
    delete h;
    return nullptr;
  }
  return h;
}

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
WindowPlan window_plan(const RockConvParams &p, int ti, bool equal_padding, const OptMap &o) {
  WindowPlan w;
  const int es = dtype_size(ti);
  const int64_t cbytes = (int64_t)p.c * es;
  const bool wide_operands = ti == ROCK_FP8 || ti == ROCK_BF8; // 4 pixel blocks per tile, else 7
  const int64_t tile_px = wide_operands ? 128 : kDirectTilePixels;
  const int64_t row_pitch = ((p.wi + 2 * p.pad_w) * cbytes + 1023) / 1024 * 1024; // whole 1 KiB load slabs
  auto window_rows = [&](int64_t rows) { return rows + (p.y - 1) + (p.ho % rows ? p.y - 1 : 0); };
  w.tiles_n = ceil_div(p.k, 128);
  auto tiles_of = [&](int64_t rows) { return (int64_t)ceil_div((int64_t)p.n * p.ho, rows) * w.tiles_n * p.g; };
  // rows per tile: the fewest rounds of blocks (two per CU), then the most rows
  const int64_t per_round = 2 * (int64_t)kNumCU;
  for (int64_t rows = std::min<int64_t>(p.ho, p.wo > 0 ? tile_px / p.wo : 0); rows >= 1; --rows) {
    if (window_rows(rows) * row_pitch > kDirectWindowBytes)
      continue;
    if (w.rows == 0 || ceil_div(tiles_of(rows), per_round) < ceil_div(tiles_of(w.rows), per_round))
      w.rows = rows;
  }
  w.ok = p.stride_h == 1 && p.stride_w == 1 && p.dil_h == 1 && p.dil_w == 1 && p.y * p.x > 1 && equal_padding &&
         p.k % 32 == 0 && cbytes >= 128 && cbytes <= 1024 && (cbytes & (cbytes - 1)) == 0 && w.rows >= 1 &&
         row_pitch <= 32 * 1024 && p.in_cs == 1;
  // by itself: 16-bit types and int8 (measured: 1.13-1.3x), tiles at least 85 % full in pixels and 75 % in
  // channels, enough of them for every CU, no tile requested
  w.by_itself = w.ok && bool_or(o, "window_resident", true) && (ti == ROCK_F16 || ti == ROCK_BF16 || ti == ROCK_I8) &&
                forced_tile(o).empty() && p.y * p.x >= 4 && w.rows * p.wo * 100 >= tile_px * 85 &&
                tiles_of(w.rows) >= per_round &&
                (p.k % 128 == 0 || p.k % 128 >= 96); // (a 64-channel layer leaves half the block's waves idle)
  w.filter_bytes = align256((int64_t)p.g * w.tiles_n * 128 * p.c * p.y * p.x * es);
  return w;
}
// h becomes the window-resident kernel over p (the caller sets the pointer map)
void apply_window_plan(Handle *h, RockConvParams &p, const WindowPlan &w, int ti, const OptMap &o) {
  p.rows_per_tile = (int)w.rows;
  p.tiles_m = ceil_div((int64_t)p.n * p.ho, w.rows);
  p.tiles_n = (int)w.tiles_n;
  p.group_m = std::min(p.tiles_m, 8);
  const int64_t total = (int64_t)p.tiles_m * p.tiles_n * p.g;
  p.xcd_remap = total >= 2 * kNumXCD ? 1 : 0;
  h->block_size = 256;
  h->grid_size = (uint32_t)total;
  h->kernel_name = std::string("rock_conv_") + dtype_name(ti) + "_direct224" + rich_suffix(p.epi, true, o);
  char buf[96];
  std::snprintf(buf, sizeof buf, "v2:224,128,8,224,32,%d,1,1,1", 16 / dtype_size(ti));
  h->perf_config = buf;
}

Handle *utility_fill_handle(int64_t bytes) {
  auto *h = new Handle;
  RockFillParams f{bytes};
  h->op = OP_RELAYOUT;
  h->epi = nullptr;
  h->params.assign(sizeof f, 0);
  std::memcpy(h->params.data(), &f, sizeof f);
  h->kernel_name = "rock_fill_zero";
  h->block_size = 256;
  h->grid_size = (uint32_t)((bytes + 16 * 256 - 1) / (16 * 256));
  h->num_pointers = 1;
  h->perf_config = "";
  return h;
}

// A conversion kernel between two views of one tensor of more than five
// dimensions, listed in the destination's order (the last one contiguous
// there): unit dimensions go, neighbours that lie back to back on both sides
// fold, and what is left has to fit the kernel's five.
struct ViewDim { int64_t size, src_size, ss, ds; };
bool relayout_handle_nd(Handle *h, std::vector<ViewDim> dims, int es, const char *what) {
  for (size_t d = 0; d + 1 < dims.size();)
    if (dims[d].size == 1)
      dims.erase(dims.begin() + d);
    else
      ++d;
  for (size_t d = 0; d + 1 < dims.size() && dims.size() > 5;) {
    const ViewDim &o = dims[d], &i = dims[d + 1];
    if (i.src_size == i.size && o.ss == i.size * i.ss && o.ds == i.size * i.ds && o.size * i.size <= INT32_MAX) {
      dims[d] = ViewDim{o.size * i.size, o.src_size * i.size, i.ss, i.ds};
      dims.erase(dims.begin() + d + 1);
    } else {
      ++d;
    }
  }
  if (dims.size() > 5) {
    set_error(std::string("conv: this 3-D ") + what + " layout needs more than five independent dimensions");
    return false;
  }
  while (dims.size() < 5)
    dims.insert(dims.begin(), ViewDim{1, 1, 0, 0});
  int64_t size[5], src_size[5], ss[5], ds[5];
  for (int d = 0; d < 5; ++d) {
    size[d] = dims[d].size;
    src_size[d] = dims[d].src_size;
    ss[d] = dims[d].ss;
    ds[d] = dims[d].ds;
  }
  return fill_relayout_handle(h, size, src_size, ss, es, ds);
}

// One spatial axis of the backward-data decomposition.  Input positions with
// (i + pad) % stride == r receive only the filter taps y with
// (r - y * dilation) % stride == 0: y = y_first + t * y_step, t < T, which
// reach output position a + o_first - t * dd for i = stride * a + r - pad.
struct BwdAxis {
  int64_t T = 0, y_first = 0, y_step = 1, o_first = 0, dd = 1, a_min = 0, A = 0;
};
BwdAxis bwd_data_axis(int64_t r, int64_t stride, int64_t dil, int64_t Y, int64_t pad, int64_t in_len) {
  BwdAxis a;
  for (int64_t y = 0; y < Y; ++y) {
    if (floor_div(r - y * dil, stride) * stride != r - y * dil)
      continue;
    if (a.T == 0)
      a.y_first = y;
    else if (a.T == 1)
      a.y_step = y - a.y_first;
    ++a.T;
  }
  if (a.T > 0)
    a.o_first = floor_div(r - a.y_first * dil, stride);
  a.dd = a.T > 1 ? a.y_step * dil / stride : 1;
  a.a_min = floor_div(pad - r + stride - 1, stride);
  const int64_t a_max = floor_div(in_len - 1 + pad - r, stride);
  a.A = std::max<int64_t>(0, a_max - a.a_min + 1);
  return a;
}

// Gradient with respect to the input.  Pointer order as the forward problem:
// filter, input (written), output (the incoming gradient), unused, [workspace].
// For every phase (rh, rw) of (input position + padding) modulo the stride, the
// input positions of that phase are a stride-1 convolution of the output
// gradient with the flipped sub-filter of the taps that reach them
// (the reference makes one kernel per such phase too: kernel_id selects it,
// ConvToGemm.cpp:735-1131).  Phases without taps are left at zero by a
// zero-fill kernel that runs first.
Handle *make_conv_bwd_data(const OptMap &o, const ConvProblem &cp) {
  const int es = dtype_size(cp.ti);
  const int kid = (int)int_or(o, "kernel_id", 0);
  // 1x1 filter, unit stride, no padding, one group: dX[pixel, c] = sum over k
  // of dY[pixel, k] * W[k, c] is a GEMM over the tensors as they lie.  With
  // contiguous pixels (NCHW) it runs per image as W^T x dY_n, both operands
  // K-major; with contiguous channels (NHWC) as dY x W with the filter
  // K-major, over all images at once when their pixels are equally spaced.
  // One kernel, no workspace.
  if (cp.y == 1 && cp.x == 1 && cp.sh == 1 && cp.sw == 1 && cp.ph == 0 && cp.pw == 0 && cp.g == 1 &&
      cp.hi * cp.wi <= INT32_MAX && cp.n * cp.hi * cp.wi <= INT32_MAX && bool_or(o, "pointwise_as_gemm", true) &&
      bool_or(o, "layout_conversion", true)) {
    const int64_t P = cp.hi * cp.wi;
    const bool lin_x = cp.is[3] == cp.wi * cp.is[4], lin_y = cp.os[3] == cp.wo * cp.os[4];
    RockGemmParams gp;
    std::memset(&gp, 0, sizeof gp);
    bool shaped = false, pixels = false;
    if (lin_x && lin_y && cp.is[4] == 1 && cp.os[4] == 1) { // pixels contiguous
      pixels = true;
      gp.G = (int)cp.n; gp.M = (int)cp.c; gp.N = (int)P; gp.K = (int)cp.k;
      gp.a_gs = 0; gp.a_ms = cp.fs[2]; gp.a_ks = cp.fs[1];
      gp.b_gs = cp.os[0]; gp.b_ns = 1; gp.b_ks = cp.os[2];
      gp.c_gs = cp.is[0]; gp.c_ms = cp.is[2]; gp.c_ns = 1;
      shaped = true;
    } else if (lin_x && lin_y && cp.is[2] == 1 && cp.os[2] == 1) { // channels contiguous
      const bool whole = cp.is[0] == P * cp.is[4] && cp.os[0] == P * cp.os[4];
      gp.G = whole ? 1 : (int)cp.n; gp.M = (int)(whole ? cp.n * P : P); gp.N = (int)cp.c; gp.K = (int)cp.k;
      gp.a_gs = whole ? 0 : cp.os[0]; gp.a_ms = cp.os[4]; gp.a_ks = 1;
      gp.b_gs = 0; gp.b_ns = cp.fs[2]; gp.b_ks = cp.fs[1];
      gp.c_gs = whole ? 0 : cp.is[0]; gp.c_ms = cp.is[4]; gp.c_ns = 1;
      shaped = true;
    }
    if (shaped) {
      default_epilogue(gp.epi, cp.ti);
      auto *h = new Handle;
      if (plan_gemm_kernel(h, gp, operand_code(cp.ti, cp.ti), es, o)) {
        if (kid != 0) {
          delete h;
          set_error("conv: kernel_id out of range");
          return nullptr;
        }
        h->op = OP_GEMM;
        h->params.assign(sizeof gp, 0);
        std::memcpy(h->params.data(), &gp, sizeof gp);
        h->epi = &reinterpret_cast<RockGemmParams *>(h->params.data())->epi;
        // GEMM A, B, C from the caller's filter, input (written), output
        h->ptr_map = pixels ? std::vector<Handle::PtrSrc>{{0, 0}, {2, 0}, {1, 0}, {-1, 0}, {-1, 0}}
                            : std::vector<Handle::PtrSrc>{{2, 0}, {0, 0}, {1, 0}, {-1, 0}, {-1, 0}};
        h->problem_key = conv_problem_key(h, o, cp, 2);
        h->kernel_count = 1;
        h->workspace_bytes = 0;
        h->caller_pointers = 4;
        return h;
      }
      delete h;
    }
  }
  struct Phase {
    BwdAxis h, w;
    int64_t rh, rw;
  };
  std::vector<Phase> phases;
  bool need_fill = false;
  for (int64_t rh = 0; rh < cp.sh; ++rh)
    for (int64_t rw = 0; rw < cp.sw; ++rw) {
      Phase ph{bwd_data_axis(rh, cp.sh, cp.dh, cp.y, cp.ph, cp.hi), bwd_data_axis(rw, cp.sw, cp.dw, cp.x, cp.pw, cp.wi),
               rh, rw};
      if (ph.h.A == 0 || ph.w.A == 0)
        continue; // no input position in this phase
      if (ph.h.T == 0 || ph.w.T == 0) {
        need_fill = true; // positions no tap reaches
        continue;
      }
      phases.push_back(ph);
    }
  // the convolution of one phase over the caller's tensors as they lie
  auto phase_view = [&](const Phase &ph, int64_t &fil_off, int64_t &out_off) {
    RockConvParams q;
    std::memset(&q, 0, sizeof q);
    q.n = (int)cp.n; q.g = (int)cp.g; q.c = (int)cp.k; q.k = (int)cp.c;
    q.hi = (int)cp.ho; q.wi = (int)cp.wo; q.y = (int)ph.h.T; q.x = (int)ph.w.T;
    q.ho = (int)ph.h.A; q.wo = (int)ph.w.A;
    q.stride_h = q.stride_w = 1;
    q.dil_h = (int)ph.h.dd; q.dil_w = (int)ph.w.dd;
    q.pad_h = (int)((ph.h.T - 1) * ph.h.dd - ph.h.o_first - ph.h.a_min);
    q.pad_w = (int)((ph.w.T - 1) * ph.w.dd - ph.w.o_first - ph.w.a_min);
    q.in_ns = cp.os[0]; q.in_gs = cp.os[1]; q.in_cs = cp.os[2]; q.in_hs = cp.os[3]; q.in_ws = cp.os[4];
    q.fil_gs = cp.fs[0]; q.fil_ks = cp.fs[2]; q.fil_cs = cp.fs[1];
    q.fil_ys = -ph.h.y_step * cp.fs[3]; q.fil_xs = -ph.w.y_step * cp.fs[4];
    fil_off = (ph.h.y_first + (ph.h.T - 1) * ph.h.y_step) * cp.fs[3] +
              (ph.w.y_first + (ph.w.T - 1) * ph.w.y_step) * cp.fs[4];
    q.out_ns = cp.is[0]; q.out_gs = cp.is[1]; q.out_ks = cp.is[2];
    q.out_hs = cp.sh * cp.is[3]; q.out_ws = cp.sw * cp.is[4];
    out_off = (cp.sh * ph.h.a_min + ph.rh - cp.ph) * cp.is[3] + (cp.sw * ph.w.a_min + ph.rw - cp.pw) * cp.is[4];
    default_epilogue(q.epi, cp.ti);
    return q;
  };
  // the same with the sub-filter and the output gradient converted to the
  // vector kernels' form (reduction channel k contiguous, whole 16-byte chunks)
  const int64_t kp = (cp.k * es + 15) / 16 * 16 / es;
  auto al = [&](int64_t elems) { return (elems * es) % 16 == 0; };
  const bool dy_as_is = cp.os[2] == 1 && kp == cp.k && al(cp.os[4]) && al(cp.os[3]) && al(cp.os[0]) && al(cp.os[1]);
  const int64_t dy_bytes = dy_as_is ? 0 : align256(cp.n * cp.ho * cp.wo * cp.g * kp * es);
  auto phase_fast_view = [&](const Phase &ph, int64_t &out_off) {
    int64_t unused;
    RockConvParams q = phase_view(ph, unused, out_off);
    q.c = (int)kp;
    q.fil_cs = 1; q.fil_xs = kp; q.fil_ys = ph.w.T * kp; q.fil_ks = ph.h.T * ph.w.T * kp; q.fil_gs = cp.c * q.fil_ks;
    if (!dy_as_is) {
      q.in_cs = 1; q.in_gs = kp; q.in_ws = cp.g * kp; q.in_hs = cp.wo * q.in_ws; q.in_ns = cp.ho * q.in_hs;
    }
    return q;
  };
  bool fast = bool_or(o, "layout_conversion", true);
  for (const Phase &ph : phases) {
    int64_t unused;
    fast = fast && conv_view_fast(phase_fast_view(ph, unused), es);
  }
  // A strided layer with few input channels (the 3-channel first layer): each phase alone fills 3 of the 64
  // output columns of a tile.  The phases read the same neighbourhood of the output gradient, so they run as
  // ONE unit-stride convolution whose output columns are (phase, channel): its window is the union of the
  // offsets that any phase reaches, its filter [(phase, c)][u_h][u_w][k] holds every phase's flipped taps at
  // their offsets and zeros elsewhere, and its output T[n][b_h][b_w][(j_h, j_w, c)] (in the workspace) is the
  // input gradient with the position i = stride * b + j taken apart; a conversion kernel puts it together.
  // Kernels: [output gradient copy], zero fill of the filter, one filter conversion per phase, the
  // convolution, T -> channels-last gradient, [-> the caller's layout].
  if (fast && phases.size() > 1 && (int64_t)phases.size() == cp.sh * cp.sw && !need_fill && cp.g == 1 &&
      cp.dh == 1 && cp.dw == 1 && cp.hi % cp.sh == 0 && cp.wi % cp.sw == 0 && (int64_t)phases.size() * cp.c <= 64 &&
      bool_or(o, "merge_phases", true)) {
    const int64_t P = (int64_t)phases.size(), Bh = cp.hi / cp.sh, Bw = cp.wi / cp.sw, cols = P * cp.c;
    int64_t lo_h = INT64_MAX, hi_h = INT64_MIN, lo_w = INT64_MAX, hi_w = INT64_MIN;
    bool regular = true;
    for (const Phase &ph : phases) {
      const int64_t eh = ph.h.a_min + ph.h.o_first, ew = ph.w.a_min + ph.w.o_first;
      lo_h = std::min(lo_h, eh - (ph.h.T - 1)); hi_h = std::max(hi_h, eh);
      lo_w = std::min(lo_w, ew - (ph.w.T - 1)); hi_w = std::max(hi_w, ew);
      regular = regular && ph.h.dd == 1 && ph.w.dd == 1 && ph.h.A == Bh && ph.w.A == Bw;
    }
    const int64_t Uh = hi_h - lo_h + 1, Uw = hi_w - lo_w + 1;
    RockConvParams q;
    std::memset(&q, 0, sizeof q);
    q.n = (int)cp.n; q.g = 1; q.c = (int)kp; q.k = (int)cols;
    q.hi = (int)cp.ho; q.wi = (int)cp.wo; q.y = (int)Uh; q.x = (int)Uw; q.ho = (int)Bh; q.wo = (int)Bw;
    q.stride_h = q.stride_w = q.dil_h = q.dil_w = 1;
    q.pad_h = (int)-lo_h; q.pad_w = (int)-lo_w;
    if (dy_as_is) {
      q.in_ns = cp.os[0]; q.in_gs = cp.os[1]; q.in_cs = cp.os[2]; q.in_hs = cp.os[3]; q.in_ws = cp.os[4];
    } else {
      q.in_cs = 1; q.in_gs = kp; q.in_ws = kp; q.in_hs = cp.wo * kp; q.in_ns = cp.ho * q.in_hs;
    }
    q.fil_cs = 1; q.fil_xs = kp; q.fil_ys = Uw * kp; q.fil_ks = Uh * Uw * kp; q.fil_gs = cols * q.fil_ks;
    q.out_ks = 1; q.out_ws = cols; q.out_hs = Bw * cols; q.out_ns = Bh * Bw * cols; q.out_gs = 0;
    default_epilogue(q.epi, cp.ti);
    // the gradient in the caller's tensor when that is dense channels-last, else by way of such a copy
    const bool cl = cp.is[2] == 1 && cp.is[4] == cp.c && cp.is[3] == cp.wi * cp.c && cp.is[0] == cp.hi * cp.wi * cp.c;
    std::vector<ViewDim> to_layout = {{cp.n, cp.n, cp.hi * cp.wi * cp.c, cp.is[0]}, {cp.c, cp.c, 1, cp.is[2]},
                                      {cp.hi, cp.hi, cp.wi * cp.c, cp.is[3]}, {cp.wi, cp.wi, cp.c, cp.is[4]}};
    std::stable_sort(to_layout.begin(), to_layout.end(), [](const ViewDim &a, const ViewDim &b) { return a.ds > b.ds; });
    // (moved as 4-byte words when the runs of s_w * c elements are whole words: every stride and offset is
    // a multiple of such a run)
    const int64_t wide = (es < 4 && (cp.sw * cp.c * es) % 4 == 0) ? 4 / es : 1;
    const int es_scatter = (int)(es * wide);
    const std::vector<ViewDim> scatter = {{cp.n, cp.n, Bh * Bw * cols / wide, cp.hi * cp.wi * cp.c / wide},
                                          {Bh, Bh, Bw * cols / wide, cp.sh * cp.wi * cp.c / wide},
                                          {cp.sh, cp.sh, cp.sw * cp.c / wide, cp.wi * cp.c / wide},
                                          {Bw, Bw, cols / wide, cp.sw * cp.c / wide},
                                          {cp.sw * cp.c / wide, cp.sw * cp.c / wide, 1, 1}};
    bool take = regular && lo_h <= 0 && lo_w <= 0 && conv_view_fast(q, es) && (cl || to_layout.back().ds == 1) &&
                cp.n * cp.hi * cp.wi * cp.c <= INT32_MAX;
    if (take) {
      const std::string keep_error = g_last_error;
      Handle probe;
      take = relayout_handle_nd(&probe, scatter, es_scatter, "input gradient") &&
             (cl || relayout_handle_nd(&probe, to_layout, es, "input gradient"));
      g_last_error = keep_error;
    }
    if (take) {
      const int64_t fil_off_ws = dy_bytes, t_off = fil_off_ws + align256(cols * Uh * Uw * kp * es);
      const int64_t cl_off = t_off + align256(cp.n * Bh * Bw * cols * es);
      const int64_t total = cl_off + (cl ? 0 : align256(cp.n * cp.hi * cp.wi * cp.c * es));
      const int pre = dy_as_is ? 0 : 1, count = pre + 1 + (int)P + 2 + (cl ? 0 : 1);
      if (kid < 0 || kid >= count) {
        set_error("conv: kernel_id out of range");
        return nullptr;
      }
      const int ws = 4;
      Handle *h = nullptr;
      int idx = kid - pre;
      if (idx < 0) {
        h = new Handle;
        const int64_t size[5] = {cp.n, cp.ho, cp.wo, 1, kp}, src_size[5] = {cp.n, cp.ho, cp.wo, 1, cp.k};
        const int64_t stride[5] = {cp.os[0], cp.os[3], cp.os[4], cp.os[1], cp.os[2]};
        if (!fill_relayout_handle(h, size, src_size, stride, es)) {
          delete h;
          return nullptr;
        }
        h->ptr_map = {{2, 0}, {ws, 0}};
        h->problem_key = "relayout output gradient " + cp.ol;
      } else if (idx == 0) {
        h = utility_fill_handle(cols * Uh * Uw * kp * es);
        h->ptr_map = {{ws, fil_off_ws}};
        h->problem_key = "zero fill of the merged filter";
      } else if (idx <= P) {
        const Phase &ph = phases[idx - 1];
        int64_t fil_off, out_off;
        const RockConvParams generic = phase_view(ph, fil_off, out_off);
        // the phase's columns and where its window starts inside the union
        const int64_t jh = cp.sh * ph.h.a_min + ph.rh - cp.ph, jw = cp.sw * ph.w.a_min + ph.rw - cp.pw;
        const int64_t uh0 = ph.h.a_min + ph.h.o_first - (ph.h.T - 1) - lo_h, uw0 = ph.w.a_min + ph.w.o_first - (ph.w.T - 1) - lo_w;
        const int64_t size[5] = {1, cp.c, ph.h.T, ph.w.T, kp}, src_size[5] = {1, cp.c, ph.h.T, ph.w.T, cp.k};
        const int64_t stride[5] = {generic.fil_gs, generic.fil_ks, generic.fil_ys, generic.fil_xs, generic.fil_cs};
        const int64_t dst_stride[5] = {q.fil_gs, q.fil_ks, q.fil_ys, q.fil_xs, 1};
        h = new Handle;
        if (!fill_relayout_handle(h, size, src_size, stride, es, dst_stride)) {
          delete h;
          return nullptr;
        }
        const int64_t dst_off = (jh * cp.sw + jw) * cp.c * q.fil_ks + uh0 * q.fil_ys + uw0 * q.fil_xs;
        h->ptr_map = {{0, fil_off * es}, {ws, fil_off_ws + dst_off * es}};
        h->problem_key = "relayout filter phase " + std::to_string(ph.rh) + "," + std::to_string(ph.rw);
      } else if (idx == P + 1) {
        h = conv_handle_from_view(q, cp.ti, o);
        if (!h)
          return nullptr;
        h->ptr_map = {{ws, fil_off_ws}, dy_as_is ? Handle::PtrSrc{2, 0} : Handle::PtrSrc{ws, 0}, {ws, t_off}, {-1, 0}, {-1, 0}};
        h->problem_key = conv_problem_key(h, o, cp, 2);
      } else {
        h = new Handle;
        const bool last = idx == P + 3;
        if (!relayout_handle_nd(h, last ? to_layout : scatter, last ? es : es_scatter, "input gradient")) {
          delete h;
          return nullptr;
        }
        h->ptr_map = last ? std::vector<Handle::PtrSrc>{{ws, cl_off}, {1, 0}}
                          : std::vector<Handle::PtrSrc>{{ws, t_off}, cl ? Handle::PtrSrc{1, 0} : Handle::PtrSrc{ws, cl_off}};
        h->problem_key = last ? "relayout input gradient " + cp.il : "phases of the input gradient put together";
      }
      h->kernel_count = count;
      h->workspace_bytes = (size_t)total;
      h->caller_pointers = 5;
      return h;
    }
  }
  // Phases that the window-resident kernel takes (unit stride: the one phase there is): the conversion of the
  // flipped sub-filter then writes it fragment-major,
  //   F'[g][32-channel block of c][(t_h, t_w, 16-byte chunk of k)][channel][k in chunk],
  // for that kernel instead of as K-contiguous rows.  One conversion kernel has to do (five independent
  // dimensions: one group, taps that fold), else the phase stays on the implicit-GEMM kernel.
  const int64_t ek = 16 / es; // elements per chunk
  auto window_filter_dims = [&](const Phase &ph, const RockConvParams &generic, const WindowPlan &w) {
    const int64_t chunks = kp / ek, tap = 32 * kp; // elements of one tap of one channel block in F'
    std::vector<ViewDim> dims = {
        {cp.g, cp.g, generic.fil_gs, w.tiles_n * 4 * ph.h.T * ph.w.T * tap},
        {w.tiles_n * 4, cp.c / 32, 32 * generic.fil_ks, ph.h.T * ph.w.T * tap},
        {ph.h.T, ph.h.T, generic.fil_ys, ph.w.T * tap},
        {ph.w.T, ph.w.T, generic.fil_xs, tap},
        {chunks, chunks, ek * generic.fil_cs, 32 * ek},
        {32, 32, generic.fil_ks, ek},
        {ek, ek, generic.fil_cs, 1}};
    return dims;
  };
  std::vector<WindowPlan> win(phases.size());
  if (fast && kp == cp.k) {
    const std::string keep_error = g_last_error;
    for (size_t i = 0; i < phases.size(); ++i) {
      int64_t u0, u1;
      const RockConvParams q = phase_fast_view(phases[i], u0);
      // (the view's padding is equal on both sides when the last output row ends where the padded input does)
      const bool equal = q.ho - 1 + q.y - 1 - q.pad_h - (q.hi - 1) == q.pad_h &&
                         q.wo - 1 + q.x - 1 - q.pad_w - (q.wi - 1) == q.pad_w;
      const WindowPlan w = window_plan(q, cp.ti, equal, o);
      if (!w.by_itself)
        continue;
      Handle probe;
      if (relayout_handle_nd(&probe, window_filter_dims(phases[i], phase_view(phases[i], u0, u1), w), es, "filter"))
        win[i] = w;
    }
    g_last_error = keep_error;
  }
  // A single phase (unit stride) with few output tiles and a long reduction: the (taps, k) range split over
  // blocks as in the forward direction (make_conv), partial sums in the workspace, a reduction kernel
  // behind the contraction that writes the input gradient.
  int64_t S = 1, k_part = 0, part_off = 0, part_bytes = 0;
  if (fast && phases.size() == 1 && !win[0].ok && cp.g == 1 && bool_or(o, "split_k", true)) {
    const Phase &ph = phases[0];
    const int64_t Mg = cp.n * ph.h.A * ph.w.A, Kfull = kp * ph.h.T * ph.w.T, step = 128 / es;
    const int64_t tiles64 = (int64_t)ceil_div(Mg, 64) * ceil_div(cp.c, 64);
    const int64_t s_req = requested_block_splits(o); // a perf_config names the split itself
    auto share_ok = [&](int64_t d) { return Kfull % d == 0 && (Kfull / d) % step == 0; };
    if (Mg * cp.c <= INT32_MAX) {
      if (s_req > 1 && share_ok(s_req))
        S = s_req;
      else if (s_req < 0 && tiles64 <= 2 * kNumCU && Kfull >= 2048) {
        const int64_t want = std::min<int64_t>(4 * kNumCU / tiles64, Kfull / 1024);
        for (int64_t d = want; d >= 2; --d)
          if (share_ok(d)) {
            S = d;
            break;
          }
      }
      if (S > 1) {
        k_part = Kfull / S;
        part_bytes = align256(S * Mg * cp.c * 4);
      }
    }
  }
  // kernel list
  const int first_phase = (need_fill ? 1 : 0) + (fast && !dy_as_is ? 1 : 0);
  const int per_phase = fast ? (S > 1 ? 3 : 2) : 1;
  const int count = first_phase + per_phase * (int)phases.size();
  int64_t workspace = 0;
  std::vector<int64_t> fil_ws(phases.size(), 0);
  if (fast) {
    workspace = dy_bytes;
    for (size_t i = 0; i < phases.size(); ++i) {
      fil_ws[i] = workspace;
      workspace += win[i].ok ? win[i].filter_bytes : align256(cp.g * cp.c * phases[i].h.T * phases[i].w.T * kp * es);
    }
    part_off = workspace;
    workspace += part_bytes;
  }
  if (count == 0 || kid < 0 || kid >= count) {
    set_error(count == 0 ? "conv_bwd_data: empty problem" : "conv: kernel_id out of range");
    return nullptr;
  }
  Handle *h = nullptr;
  const int ws = 4; // filter, input, output, unused, workspace
  int idx = kid;
  if (need_fill && idx-- == 0) {
    h = utility_fill_handle(cp.n * cp.g * cp.c * cp.hi * cp.wi * es);
    h->ptr_map = {{1, 0}};
    h->problem_key = "zero fill of the input gradient";
  } else if (fast && !dy_as_is && idx-- == 0) {
    h = new Handle;
    const int64_t size[5] = {cp.n, cp.ho, cp.wo, cp.g, kp}, src_size[5] = {cp.n, cp.ho, cp.wo, cp.g, cp.k};
    const int64_t stride[5] = {cp.os[0], cp.os[3], cp.os[4], cp.os[1], cp.os[2]};
    if (!fill_relayout_handle(h, size, src_size, stride, es)) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{2, 0}, {ws, 0}};
    h->problem_key = "relayout output gradient " + cp.ol;
  } else {
    const Phase &ph = phases[idx / per_phase];
    const int64_t fil_dst = fil_ws[idx / per_phase];
    int64_t fil_off, out_off;
    const RockConvParams generic = phase_view(ph, fil_off, out_off);
    const WindowPlan &w = win[idx / per_phase];
    if (fast && idx % per_phase == 2) {
      // the split's partial sums [S][n][a_h][a_w][c] added into the phase's positions of the input gradient
      const int64_t Mg = cp.n * ph.h.A * ph.w.A;
      RockReduceParams r;
      std::memset(&r, 0, sizeof r);
      r.split_stride = Mg * cp.c;
      r.size[0] = (int)cp.n; r.size[1] = (int)ph.h.A; r.size[2] = (int)ph.w.A; r.size[3] = (int)cp.c;
      r.dst_stride[0] = generic.out_ns; r.dst_stride[1] = generic.out_hs; r.dst_stride[2] = generic.out_ws;
      r.dst_stride[3] = generic.out_ks;
      r.splits = (int)S;
      r.out_dtype = cp.ti;
      h = new Handle;
      h->op = OP_RELAYOUT;
      h->epi = nullptr;
      h->params.assign(sizeof r, 0);
      std::memcpy(h->params.data(), &r, sizeof r);
      h->kernel_name = "rock_reduce_splits";
      h->block_size = 256;
      h->grid_size = (uint32_t)((Mg * cp.c + 255) / 256);
      h->num_pointers = 2;
      h->perf_config = "";
      h->ptr_map = {{ws, part_off}, {1, out_off * es}};
      h->problem_key = "reduction of the split partial sums";
    } else if (fast && idx % per_phase == 0) {
      // flipped sub-filter -> [g][c][T_h][T_w][kp], or fragment-major for the window-resident kernel
      h = new Handle;
      const int64_t size[5] = {cp.g, cp.c, ph.h.T, ph.w.T, kp}, src_size[5] = {cp.g, cp.c, ph.h.T, ph.w.T, cp.k};
      const int64_t stride[5] = {generic.fil_gs, generic.fil_ks, generic.fil_ys, generic.fil_xs, generic.fil_cs};
      if (!(w.ok ? relayout_handle_nd(h, window_filter_dims(ph, generic, w), es, "filter")
                 : fill_relayout_handle(h, size, src_size, stride, es))) {
        delete h;
        return nullptr;
      }
      h->ptr_map = {{0, fil_off * es}, {ws, fil_dst}};
      h->problem_key = "relayout filter phase " + std::to_string(ph.rh) + "," + std::to_string(ph.rw);
    } else {
      int64_t off2;
      RockConvParams view = fast ? phase_fast_view(ph, off2) : generic;
      if (S > 1) { // the shares of the reduction as groups, each into its own f32 partial result
        view.g = (int)S;
        view.k_group_stride = (int)k_part;
        view.in_gs = 0;
        view.fil_gs = k_part;
        view.out_ks = 1; view.out_ws = cp.c; view.out_hs = ph.w.A * cp.c; view.out_ns = ph.h.A * ph.w.A * cp.c;
        view.out_gs = cp.n * view.out_ns;
        view.epi.out_dtype = ROCK_F32;
      }
      h = conv_handle_from_view(view, cp.ti, o);
      if (!h)
        return nullptr;
      if (S > 1) {
        reinterpret_cast<RockConvParams *>(h->params.data())->K = (int)k_part;
        h->perf_config = with_block_splits(h->perf_config, S);
      }
      if (w.ok)
        apply_window_plan(h, *reinterpret_cast<RockConvParams *>(h->params.data()), w, cp.ti, o);
      h->ptr_map = {fast ? Handle::PtrSrc{ws, fil_dst} : Handle::PtrSrc{0, fil_off * es},
                    (fast && !dy_as_is) ? Handle::PtrSrc{ws, 0} : Handle::PtrSrc{2, 0},
                    S > 1 ? Handle::PtrSrc{ws, part_off} : Handle::PtrSrc{1, out_off * es}, {-1, 0}, {-1, 0}};
      h->problem_key = conv_problem_key(h, o, cp, 2);
    }
  }
  h->kernel_count = count;
  h->workspace_bytes = (size_t)workspace;
  h->caller_pointers = workspace ? 5 : 4;
  return h;
}

// Gradient with respect to the filter.  Pointer order as the forward problem:
// filter (written), input, output (the incoming gradient), unused, [workspace].
//   dW[k, c, y, x] = sum over n, ho, wo of  X[n, c, ho*s + y*d - p, ...] * dY[n, k, ho, wo]
// is a forward convolution with the roles re-labelled: its batch is c, its
// reduction channel n, its "filter" the output gradient (spatial size ho x wo),
// its output spatial size y x x, its stride the dilation and its dilation the
// stride.  For the vector kernels both operands are copied with n contiguous;
// with one group the reduction over n is split into S chunks that run as the
// groups of that convolution into f32 partial sums, added up in split order by
// a reduction kernel (the reference's answer is atomic adds into a zero-filled
// f32 workspace, ConvGenerator.cpp:434-480).
// Tensors that are not channels-last are copied into that form in the
// workspace and the filter gradient is planned again over the copies (all
// pixels of all images then form one equally spaced run).  nullptr with no
// error set when the copies would not help (channel runs not in whole 16-byte
// chunks, or conversions switched off).
Handle *make_conv_bwd_weight(const OptMap &o, const ConvProblem &cp);
Handle *bwd_weight_over_channels_last_copies(const OptMap &o, const ConvProblem &cp, bool &applies) {
  const int es = dtype_size(cp.ti);
  const int kid = (int)int_or(o, "kernel_id", 0);
  const bool cl_in = cp.is[2] == 1, cl_out = cp.os[2] == 1;
  applies = (!cl_in || !cl_out) && (cp.c * es) % 16 == 0 && (cp.k * es) % 16 == 0 && bool_or(o, "layout_conversion", true);
  if (!applies)
    return nullptr;
  ConvProblem inner = cp;
  const int64_t isz[5] = {cp.n, cp.g, cp.c, cp.hi, cp.wi}, osz[5] = {cp.n, cp.g, cp.k, cp.ho, cp.wo};
  if (!cl_in) {
    inner.il = "nhwgc";
    layout_strides(inner.il, "ngchw", isz, inner.is);
  }
  if (!cl_out) {
    inner.ol = "nhwgk";
    layout_strides(inner.ol, "ngkhw", osz, inner.os);
  }
  const int64_t x_bytes = cl_in ? 0 : align256(cp.n * cp.c * cp.hi * cp.wi * es);
  const int64_t y_bytes = cl_out ? 0 : align256(cp.n * cp.k * cp.ho * cp.wo * es);
  const int pre = (cl_in ? 0 : 1) + (cl_out ? 0 : 1);
  OptMap o2 = o;
  o2["kernel_id"] = std::to_string(std::max(0, kid - pre));
  Handle *sub = make_conv_bwd_weight(o2, inner);
  if (!sub)
    return nullptr;
  const int total = sub->kernel_count + pre;
  const size_t ws_total = (size_t)(x_bytes + y_bytes) + sub->workspace_bytes;
  if (kid < pre) {
    delete sub;
    const bool input = kid == 0 && !cl_in;
    auto *c2 = new Handle;
    const int64_t size_x[5] = {cp.n, cp.hi, cp.wi, cp.g, cp.c}, size_y[5] = {cp.n, cp.ho, cp.wo, cp.g, cp.k};
    const int64_t str_x[5] = {cp.is[0], cp.is[3], cp.is[4], cp.is[1], cp.is[2]};
    const int64_t str_y[5] = {cp.os[0], cp.os[3], cp.os[4], cp.os[1], cp.os[2]};
    if (!fill_relayout_handle(c2, input ? size_x : size_y, input ? size_x : size_y, input ? str_x : str_y, es)) {
      delete c2;
      return nullptr;
    }
    c2->ptr_map = input ? std::vector<Handle::PtrSrc>{{1, 0}, {4, 0}}
                        : std::vector<Handle::PtrSrc>{{2, 0}, {4, x_bytes}};
    c2->problem_key = input ? "relayout input " + cp.il : "relayout output gradient " + cp.ol;
    sub = c2;
  } else {
    for (auto &src : sub->ptr_map) {
      if (src.source == 4)
        src.offset += x_bytes + y_bytes;
      else if (src.source == 1 && !cl_in)
        src = Handle::PtrSrc{4, src.offset};
      else if (src.source == 2 && !cl_out)
        src = Handle::PtrSrc{4, x_bytes + src.offset};
    }
    if (sub->op != OP_RELAYOUT)
      sub->problem_key = conv_problem_key(sub, o, cp, 4);
  }
  sub->kernel_count = total;
  sub->workspace_bytes = ws_total;
  sub->caller_pointers = 5;
  return sub;
}

// Filter gradient of a convolution over images with a few channels (the
// 3-channel first layer of a CNN), one group, no padding or dilation along w.
// The input is copied channels-last with the channel run padded to a power of
// two that divides a 16-byte chunk (3 -> 4 of 16 bits); a row of x filter taps
// then reads x neighbouring pixels, one contiguous run, which is padded to
// whole chunks.  The K-major GEMM of the channels-last route runs over that
// view -- "channels" = the run, a filter one tap wide:
//   dW'[k, (y, run)] = sum over pixels of dY[pixel, k] * X4[n, ho*sh + y*dh - ph, (wo*sw)*cpad + run]
// The columns of a run beyond x taps (the next pixels, or the neighbouring
// row or image at the end of a row) and the padded channels are outputs of
// their own, which the reduction kernel leaves out when it adds up the
// partial sums and writes the caller's layout.  nullptr with `applies` false
// when the problem is not of this kind.
Handle *bwd_weight_narrow_channels(const OptMap &o, const ConvProblem &cp, bool &applies) {
  applies = false;
  const int es = dtype_size(cp.ti);
  const int kid = (int)int_or(o, "kernel_id", 0);
  if (!(cp.g == 1 && (cp.ti == ROCK_F32 || cp.ti == ROCK_F16 || cp.ti == ROCK_BF16) && cp.y * cp.x > 1 &&
        bool_or(o, "bwd_weight_gemm", true) && bool_or(o, "layout_conversion", true)))
    return nullptr;
  int64_t cpad = 1;
  while (cpad < cp.c)
    cpad *= 2;
  const int64_t pix_bytes = cpad * es;
  if ((cp.c * es) % 16 == 0 || pix_bytes > 16 || cp.pw != 0 || cp.dw != 1 || (cp.sw * pix_bytes) % 16 != 0 ||
      (cp.wi * pix_bytes) % 16 != 0 || (cp.k * es) % 16 != 0)
    return nullptr;
  const int64_t run = (cp.x * pix_bytes + 15) / 16 * 16 / es; // elements of a row of taps, in whole chunks
  const int64_t Ng = cp.y * run, P = cp.n * cp.ho * cp.wo;
  const int64_t x_bytes = align256(cp.n * cp.hi * cp.wi * pix_bytes + run * es); // the last run reaches past the end
  if (P > INT32_MAX || Ng > INT32_MAX || x_bytes >= ((int64_t)1 << 31))
    return nullptr;
  auto al = [&](int64_t elems) { return (elems * es) % 16 == 0; };
  const bool dy_ok = cp.os[2] == 1 && cp.os[3] == cp.wo * cp.os[4] && cp.os[0] == cp.ho * cp.os[3] && al(cp.os[4]);
  const int64_t dy_pix = dy_ok ? cp.os[4] : cp.k; // elements between neighbouring pixels of the gradient read
  const Tile &tile = cp.k <= 64 ? kFastTiles[3] : kFastTiles[2]; // 64x64 or 128x128
  const int64_t tiles = (int64_t)ceil_div(cp.k, tile.bm) * ceil_div(Ng, tile.bn);
  const int64_t want = std::max<int64_t>(1, std::min<int64_t>(tile.blocks_per_cu * kNumCU / tiles, P / 256));
  int64_t S = 1;
  for (int64_t d = want; d >= 1; --d)
    if (P % d == 0) {
      S = d;
      break;
    }
  const int64_t Ks = P / S;
  if (Ks * dy_pix * es >= ((int64_t)1 << 31))
    return nullptr;
  applies = true;
  const int64_t dy_bytes = dy_ok ? 0 : align256(P * cp.k * es);
  const int64_t part_off = x_bytes + dy_bytes, part_bytes = align256(S * cp.k * Ng * 4);
  const int pre = dy_ok ? 1 : 2, count = pre + 2;
  if (kid < 0 || kid >= count) {
    set_error("conv: kernel_id out of range");
    return nullptr;
  }
  auto *h = new Handle;
  if (kid < pre) {
    const bool input = kid == 0;
    // dimensions in the destination's order n, h, w, g, c
    const int64_t size[5] = {cp.n, input ? cp.hi : cp.ho, input ? cp.wi : cp.wo, 1, input ? cpad : cp.k};
    const int64_t src_size[5] = {size[0], size[1], size[2], 1, input ? cp.c : cp.k};
    const int64_t *st = input ? cp.is : cp.os;
    const int64_t stride[5] = {st[0], st[3], st[4], st[1], st[2]};
    if (!fill_relayout_handle(h, size, src_size, stride, es)) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{input ? 1 : 2, 0}, {4, input ? 0 : x_bytes}};
    h->problem_key = input ? "relayout input: channel runs padded to a fraction of a chunk" : "relayout output gradient";
  } else if (kid == pre) {
    RockConvBwdWeightParams bp;
    std::memset(&bp, 0, sizeof bp);
    bp.G = (int)S; bp.M = (int)cp.k; bp.N = (int)Ng; bp.K = (int)Ks;
    bp.a_ms = 1; bp.a_ks = dy_pix; bp.a_gs = Ks * dy_pix;
    bp.c_ms = Ng; bp.c_ns = 1; bp.c_gs = cp.k * Ng;
    default_epilogue(bp.epi, ROCK_F32);
    bp.in_pix_stride = cpad;
    bp.c = (int)run; bp.hi = (int)cp.hi; bp.wi = (int)cp.wi; bp.ho = (int)cp.ho; bp.wo = (int)cp.wo;
    bp.x = 1;
    bp.stride_h = (int)cp.sh; bp.stride_w = (int)cp.sw; bp.pad_h = (int)cp.ph; bp.pad_w = 0;
    bp.dil_h = (int)cp.dh; bp.dil_w = 1;
    apply_tile_grid(tile, cp.k, Ng, (int)S, bp.tiles_m, bp.tiles_n, bp.group_m, bp.xcd_remap, h->block_size,
                    h->grid_size);
    h->op = OP_GEMM;
    h->params.assign(sizeof bp, 0);
    std::memcpy(h->params.data(), &bp, sizeof bp);
    h->epi = &reinterpret_cast<RockConvBwdWeightParams *>(h->params.data())->epi;
    h->kernel_name = std::string("rock_conv_bwd_weight_") + dtype_name(cp.ti) + (tile.bm == 64 ? "_64x64" : "_128x128");
    h->num_pointers = 5;
    h->perf_config = perf_string(tile, es, &o);
    h->ptr_map = {dy_ok ? Handle::PtrSrc{2, 0} : Handle::PtrSrc{4, x_bytes}, {4, 0}, {4, part_off}, {-1, 0}, {-1, 0}};
    h->problem_key = conv_problem_key(h, o, cp, 4);
  } else {
    RockReduceParams r;
    std::memset(&r, 0, sizeof r);
    r.split_stride = cp.k * Ng;
    r.size[0] = (int)cp.k; r.size[1] = (int)cp.y; r.size[2] = (int)(run / cpad); r.size[3] = (int)cpad;
    r.valid[0] = (int)cp.k_valid; r.valid[2] = (int)cp.x; r.valid[3] = (int)cp.c;
    r.dst_stride[0] = cp.fs[1]; r.dst_stride[1] = cp.fs[3]; r.dst_stride[2] = cp.fs[4]; r.dst_stride[3] = cp.fs[2];
    r.splits = (int)S;
    r.out_dtype = cp.ti;
    h->op = OP_RELAYOUT;
    h->epi = nullptr;
    h->params.assign(sizeof r, 0);
    std::memcpy(h->params.data(), &r, sizeof r);
    h->kernel_name = "rock_reduce_splits";
    h->block_size = 256;
    h->grid_size = (uint32_t)((cp.k * Ng + 255) / 256);
    h->num_pointers = 2;
    h->perf_config = "";
    h->ptr_map = {{4, part_off}, {0, 0}};
    h->problem_key = "reduction of the split partial sums";
  }
  h->kernel_count = count;
  h->workspace_bytes = (size_t)(part_off + part_bytes);
  h->caller_pointers = 5;
  return h;
}

Handle *make_conv_bwd_weight(const OptMap &o, const ConvProblem &cp) {
  // A strided 1x1 filter without padding touches one input pixel in
  // stride_h * stride_w.  A first kernel gathers those into the workspace
  // (ho x wo pixels, channels last when the channel runs are whole 16-byte
  // chunks, else in the caller's letter order); what remains is the
  // unit-stride problem over the gathered tensor, planned as such (a split GEMM
  // over the tensors as they lie when the runs are whole 16-byte chunks).
  if (cp.y == 1 && cp.x == 1 && cp.ph == 0 && cp.pw == 0 && (cp.sh > 1 || cp.sw > 1) &&
      bool_or(o, "layout_conversion", true) && bool_or(o, "pointwise_as_gemm", true)) {
    const int es = dtype_size(cp.ti);
    const int kid = (int)int_or(o, "kernel_id", 0);
    ConvProblem inner = cp;
    inner.hi = cp.ho; inner.wi = cp.wo; inner.sh = inner.sw = 1;
    const int64_t isz[5] = {cp.n, cp.g, cp.c, cp.ho, cp.wo};
    if ((cp.c * es) % 16 == 0)
      inner.il = "nhwgc"; // channel runs of whole chunks: the form the GEMM route reads best
    layout_strides(inner.il, "ngchw", isz, inner.is);
    const int64_t gathered = align256(cp.n * cp.g * cp.c * cp.ho * cp.wo * es);
    OptMap o2 = o;
    o2["kernel_id"] = std::to_string(kid == 0 ? 0 : kid - 1);
    Handle *sub = make_conv_bwd_weight(o2, inner);
    if (!sub)
      return nullptr;
    const int count = sub->kernel_count + 1;
    const size_t workspace = (size_t)gathered + sub->workspace_bytes;
    if (kid == 0) {
      delete sub;
      auto *h = new Handle;
      int64_t size[5], stride[5];
      for (int d = 0; d < 5; ++d) { // dimensions in the order of the gathered tensor's layout
        const size_t idx = std::string("ngchw").find(inner.il[d]);
        size[d] = isz[idx];
        stride[d] = cp.is[idx] * (idx == 3 ? cp.sh : idx == 4 ? cp.sw : 1);
      }
      if (!fill_relayout_handle(h, size, size, stride, es)) {
        delete h;
        return nullptr;
      }
      h->ptr_map = {{1, 0}, {4, 0}};
      h->problem_key = "gather of the input pixels a strided 1x1 filter reads";
      h->kernel_count = count;
      h->workspace_bytes = workspace;
      h->caller_pointers = 5;
      return h;
    }
    // the inner plan's input is the gathered tensor, its workspace lies behind it
    for (auto &src : sub->ptr_map) {
      if (src.source == 4)
        src.offset += gathered;
      else if (src.source == 1)
        src = Handle::PtrSrc{4, src.offset};
    }
    if (sub->op != OP_RELAYOUT)
      sub->problem_key = conv_problem_key(sub, o, cp, 4);
    sub->kernel_count = count;
    sub->workspace_bytes = workspace;
    sub->caller_pointers = 5;
    return sub;
  }
  const int es = dtype_size(cp.ti);
  const int kid = (int)int_or(o, "kernel_id", 0);

  // An output gradient with a few channels (k * es not a whole 16-byte chunk: a layer that ends in 4
  // channels): a first kernel copies it channels-last with the k run padded with zeros to whole chunks,
  // which the K-major GEMM route below reads; the rows of the gradient beyond k come out zero and the
  // reduction kernel leaves them out (k_valid).  Only where that route is certain to take the padded
  // problem (more than one tap, one group, channel runs of the input in whole chunks).
  if (!cp.k_valid && cp.g == 1 && cp.y * cp.x > 1 && (cp.k * es) % 16 != 0 && (cp.c * es) % 16 == 0 &&
      (cp.ti == ROCK_F32 || cp.ti == ROCK_F16 || cp.ti == ROCK_BF16) && bool_or(o, "bwd_weight_gemm", true) &&
      bool_or(o, "layout_conversion", true)) {
    const int64_t kpad = (cp.k * es + 15) / 16 * 16 / es;
    ConvProblem inner = cp;
    inner.k = kpad;
    inner.k_valid = cp.k;
    inner.ol = "nhwgk";
    const int64_t osz[5] = {cp.n, cp.g, kpad, cp.ho, cp.wo};
    layout_strides(inner.ol, "ngkhw", osz, inner.os);
    const int64_t dy_bytes = align256(cp.n * cp.ho * cp.wo * kpad * es);
    const std::string keep_error = g_last_error;
    // the padded problem ends in rock_conv_bwd_weight_* and the reduction kernel when the GEMM route took it
    // (decided on the plan as a whole, whatever kernel_id asks for)
    bool took = false;
    int inner_count = 0;
    {
      OptMap probe = o;
      probe["kernel_id"] = "0";
      Handle *first = make_conv_bwd_weight(probe, inner);
      inner_count = first ? first->kernel_count : 0;
      delete first;
      if (inner_count >= 2) {
        probe["kernel_id"] = std::to_string(inner_count - 2);
        Handle *gemm = make_conv_bwd_weight(probe, inner);
        probe["kernel_id"] = std::to_string(inner_count - 1);
        Handle *last = make_conv_bwd_weight(probe, inner);
        took = gemm && last && gemm->kernel_name.rfind("rock_conv_bwd_weight_", 0) == 0 &&
               last->kernel_name == "rock_reduce_splits";
        delete gemm;
        delete last;
      }
    }
    Handle *sub = nullptr;
    if (took) {
      if (kid < 0 || kid > inner_count) {
        set_error("conv: kernel_id out of range");
        return nullptr;
      }
      OptMap o2 = o;
      o2["kernel_id"] = std::to_string(kid == 0 ? 0 : kid - 1);
      sub = make_conv_bwd_weight(o2, inner);
      if (!sub)
        return nullptr;
    }
    if (took) {
      const int count = sub->kernel_count + 1;
      const size_t workspace = (size_t)dy_bytes + sub->workspace_bytes;
      if (kid == 0) {
        delete sub;
        auto *h = new Handle;
        // dimensions in the destination's order n, h, w, g, k
        const int64_t size[5] = {cp.n, cp.ho, cp.wo, 1, kpad}, src_size[5] = {cp.n, cp.ho, cp.wo, 1, cp.k};
        const int64_t stride[5] = {cp.os[0], cp.os[3], cp.os[4], cp.os[1], cp.os[2]};
        if (!fill_relayout_handle(h, size, src_size, stride, es)) {
          delete h;
          return nullptr;
        }
        h->ptr_map = {{2, 0}, {4, 0}};
        h->problem_key = "relayout output gradient: channel runs padded to whole chunks";
        h->kernel_count = count;
        h->workspace_bytes = workspace;
        h->caller_pointers = 5;
        return h;
      }
      // the inner plan reads the copy; its own workspace lies behind it
      for (auto &src : sub->ptr_map) {
        if (src.source == 4)
          src.offset += dy_bytes;
        else if (src.source == 2)
          src = Handle::PtrSrc{4, src.offset};
      }
      if (sub->op != OP_RELAYOUT)
        sub->problem_key = conv_problem_key(sub, o, cp, 4);
      sub->kernel_count = count;
      sub->workspace_bytes = workspace;
      sub->caller_pointers = 5;
      return sub;
    }
    delete sub;
    g_last_error = keep_error; // not taken: the plans below see the problem as it is
  }
  RockConvParams q;
  std::memset(&q, 0, sizeof q);
  q.n = (int)cp.c; q.g = (int)cp.g; q.c = (int)cp.n; q.k = (int)cp.k;
  q.hi = (int)cp.hi; q.wi = (int)cp.wi; q.y = (int)cp.ho; q.x = (int)cp.wo; q.ho = (int)cp.y; q.wo = (int)cp.x;
  q.stride_h = (int)cp.dh; q.stride_w = (int)cp.dw; q.dil_h = (int)cp.sh; q.dil_w = (int)cp.sw;
  q.pad_h = (int)cp.ph; q.pad_w = (int)cp.pw;
  q.in_ns = cp.is[2]; q.in_gs = cp.is[1]; q.in_cs = cp.is[0]; q.in_hs = cp.is[3]; q.in_ws = cp.is[4];
  q.fil_gs = cp.os[1]; q.fil_ks = cp.os[2]; q.fil_cs = cp.os[0]; q.fil_ys = cp.os[3]; q.fil_xs = cp.os[4];
  q.out_ns = cp.fs[2]; q.out_gs = cp.fs[0]; q.out_ks = cp.fs[1]; q.out_hs = cp.fs[3]; q.out_ws = cp.fs[4];
  default_epilogue(q.epi, cp.ti);

  // 1x1 filter, unit stride, no padding, one group, pixels equally spaced in
  // both tensors: dW[k, c] = sum over pixels of dY[pixel, k] * X[pixel, c] is a
  // plain GEMM over the tensors as they lie -- both operands K-major when the
  // channels are contiguous (NHWC), both K-contiguous when the pixels are
  // (NCHW, one GEMM per image).  The pixel range is cut into S batch entries
  // whose f32 partial results the reduction kernel adds up.
  {
    const bool lin_x = cp.is[3] == cp.wi * cp.is[4], lin_y = cp.os[3] == cp.wo * cp.os[4];
    const bool all_x = lin_x && cp.is[0] == cp.hi * cp.is[3], all_y = lin_y && cp.os[0] == cp.ho * cp.os[3];
    if (cp.y == 1 && cp.x == 1 && cp.sh == 1 && cp.sw == 1 && cp.ph == 0 && cp.pw == 0 && cp.g == 1 && lin_x && lin_y &&
        bool_or(o, "pointwise_as_gemm", true)) {
      const int64_t P = cp.hi * cp.wi;
      const bool whole = all_x && all_y; // pixels of all images form one equally spaced run
      const int64_t Ktot = whole ? cp.n * P : P;
      // enough batch entries to fill the chip, each a divisor's share of the pixels
      int64_t S = 1;
      if (whole) {
        const int64_t tiles = (int64_t)ceil_div(cp.k, 128) * ceil_div(cp.c, 128);
        const int64_t want = std::max<int64_t>(1, std::min<int64_t>(2 * kNumCU / tiles, Ktot / 256));
        for (int64_t d = want; d >= 1; --d)
          if (Ktot % d == 0) {
            S = d;
            break;
          }
      } else {
        S = cp.n;
      }
      const int64_t Ks = whole ? Ktot / S : P;
      RockGemmParams gp;
      std::memset(&gp, 0, sizeof gp);
      gp.G = (int)S; gp.M = (int)cp.k; gp.N = (int)cp.c; gp.K = (int)Ks;
      gp.a_ms = cp.os[2]; gp.a_ks = cp.os[4]; gp.a_gs = whole ? Ks * cp.os[4] : cp.os[0];
      gp.b_ns = cp.is[2]; gp.b_ks = cp.is[4]; gp.b_gs = whole ? Ks * cp.is[4] : cp.is[0];
      const int64_t dw = cp.k * cp.c;
      if (S > 1) {
        gp.c_ms = cp.c; gp.c_ns = 1; gp.c_gs = dw;
        default_epilogue(gp.epi, ROCK_F32);
      } else {
        gp.c_ms = cp.fs[1]; gp.c_ns = cp.fs[2]; gp.c_gs = 0;
        default_epilogue(gp.epi, cp.ti);
      }
      const int count = S > 1 ? 2 : 1;
      const int64_t workspace = S > 1 ? align256(S * dw * 4) : 0;
      auto *h = new Handle;
      bool ok = false;
      if (kid == 0) {
        ok = Ks <= INT32_MAX && plan_gemm_kernel(h, gp, operand_code(cp.ti, cp.ti), es, o);
        if (ok) {
          h->op = OP_GEMM;
          h->params.assign(sizeof gp, 0);
          std::memcpy(h->params.data(), &gp, sizeof gp);
          h->epi = &reinterpret_cast<RockGemmParams *>(h->params.data())->epi;
          h->ptr_map = {{2, 0}, {1, 0}, S > 1 ? Handle::PtrSrc{4, 0} : Handle::PtrSrc{0, 0}, {-1, 0}, {-1, 0}};
          h->problem_key = conv_problem_key(h, o, cp, 4);
        }
      } else if (kid == 1 && S > 1) {
        // only reached when kernel 0 took this route as well (same decision below)
        RockGemmParams probe = gp;
        Handle tmp;
        ok = Ks <= INT32_MAX && plan_gemm_kernel(&tmp, probe, operand_code(cp.ti, cp.ti), es, o);
        if (ok) {
          RockReduceParams r;
          std::memset(&r, 0, sizeof r);
          r.split_stride = dw;
          r.size[0] = 1; r.size[1] = 1; r.size[2] = (int)cp.k; r.size[3] = (int)cp.c;
          r.dst_stride[2] = cp.fs[1]; r.dst_stride[3] = cp.fs[2];
          r.splits = (int)S;
          r.out_dtype = cp.ti;
          h->op = OP_RELAYOUT;
          h->epi = nullptr;
          h->params.assign(sizeof r, 0);
          std::memcpy(h->params.data(), &r, sizeof r);
          h->kernel_name = "rock_reduce_splits";
          h->block_size = 256;
          h->grid_size = (uint32_t)((dw + 255) / 256);
          h->num_pointers = 2;
          h->perf_config = "";
          h->ptr_map = {{4, 0}, {0, 0}};
          h->problem_key = "reduction of the split partial sums";
        }
      } else {
        // does the route apply at all?  (a kernel_id beyond its list is an error, not a fallback)
        RockGemmParams probe = gp;
        Handle tmp;
        if (Ks <= INT32_MAX && plan_gemm_kernel(&tmp, probe, operand_code(cp.ti, cp.ti), es, o)) {
          delete h;
          set_error("conv: kernel_id out of range");
          return nullptr;
        }
      }
      if (ok) {
        h->kernel_count = count;
        h->workspace_bytes = (size_t)workspace;
        h->caller_pointers = workspace ? 5 : 4;
        return h;
      }
      delete h; // operands not in whole 16-byte chunks
      // Pixel runs that are not whole chunks (14x14 and 7x7 images in NCHW)
      // while the channel runs are: the tensors that are not channels-last are
      // copied into that form in the workspace and the problem is planned
      // again over the copies (all pixels of all images then form one run).
      {
        bool applies = false;
        Handle *via = bwd_weight_over_channels_last_copies(o, cp, applies);
        if (applies)
          return via;
      }
    }
  }

  // Channels-last input and output gradient, one group, a filter gradient whose
  // (y, x, c) run is contiguous: one K-major GEMM over the tensors as they lie,
  //   dW[k, (y, x, c)] = sum over pixels of dY[pixel, k] * im2col(X)[pixel, (y, x, c)],
  // the second operand gathered by the kernel's loader (no copies), the pixel
  // range cut into S batch entries whose f32 partial results the reduction
  // kernel adds up in split order.  The reference lowers the same contraction
  // through its backward-weight coordinate transforms with atomic adds into a
  // zero-filled workspace (ConvToGemm.cpp:530-768).
  {
    bool applies = false;
    Handle *via = bwd_weight_narrow_channels(o, cp, applies);
    if (applies)
      return via;
  }
  if (cp.g == 1 && (cp.ti == ROCK_F32 || cp.ti == ROCK_F16 || cp.ti == ROCK_BF16) &&
      bool_or(o, "bwd_weight_gemm", true)) {
    auto al = [&](int64_t elems) { return (elems * es) % 16 == 0; };
    const int64_t P = cp.n * cp.ho * cp.wo, Ng = cp.y * cp.x * cp.c;
    const bool in_ok = cp.is[2] == 1 && cp.is[3] == cp.wi * cp.is[4] && cp.is[0] == cp.hi * cp.is[3] && al(cp.c) &&
                       al(cp.is[4]) && cp.n * cp.hi * cp.wi * cp.is[4] * es < ((int64_t)1 << 31);
    const bool dy_ok = cp.os[2] == 1 && cp.os[3] == cp.wo * cp.os[4] && cp.os[0] == cp.ho * cp.os[3] && al(cp.k) &&
                       al(cp.os[4]);
    // a gradient whose (y, x, c) run is contiguous can be written by the GEMM itself when the pixels are
    // not split; any other layout is produced by the reduction kernel from the [k][y][x][c] partial sums
    const bool dw_direct = cp.fs[2] == 1 && cp.fs[4] == cp.c && cp.fs[3] == cp.x * cp.c && cp.fs[1] >= Ng && al(cp.fs[1]) &&
                           !cp.k_valid;
    if (!(in_ok && dy_ok) && cp.y * cp.x > 1 && P <= INT32_MAX && Ng <= INT32_MAX) {
      // not channels-last: copies in that form first (the 1 x 1 case has its own plans below)
      bool applies = false;
      Handle *via = bwd_weight_over_channels_last_copies(o, cp, applies);
      if (applies)
        return via;
    }
    if (in_ok && dy_ok && P <= INT32_MAX && Ng <= INT32_MAX) {
      const Tile &tile = cp.k <= 64 ? kFastTiles[3] : kFastTiles[2]; // 64x64 or 128x128
      const int64_t tiles = (int64_t)ceil_div(cp.k, tile.bm) * ceil_div(Ng, tile.bn);
      // enough batch entries to fill the chip, each a divisor's share of the pixels (at least 256 of them)
      const int64_t want = std::max<int64_t>(1, std::min<int64_t>(tile.blocks_per_cu * kNumCU / tiles, P / 256));
      int64_t S = 1;
      for (int64_t d = want; d >= 1; --d)
        if (P % d == 0) {
          S = d;
          break;
        }
      const int64_t Ks = P / S;
      const bool reduce = S > 1 || !dw_direct;
      const int count = reduce ? 2 : 1;
      const int64_t workspace = reduce ? align256(S * cp.k * Ng * 4) : 0;
      if (Ks * cp.os[4] * es < ((int64_t)1 << 31)) {
        if (kid < 0 || kid >= count) {
          set_error("conv: kernel_id out of range");
          return nullptr;
        }
        auto *h = new Handle;
        if (kid == 0) {
          RockConvBwdWeightParams bp;
          std::memset(&bp, 0, sizeof bp);
          bp.G = (int)S; bp.M = (int)cp.k; bp.N = (int)Ng; bp.K = (int)Ks;
          bp.a_ms = 1; bp.a_ks = cp.os[4]; bp.a_gs = Ks * cp.os[4];
          if (reduce) {
            bp.c_ms = Ng; bp.c_ns = 1; bp.c_gs = cp.k * Ng;
            default_epilogue(bp.epi, ROCK_F32);
          } else {
            bp.c_ms = cp.fs[1]; bp.c_ns = 1; bp.c_gs = 0;
            default_epilogue(bp.epi, cp.ti);
          }
          bp.in_pix_stride = cp.is[4];
          bp.c = (int)cp.c; bp.hi = (int)cp.hi; bp.wi = (int)cp.wi; bp.ho = (int)cp.ho; bp.wo = (int)cp.wo;
          bp.x = (int)cp.x;
          bp.stride_h = (int)cp.sh; bp.stride_w = (int)cp.sw; bp.pad_h = (int)cp.ph; bp.pad_w = (int)cp.pw;
          bp.dil_h = (int)cp.dh; bp.dil_w = (int)cp.dw;
          apply_tile_grid(tile, cp.k, Ng, (int)S, bp.tiles_m, bp.tiles_n, bp.group_m, bp.xcd_remap, h->block_size,
                          h->grid_size);
          h->op = OP_GEMM;
          h->params.assign(sizeof bp, 0);
          std::memcpy(h->params.data(), &bp, sizeof bp);
          h->epi = &reinterpret_cast<RockConvBwdWeightParams *>(h->params.data())->epi;
          h->kernel_name = std::string("rock_conv_bwd_weight_") + dtype_name(cp.ti) + (tile.bm == 64 ? "_64x64" : "_128x128");
          h->num_pointers = 5;
          h->perf_config = perf_string(tile, es, &o);
          h->ptr_map = {{2, 0}, {1, 0}, reduce ? Handle::PtrSrc{4, 0} : Handle::PtrSrc{0, 0}, {-1, 0}, {-1, 0}};
          h->problem_key = conv_problem_key(h, o, cp, 4);
        } else {
          RockReduceParams r;
          std::memset(&r, 0, sizeof r);
          r.split_stride = cp.k * Ng;
          r.size[0] = (int)cp.k; r.size[1] = (int)cp.y; r.size[2] = (int)cp.x; r.size[3] = (int)cp.c;
          r.valid[0] = (int)cp.k_valid;
          r.dst_stride[0] = cp.fs[1]; r.dst_stride[1] = cp.fs[3]; r.dst_stride[2] = cp.fs[4]; r.dst_stride[3] = cp.fs[2];
          r.splits = (int)S;
          r.out_dtype = cp.ti;
          h->op = OP_RELAYOUT;
          h->epi = nullptr;
          h->params.assign(sizeof r, 0);
          std::memcpy(h->params.data(), &r, sizeof r);
          h->kernel_name = "rock_reduce_splits";
          h->block_size = 256;
          h->grid_size = (uint32_t)((cp.k * Ng + 255) / 256);
          h->num_pointers = 2;
          h->perf_config = "";
          h->ptr_map = {{4, 0}, {0, 0}};
          h->problem_key = "reduction of the split partial sums";
        }
        h->kernel_count = count;
        h->workspace_bytes = (size_t)workspace;
        h->caller_pointers = workspace ? 5 : 4;
        return h;
      }
    }
  }

  // split of the reduction over n (one group only: the splits take the group index)
  int64_t S = 1;
  if (cp.g == 1) {
    const int64_t base = (int64_t)ceil_div(cp.c * cp.y * cp.x, 128) * ceil_div(cp.k, 128);
    while (S < 64 && cp.n % (2 * S) == 0 && cp.n / (2 * S) >= 8 && base * S < 2 * kNumCU)
      S *= 2;
  }
  const int64_t G2 = cp.g == 1 ? S : cp.g, n_per = cp.n / S;
  const int64_t np = (n_per * es + 15) / 16 * 16 / es;
  RockConvParams f = q; // converted operands
  f.g = (int)G2; f.c = (int)np;
  f.in_cs = 1; f.in_gs = np; f.in_ws = G2 * np; f.in_hs = cp.wi * f.in_ws; f.in_ns = cp.hi * f.in_hs;
  f.fil_cs = 1; f.fil_xs = np; f.fil_ys = cp.wo * np; f.fil_ks = cp.ho * f.fil_ys; f.fil_gs = cp.k * f.fil_ks;
  const int64_t dw_elems = cp.c * cp.y * cp.x * cp.k;
  if (S > 1) { // f32 partial sums [S][c][y][x][k]
    f.out_ks = 1; f.out_ws = cp.k; f.out_hs = cp.x * cp.k; f.out_ns = cp.y * f.out_hs; f.out_gs = dw_elems;
    f.epi.out_dtype = ROCK_F32;
  }
  const bool fast = bool_or(o, "layout_conversion", true) && conv_view_fast(f, es) &&
                    (int64_t)np * cp.ho * cp.wo <= INT32_MAX;
  if (!fast)
    S = 1;
  const int64_t x_bytes = align256(cp.c * cp.hi * cp.wi * G2 * np * es);
  const int64_t dy_bytes = align256(G2 * cp.k * cp.ho * cp.wo * np * es);
  const int64_t part_bytes = S > 1 ? align256(S * dw_elems * 4) : 0;
  const int count = fast ? (S > 1 ? 4 : 3) : 1;
  const int64_t workspace = fast ? x_bytes + dy_bytes + part_bytes : 0;
  if (kid < 0 || kid >= count) {
    set_error("conv: kernel_id out of range");
    return nullptr;
  }
  const int ws = 4;
  const int64_t group_is = cp.g == 1 ? n_per * cp.is[0] : cp.is[1], group_os = cp.g == 1 ? n_per * cp.os[0] : cp.os[1];
  Handle *h = nullptr;
  if (!fast) {
    h = conv_handle_from_view(q, cp.ti, o);
    if (!h)
      return nullptr;
    h->ptr_map = {{2, 0}, {1, 0}, {0, 0}, {-1, 0}, {-1, 0}};
    h->problem_key = conv_problem_key(h, o, cp, 4);
  } else if (kid == 0) { // input -> [c][hi][wi][G2][np]
    h = new Handle;
    const int64_t size[5] = {cp.c, cp.hi, cp.wi, G2, np}, src_size[5] = {cp.c, cp.hi, cp.wi, G2, n_per};
    const int64_t stride[5] = {cp.is[2], cp.is[3], cp.is[4], group_is, cp.is[0]};
    if (!fill_relayout_handle(h, size, src_size, stride, es)) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{1, 0}, {ws, 0}};
    h->problem_key = "relayout input " + cp.il;
  } else if (kid == 1) { // output gradient -> [G2][k][ho][wo][np]
    h = new Handle;
    const int64_t size[5] = {G2, cp.k, cp.ho, cp.wo, np}, src_size[5] = {G2, cp.k, cp.ho, cp.wo, n_per};
    const int64_t stride[5] = {group_os, cp.os[2], cp.os[3], cp.os[4], cp.os[0]};
    if (!fill_relayout_handle(h, size, src_size, stride, es)) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{2, 0}, {ws, x_bytes}};
    h->problem_key = "relayout output gradient " + cp.ol;
  } else if (kid == 2) {
    h = conv_handle_from_view(f, cp.ti, o);
    if (!h)
      return nullptr;
    h->ptr_map = {{ws, x_bytes}, {ws, 0}, S > 1 ? Handle::PtrSrc{ws, x_bytes + dy_bytes} : Handle::PtrSrc{0, 0},
                  {-1, 0}, {-1, 0}};
    h->problem_key = conv_problem_key(h, o, cp, 4);
  } else {
    h = new Handle;
    RockReduceParams r;
    std::memset(&r, 0, sizeof r);
    r.split_stride = dw_elems;
    r.size[0] = (int)cp.c; r.size[1] = (int)cp.y; r.size[2] = (int)cp.x; r.size[3] = (int)cp.k;
    r.dst_stride[0] = cp.fs[2]; r.dst_stride[1] = cp.fs[3]; r.dst_stride[2] = cp.fs[4]; r.dst_stride[3] = cp.fs[1];
    r.splits = (int)S;
    r.out_dtype = cp.ti;
    h->op = OP_RELAYOUT;
    h->epi = nullptr;
    h->params.assign(sizeof r, 0);
    std::memcpy(h->params.data(), &r, sizeof r);
    h->kernel_name = "rock_reduce_splits";
    h->block_size = 256;
    h->grid_size = (uint32_t)((dw_elems + 255) / 256);
    h->num_pointers = 2;
    h->perf_config = "";
    h->ptr_map = {{ws, x_bytes + dy_bytes}, {0, 0}};
    h->problem_key = "reduction of the split partial sums";
  }
  h->kernel_count = count;
  h->workspace_bytes = (size_t)workspace;
  h->caller_pointers = workspace ? 5 : 4;
  return h;
}


// ---- 3-D convolution ----------------------------------------------------------
// Layout strings of six letters (rocmlir-gen's "ngc012" / "gkc012" / "ngk012",
// rocmlir-gen.cpp:865-877; h, w, d and y, x, z are accepted for 0, 1, 2).
bool canon_layout3(std::string s, char channel, bool filter, std::string &out) {
  std::string r;
  for (char raw : s) {
    char ch = (char)std::tolower((unsigned char)raw);
    if (ch == 'h' || ch == 'y') ch = '0';
    else if (ch == 'w' || ch == 'x') ch = '1';
    else if (ch == 'd' || ch == 'z') ch = '2';
    else if (filter && ch == 'n') ch = 'k';
    else if (!filter && channel == 'k' && ch == 'c') ch = 'k';
    r.push_back(ch);
  }
  if (r.find('g') == std::string::npos) {
    const std::string c1(1, channel);
    if (filter)
      r = "g" + r;
    else if (r.size() >= 2 && r.substr(0, 2) == "n" + c1)
      r = "ng" + c1 + r.substr(2);
    else if (!r.empty() && r[0] == 'n' && r.back() == channel)
      r = r.substr(0, r.size() - 1) + "g" + c1;
    else
      r = "g" + r;
  }
  std::string a = r, b = filter ? "gkc012" : std::string("ng") + channel + "012";
  std::sort(a.begin(), a.end());
  std::sort(b.begin(), b.end());
  if (a != b)
    return false;
  out = r;
  return true;
}

// What the option list says about a convolution over three spatial dimensions.
struct Conv3dProblem {
  int ti, to;
  RockEpilogue epi;
  std::string fl, il, ol; // canonical six-letter layouts
  int64_t n, g, ct, kt;   // channels over all groups
  int64_t in[3], fil[3], out[3], dil[3], str[3], pl[3], pr[3]; // h, w, d
};

bool parse_conv3d(const OptMap &o, Conv3dProblem &P, bool backward) {
  std::string t_all = str_or(o, "t", "");
  std::string in_t = str_or(o, "in_type", t_all), fil_t = str_or(o, "fil_type", t_all),
              out_t = str_or(o, "out_type", str_or(o, "out_datatype", ""));
  static const char *req[] = {"batchsize", "in_channels", "in_h", "in_w", "in_d", "out_channels",
                              "fil_h", "fil_w", "fil_d", "in_layout", "out_layout", "fil_layout"};
  for (const char *k : req)
    if (!o.count(k)) {
      set_error(std::string("conv: missing --") + k);
      return false;
    }
  const int ti = parse_dtype(in_t), tf = parse_dtype(fil_t);
  if (ti < 0 || tf < 0 || ti != tf || ti == ROCK_I32) {
    set_error("conv: input and filter types must be given, known and equal");
    return false;
  }
  const int dflt_out = ti == ROCK_I8 ? ROCK_I32 : (ti == ROCK_FP8 || ti == ROCK_BF8) ? ROCK_F32 : ti;
  const int to = out_t.empty() ? dflt_out : parse_dtype(out_t);
  if (backward) {
    if (ti != to || (ti != ROCK_F32 && ti != ROCK_F16 && ti != ROCK_BF16)) {
      set_error("conv: the backward kernels take f32, f16 or bf16 for all three tensors");
      return false;
    }
    std::memset(&P.epi, 0, sizeof P.epi);
  } else {
    if (to < 0 || !parse_epilogue(o, ti, to, P.epi)) {
      set_error("conv: illegal input/output type combination or epilogue");
      return false;
    }
  }
  P.ti = ti;
  P.to = to;
  if (!canon_layout3(str_or(o, "fil_layout", ""), 'k', true, P.fl) ||
      !canon_layout3(str_or(o, "in_layout", ""), 'c', false, P.il) ||
      !canon_layout3(str_or(o, "out_layout", ""), 'k', false, P.ol)) {
    set_error("conv: unsupported layout string (3-D, six dimensions with g)");
    return false;
  }
  P.n = int_or(o, "batchsize", 0);
  P.g = int_or(o, "groupsize", 1);
  P.ct = int_or(o, "in_channels", 0);
  P.kt = int_or(o, "out_channels", 0);
  // spatial dimensions in the order 0 (h), 1 (w), 2 (d)
  static const char *ax[3] = {"h", "w", "d"};
  for (int a = 0; a < 3; ++a) {
    const std::string s = ax[a];
    P.in[a] = int_or(o, ("in_" + s).c_str(), 0);
    P.fil[a] = int_or(o, ("fil_" + s).c_str(), 0);
    P.dil[a] = int_or(o, ("dilation_" + s).c_str(), 1);
    P.str[a] = int_or(o, ("conv_stride_" + s).c_str(), 1);
    const int64_t both = int_or(o, ("padding_" + s).c_str(), 0);
    P.pl[a] = int_or(o, ("padding_" + s + "_l").c_str(), both);
    P.pr[a] = int_or(o, ("padding_" + s + "_r").c_str(), both);
    if (P.dil[a] <= 0 || P.str[a] <= 0 || P.pl[a] < 0 || P.pr[a] < 0) {
      set_error("conv: dilation and stride must be positive, padding non-negative");
      return false;
    }
    if (P.in[a] <= 0 || P.fil[a] <= 0) {
      set_error("conv: tensor dimensions must be positive and channels divisible by groups");
      return false;
    }
    if (P.in[a] + P.pl[a] + P.pr[a] < (P.fil[a] - 1) * P.dil[a] + 1) {
      set_error("conv: input, including padding, is smaller than the filter");
      return false;
    }
    P.out[a] = (P.in[a] + P.pl[a] + P.pr[a] - (P.fil[a] - 1) * P.dil[a] - 1) / P.str[a] + 1;
    int64_t given;
    if (get_int(o, ("out_" + s).c_str(), given) && given != P.out[a]) {
      set_error("conv: out_h/out_w/out_d do not match the value computed from the other parameters");
      return false;
    }
    if (backward && P.pl[a] != P.pr[a]) {
      set_error("conv: the backward kernels take symmetric padding only");
      return false;
    }
  }
  if (P.n <= 0 || P.g <= 0 || P.ct <= 0 || P.kt <= 0 || P.ct % P.g != 0 || P.kt % P.g != 0) {
    set_error("conv: tensor dimensions must be positive and channels divisible by groups");
    return false;
  }
  if (!bool_or(o, "layout_conversion", true)) {
    set_error("conv: three spatial dimensions run through the conversion kernels only");
    return false;
  }
  return true;
}

Handle *make_conv3d_backward(const OptMap &o, const Conv3dProblem &P, bool data);

// Forward convolution over three spatial dimensions (the reference takes them
// through the same rock.conv with a third spatial index, rocmlir-gen.cpp:171-294).
// The contraction kernels walk two spatial dimensions, so the third is
// unfolded into the channels by the conversion kernels: the workspace holds
//   T[n, do, hi, wi, g, z, c] = input[n, g, c, hi, wi, do*stride_d + z*dil_d - pad_d]
// (zero where that depth lies in the padding, c padded to whole 16-byte
// chunks) and the filter as F[g, k, y, x, z, c], after which the problem is a
// 2-D convolution with batch n*Do and Z*c channels per group.  Its output
// rows are the caller's when the output's batch stride is Do depth strides
// (channels-last layouts, or one image); otherwise it writes
// O[n, do, ho, wo, g, k] into the workspace and a last conversion kernel
// brings that into the caller's layout (a residual tensor, laid out as the
// output, is then converted into O's layout first).  Kernels: [zero fill of T], one
// conversion per (z, g) slice, the filter conversion (one per group when g
// and k are not neighbours in the filter's layout), [the residual conversion],
// the contraction, [the output conversion].
Handle *make_conv3d(const OptMap &o) {
  const std::string opn = str_or(o, "operation", "conv");
  const bool backward = opn.find("bwd") != std::string::npos;
  if (opn != "conv" && opn != "conv3d" && opn != "conv_bwd_data" && opn != "conv_bwd_weight") {
    set_error("conv: unknown operation for three spatial dimensions");
    return nullptr;
  }
  Conv3dProblem P;
  if (!parse_conv3d(o, P, backward))
    return nullptr;
  if (backward)
    return make_conv3d_backward(o, P, opn == "conv_bwd_data");
  const int ti = P.ti, to = P.to;
  const RockEpilogue epi = P.epi;
  const bool has_res = epi.residual_op != ROCK_RES_NONE;
  const std::string &fl = P.fl, &il = P.il, &ol = P.ol;
  const int64_t n = P.n, g = P.g, ct = P.ct, kt = P.kt;
  const int64_t *in = P.in, *fil = P.fil, *out = P.out, *dil = P.dil, *str = P.str, *pl = P.pl;
  const int64_t c = ct / g, k = kt / g;
  const int64_t Hi = in[0], Wi = in[1], Di = in[2], Y = fil[0], X = fil[1], Z = fil[2], Ho = out[0], Wo = out[1],
                Do = out[2];
  int64_t fs[6], is[6], os[6];
  {
    const int64_t fsz[6] = {g, k, c, Y, X, Z}, isz[6] = {n, g, c, Hi, Wi, Di}, osz[6] = {n, g, k, Ho, Wo, Do};
    layout_strides(fl, "gkc012", fsz, fs);
    layout_strides(il, "ngc012", isz, is);
    layout_strides(ol, "ngk012", osz, os);
  }
  const int es = dtype_size(ti), eso = dtype_size(to);
  const int64_t cp = (c * es + 15) / 16 * 16 / es;
  // the filter converts in one kernel when g and k fold into one dimension, else per group
  const bool fil_folds = g == 1 || fs[0] == k * fs[1];
  const int fil_kernels = fil_folds ? 1 : (int)g;
  // workspace: T, F, [O]
  const int64_t t_pix = g * Z * cp; // elements per (n, do, hi, wi)
  const int64_t t_bytes = align256(n * Do * Hi * Wi * t_pix * es);
  const int64_t f_bytes = align256(g * k * Y * X * Z * cp * es);
  const bool out_direct = n == 1 || os[0] == Do * os[5];
  const int64_t o_bytes = out_direct ? 0 : align256(n * Do * Ho * Wo * g * k * eso);
  // a residual tensor lies as the output does: read in place beside an output
  // written in place, else converted into the layout of O first
  const bool res_copy = has_res && !out_direct;
  const int64_t r_bytes = res_copy ? o_bytes : 0;
  if (n * Do > INT32_MAX || Z * cp > INT32_MAX || t_bytes / es > ((int64_t)1 << 40)) {
    set_error("conv: problem too large for 32-bit tile indices");
    return nullptr;
  }
  // slices of T: for tap z the output depths whose input depth exists
  struct Slice { int64_t z, g, lo, cnt; };
  std::vector<Slice> slices;
  bool need_fill = false;
  for (int64_t z = 0; z < Z; ++z) {
    const int64_t shift = z * dil[2] - pl[2]; // input depth = do * stride + shift
    const int64_t lo = shift >= 0 ? 0 : (-shift + str[2] - 1) / str[2];
    const int64_t hi_d = std::min(Do - 1, floor_div(Di - 1 - shift, str[2]));
    const int64_t cnt = hi_d - lo + 1;
    if (cnt < Do)
      need_fill = true;
    if (cnt > 0)
      for (int64_t gi = 0; gi < g; ++gi)
        slices.push_back(Slice{z, gi, lo, cnt});
  }
  const int first_slice = need_fill ? 1 : 0;
  const int i_filter = first_slice + (int)slices.size(), i_res = i_filter + fil_kernels;
  const int i_conv = i_res + (res_copy ? 1 : 0);
  const int count = i_conv + 1 + (out_direct ? 0 : 1);
  const int kid = (int)int_or(o, "kernel_id", 0);
  if (kid < 0 || kid >= count) {
    set_error("conv: kernel_id out of range");
    return nullptr;
  }
  const int ws = has_res ? 5 : 4; // caller list: filter, input, output, bias, [residual], workspace
  Handle *h = nullptr;
  if (need_fill && kid == 0) {
    h = utility_fill_handle(t_bytes);
    h->ptr_map = {{ws, 0}};
    h->problem_key = "zero fill of the unfolded input";
  } else if (res_copy && kid == i_res) {
    // the residual tensor -> R[n, do, ho, wo, g, k]
    const int64_t osz[6] = {n, Do, Ho, Wo, g, k};
    const int64_t css[6] = {os[0], os[5], os[3], os[4], os[1], os[2]};
    std::vector<ViewDim> dims;
    int64_t dense = 1;
    for (int d = 5; d >= 0; --d) {
      dims.insert(dims.begin(), ViewDim{osz[d], osz[d], css[d], dense});
      dense *= osz[d];
    }
    h = new Handle;
    if (!relayout_handle_nd(h, dims, eso, "output")) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{4, 0}, {ws, t_bytes + f_bytes + o_bytes}};
    h->problem_key = "relayout residual " + ol;
  } else if (kid < i_filter) {
    const Slice &sl = slices[kid - first_slice];
    h = new Handle;
    const int64_t size[5] = {n, sl.cnt, Hi, Wi, cp}, src_size[5] = {n, sl.cnt, Hi, Wi, c};
    const int64_t stride[5] = {is[0], str[2] * is[5], is[3], is[4], is[2]};
    const int64_t dstride[5] = {Do * Hi * Wi * t_pix, Hi * Wi * t_pix, Wi * t_pix, t_pix, 1};
    if (!fill_relayout_handle(h, size, src_size, stride, es, dstride)) {
      delete h;
      return nullptr;
    }
    const int64_t src_off = sl.g * is[1] + (sl.lo * str[2] + sl.z * dil[2] - pl[2]) * is[5];
    const int64_t dst_off = sl.lo * Hi * Wi * t_pix + (sl.g * Z + sl.z) * cp;
    h->ptr_map = {{1, src_off * es}, {ws, dst_off * es}};
    h->problem_key = "unfold input depth tap " + std::to_string(sl.z) + " group " + std::to_string(sl.g);
  } else if (kid < i_conv) {
    h = new Handle;
    const int64_t gi = kid - i_filter, rows = fil_folds ? g * k : k;
    const int64_t size[5] = {rows, Y, X, Z, cp}, src_size[5] = {rows, Y, X, Z, c};
    const int64_t stride[5] = {fs[1], fs[3], fs[4], fs[5], fs[2]};
    if (!fill_relayout_handle(h, size, src_size, stride, es)) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{0, gi * fs[0] * es}, {ws, t_bytes + gi * k * Y * X * Z * cp * es}};
    h->problem_key = "relayout filter " + fl;
  } else if (kid == i_conv) {
    RockConvParams q;
    std::memset(&q, 0, sizeof q);
    q.n = (int)(n * Do); q.g = (int)g; q.c = (int)(Z * cp); q.k = (int)k;
    q.hi = (int)Hi; q.wi = (int)Wi; q.y = (int)Y; q.x = (int)X; q.ho = (int)Ho; q.wo = (int)Wo;
    q.stride_h = (int)str[0]; q.stride_w = (int)str[1]; q.pad_h = (int)pl[0]; q.pad_w = (int)pl[1];
    q.dil_h = (int)dil[0]; q.dil_w = (int)dil[1];
    q.in_cs = 1; q.in_gs = Z * cp; q.in_ws = t_pix; q.in_hs = Wi * t_pix; q.in_ns = Hi * Wi * t_pix;
    q.fil_cs = 1; q.fil_xs = Z * cp; q.fil_ys = X * q.fil_xs; q.fil_ks = Y * q.fil_ys; q.fil_gs = k * q.fil_ks;
    if (out_direct) {
      q.out_ns = os[5]; q.out_gs = os[1]; q.out_ks = os[2]; q.out_hs = os[3]; q.out_ws = os[4];
    } else {
      q.out_ks = 1; q.out_gs = k; q.out_ws = g * k; q.out_hs = Wo * q.out_ws; q.out_ns = Ho * q.out_hs;
    }
    q.epi = epi;
    h = conv_handle_from_view(q, ti, o);
    if (!h)
      return nullptr;
    const bool tiled = h->kernel_name.find("generic") == std::string::npos;
    h->kernel_name += rich_suffix(epi, tiled, o);
    h->ptr_map = {{ws, t_bytes}, {ws, 0}, out_direct ? Handle::PtrSrc{2, 0} : Handle::PtrSrc{ws, t_bytes + f_bytes},
                  {3, 0},
                  !has_res ? Handle::PtrSrc{-1, 0}
                           : res_copy ? Handle::PtrSrc{ws, t_bytes + f_bytes + o_bytes} : Handle::PtrSrc{4, 0}};
    std::ostringstream key;
    const char *opname = ti == ROCK_F32 ? "conv" : ti == ROCK_F16 ? "convfp16" : ti == ROCK_BF16 ? "convbfp16"
                       : ti == ROCK_I8 ? "convint8" : ti == ROCK_FP8 ? "convfp8_fp8" : "convbf8_bf8";
    auto key_letters = [](const std::string &layout, bool filter) {
      std::string r;
      for (char ch : layout)
        r.push_back(ch == 'g' ? 'G' : ch == 'n' ? 'N' : ch == 'c' ? 'C' : ch == 'k' ? (filter ? 'N' : 'C') : ch);
      return r;
    };
    key << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << opname << " -F 1 -f " << key_letters(fl, true)
        << " -I " << key_letters(il, false) << " -O " << key_letters(ol, false) << " -n " << n << " -c " << c
        << " -H " << Hi << " -W " << Wi << " -k " << k << " -y " << Y << " -x " << X << " -p " << pl[0] << " -q "
        << pl[1] << " -u " << str[0] << " -v " << str[1] << " -l " << dil[0] << " -j " << dil[1] << " -g " << g
        // the reference's key stops here (RockTuningImpl.cpp:775-808); the depth fields keep 3-D problems apart
        << " --in_d " << Di << " --fil_d " << Z << " --padding_d " << pl[2] << " --conv_stride_d " << str[2]
        << " --dilation_d " << dil[2];
    h->problem_key = key.str();
  } else {
    // O[n, do, ho, wo, g, k] -> the caller's layout: dimensions in the caller's
    // order, unit ones dropped, (g, k) and neighbouring spatial dimensions folded
    struct Dim { int64_t size, ss; };
    std::vector<Dim> dims;
    const int64_t osz[6] = {n, g, k, Ho, Wo, Do};
    const int64_t oss[6] = {Do * Ho * Wo * g * k, k, 1, Wo * g * k, g * k, Ho * Wo * g * k}; // of O, letter order ngk012
    for (char ch : ol) {
      const size_t idx = std::string("ngk012").find(ch);
      dims.push_back(Dim{osz[idx], oss[idx]});
    }
    for (size_t d = 0; d + 1 < dims.size();)
      if (dims[d].size == 1)
        dims.erase(dims.begin() + d);
      else
        ++d;
    for (size_t d = 0; d + 1 < dims.size() && dims.size() > 5;)
      if (dims[d].ss == dims[d + 1].size * dims[d + 1].ss) {
        dims[d] = Dim{dims[d].size * dims[d + 1].size, dims[d + 1].ss};
        dims.erase(dims.begin() + d + 1);
      } else {
        ++d;
      }
    if (dims.size() > 5) {
      set_error("conv: this 3-D output layout needs more than five independent dimensions");
      return nullptr;
    }
    while (dims.size() < 5)
      dims.insert(dims.begin(), Dim{1, 0});
    int64_t size[5], stride[5];
    for (int d = 0; d < 5; ++d) {
      size[d] = dims[d].size;
      stride[d] = dims[d].ss;
    }
    h = new Handle;
    if (!fill_relayout_handle(h, size, size, stride, eso)) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{ws, t_bytes + f_bytes}, {2, 0}};
    h->problem_key = "relayout output " + ol;
  }
  h->kernel_count = count;
  h->workspace_bytes = (size_t)(t_bytes + f_bytes + o_bytes + r_bytes);
  h->caller_pointers = has_res ? 6 : 5;
  return h;
}

// The gradients of a convolution over three spatial dimensions (the reference
// lowers every direction of rock.conv with a third spatial index,
// ConvGenerator.cpp:496-512, 651-661; ConvToGemm.cpp:530-1131), on the forward
// plan's unfolding of the depth taps into the channels:
//   T[n, do, hi, wi, g, z, c] <-> input[n, g, c, hi, wi, do*stride_d + z*dil_d - pad_d]
//   F[g, k, y, x, z, c]       <-> filter,   O[n, do, ho, wo, g, k] <-> output
// make the problem a 2-D one with batch n*Do and Z*c channels per group, whose
// gradient plans (make_conv_bwd_weight / make_conv_bwd_data) run in the middle.
//  * filter gradient: T is unfolded from the input as in the forward plan, the
//    2-D plan writes dF, conversion kernels bring dF into the caller's layout;
//  * input gradient: the filter goes to F, the 2-D plan writes dT, and
//    rock_fold_depth adds up, for every input depth, the (do, z) pairs that
//    reach it -- into the caller's tensor when its channels are contiguous,
//    otherwise into a channels-last copy that one more conversion transposes.
// The output gradient is read where it lies when its batch stride is Do depth
// strides (or there is one image), else from a converted copy O.
// Pointer order as in two dimensions: filter, input, output, unused, workspace.
Handle *make_conv3d_backward(const OptMap &o, const Conv3dProblem &P, bool data) {
  const int es = dtype_size(P.ti);
  const int64_t n = P.n, g = P.g, c = P.ct / g, k = P.kt / g;
  const int64_t Hi = P.in[0], Wi = P.in[1], Di = P.in[2], Y = P.fil[0], X = P.fil[1], Z = P.fil[2], Ho = P.out[0],
                Wo = P.out[1], Do = P.out[2];
  const int64_t sd = P.str[2], dd = P.dil[2], pd = P.pl[2];
  int64_t fs[6], is[6], os[6];
  {
    const int64_t fsz[6] = {g, k, c, Y, X, Z}, isz[6] = {n, g, c, Hi, Wi, Di}, osz[6] = {n, g, k, Ho, Wo, Do};
    layout_strides(P.fl, "gkc012", fsz, fs);
    layout_strides(P.il, "ngc012", isz, is);
    layout_strides(P.ol, "ngk012", osz, os);
  }
  const int64_t cp = (c * es + 15) / 16 * 16 / es;
  const int64_t t_pix = g * Z * cp;
  const int64_t t_elems = n * Do * Hi * Wi * t_pix;
  if (n * Do > INT32_MAX || Z * cp > INT32_MAX || t_elems > ((int64_t)1 << 40) || n * Di * Hi * Wi * g * c > ((int64_t)1 << 39)) {
    set_error("conv: problem too large for 32-bit tile indices");
    return nullptr;
  }
  const bool fil_folds = g == 1 || fs[0] == k * fs[1];
  const int fil_kernels = fil_folds ? 1 : (int)g;
  const bool out_direct = n == 1 || os[0] == Do * os[5];
  const bool x_direct = is[2] == 1; // the fold writes runs of channels
  const int64_t t_bytes = align256(t_elems * es);
  const int64_t f_bytes = align256(g * k * Y * X * Z * cp * es);
  const int64_t o_bytes = out_direct ? 0 : align256(n * Do * Ho * Wo * g * k * es);
  const int64_t x_bytes = (data && !x_direct) ? align256(n * Di * Hi * Wi * g * c * es) : 0;
  const int64_t o_off = t_bytes + f_bytes, x_off = o_off + o_bytes, inner_off = x_off + x_bytes;

  // the 2-D problem over the workspace tensors
  ConvProblem inner;
  inner.ti = P.ti;
  inner.fl = "gkyxc"; inner.il = "nhwgc"; inner.ol = "nhwgk";
  inner.n = n * Do; inner.g = g; inner.c = Z * cp; inner.k = k; inner.hi = Hi; inner.wi = Wi; inner.y = Y; inner.x = X;
  inner.ho = Ho; inner.wo = Wo; inner.sh = P.str[0]; inner.sw = P.str[1]; inner.ph = P.pl[0]; inner.pw = P.pl[1];
  inner.dh = P.dil[0]; inner.dw = P.dil[1];
  {
    const int64_t zc = Z * cp;
    const int64_t f2[5] = {k * Y * X * zc, Y * X * zc, 1, X * zc, zc};
    const int64_t i2[5] = {Hi * Wi * t_pix, zc, 1, Wi * t_pix, t_pix};
    const int64_t o2d[5] = {os[5], os[1], os[2], os[3], os[4]};
    const int64_t o2w[5] = {Ho * Wo * g * k, k, 1, Wo * g * k, g * k};
    for (int d = 0; d < 5; ++d) {
      inner.fs[d] = f2[d];
      inner.is[d] = i2[d];
      inner.os[d] = out_direct ? o2d[d] : o2w[d];
    }
  }
  auto inner_at = [&](int id) {
    OptMap o2 = o;
    o2["kernel_id"] = std::to_string(id);
    return data ? make_conv_bwd_data(o2, inner) : make_conv_bwd_weight(o2, inner);
  };
  int inner_count;
  size_t inner_ws;
  {
    Handle *probe = inner_at(0);
    if (!probe)
      return nullptr;
    inner_count = probe->kernel_count;
    inner_ws = probe->workspace_bytes;
    delete probe;
  }

  // slices of T (filter gradient): for tap z the output depths whose input depth exists
  struct Slice { int64_t z, g, lo, cnt; };
  std::vector<Slice> slices;
  bool need_fill = false;
  if (!data) {
    for (int64_t z = 0; z < Z; ++z) {
      const int64_t shift = z * dd - pd; // input depth = do * stride + shift
      const int64_t lo = shift >= 0 ? 0 : (-shift + sd - 1) / sd;
      const int64_t hi_d = std::min(Do - 1, floor_div(Di - 1 - shift, sd));
      const int64_t cnt = hi_d - lo + 1;
      if (cnt < Do)
        need_fill = true;
      if (cnt > 0)
        for (int64_t gi = 0; gi < g; ++gi)
          slices.push_back(Slice{z, gi, lo, cnt});
    }
  }
  // kernel order
  const int n_fill = need_fill ? 1 : 0;
  const int n_pre = data ? fil_kernels : n_fill + (int)slices.size();
  const int i_out = n_pre;                       // conversion of the output gradient, when needed
  const int i_inner = i_out + (out_direct ? 0 : 1);
  const int i_post = i_inner + inner_count;
  const int n_post = data ? 1 + (x_direct ? 0 : 1) : fil_kernels;
  const int count = i_post + n_post;
  const int kid = (int)int_or(o, "kernel_id", 0);
  if (kid < 0 || kid >= count) {
    set_error("conv: kernel_id out of range");
    return nullptr;
  }
  const int ws = 4;
  const int64_t zc = Z * cp;
  // F[g, k, y, x, z, c] against the caller's filter, one kernel or one per group
  auto filter_kernel = [&](int gi, bool to_caller) -> Handle * {
    const int64_t rows = fil_folds ? g * k : k;
    const int64_t wstr[5] = {Y * X * zc, X * zc, zc, cp, 1};          // of F over (gk, y, x, z, c)
    const int64_t cstr[5] = {fs[1], fs[3], fs[4], fs[5], fs[2]};      // of the caller's filter
    const int64_t sz[5] = {rows, Y, X, Z, c}, szp[5] = {rows, Y, X, Z, cp};
    auto *h = new Handle;
    bool ok;
    if (!to_caller) {
      ok = fill_relayout_handle(h, szp, sz, cstr, es, nullptr);
    } else {
      // dimensions in the caller's order, dF read through F's strides
      std::vector<ViewDim> dims;
      const std::string letters = "kc012";
      const int64_t lsz[5] = {rows, c, Y, X, Z}, lws[5] = {wstr[0], 1, wstr[1], wstr[2], wstr[3]},
                    lcs[5] = {fs[1], fs[2], fs[3], fs[4], fs[5]};
      for (char ch : P.fl) {
        if (ch == 'g')
          continue;
        const size_t idx = letters.find(ch);
        dims.push_back(ViewDim{lsz[idx], lsz[idx], lws[idx], lcs[idx]});
      }
      ok = relayout_handle_nd(h, dims, es, "filter");
    }
    if (!ok) {
      delete h;
      return nullptr;
    }
    const Handle::PtrSrc user{0, gi * fs[0] * es}, work{ws, t_bytes + gi * k * Y * X * zc * es};
    h->ptr_map = to_caller ? std::vector<Handle::PtrSrc>{work, user} : std::vector<Handle::PtrSrc>{user, work};
    h->problem_key = (to_caller ? "relayout filter gradient " : "relayout filter ") + P.fl;
    return h;
  };
  Handle *h = nullptr;
  if (kid < n_pre) {
    if (data) {
      h = filter_kernel(kid, false);
      if (!h)
        return nullptr;
    } else if (need_fill && kid == 0) {
      h = utility_fill_handle(t_bytes);
      h->ptr_map = {{ws, 0}};
      h->problem_key = "zero fill of the unfolded input";
    } else {
      const Slice &sl = slices[kid - n_fill];
      h = new Handle;
      const int64_t size[5] = {n, sl.cnt, Hi, Wi, cp}, src_size[5] = {n, sl.cnt, Hi, Wi, c};
      const int64_t stride[5] = {is[0], sd * is[5], is[3], is[4], is[2]};
      const int64_t dstride[5] = {Do * Hi * Wi * t_pix, Hi * Wi * t_pix, Wi * t_pix, t_pix, 1};
      if (!fill_relayout_handle(h, size, src_size, stride, es, dstride)) {
        delete h;
        return nullptr;
      }
      const int64_t src_off = sl.g * is[1] + (sl.lo * sd + sl.z * dd - pd) * is[5];
      const int64_t dst_off = sl.lo * Hi * Wi * t_pix + (sl.g * Z + sl.z) * cp;
      h->ptr_map = {{1, src_off * es}, {ws, dst_off * es}};
      h->problem_key = "unfold input depth tap " + std::to_string(sl.z) + " group " + std::to_string(sl.g);
    }
  } else if (kid < i_inner) {
    // the output gradient -> O[n, do, ho, wo, g, k]
    const int64_t osz[6] = {n, Do, Ho, Wo, g, k};
    const int64_t css[6] = {os[0], os[5], os[3], os[4], os[1], os[2]};
    std::vector<ViewDim> dims;
    int64_t dense = 1;
    for (int d = 5; d >= 0; --d) {
      dims.insert(dims.begin(), ViewDim{osz[d], osz[d], css[d], dense});
      dense *= osz[d];
    }
    h = new Handle;
    if (!relayout_handle_nd(h, dims, es, "output")) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{2, 0}, {ws, o_off}};
    h->problem_key = "relayout output gradient " + P.ol;
  } else if (kid < i_post) {
    h = inner_at(kid - i_inner);
    if (!h)
      return nullptr;
    if (h->ptr_map.empty())
      for (int i = 0; i < h->num_pointers; ++i)
        h->ptr_map.push_back(Handle::PtrSrc{i, 0});
    for (auto &src : h->ptr_map) {
      if (src.source == 0)
        src = Handle::PtrSrc{ws, t_bytes + src.offset};
      else if (src.source == 1)
        src = Handle::PtrSrc{ws, src.offset};
      else if (src.source == 2 && !out_direct)
        src = Handle::PtrSrc{ws, o_off + src.offset};
      else if (src.source == 4)
        src.offset += inner_off;
    }
    if (h->op != OP_RELAYOUT) {
      // the 2-D key with the depth fields behind it, as the forward plan writes it
      std::ostringstream key;
      key << h->problem_key << " --in_d " << Di << " --fil_d " << Z << " --padding_d " << pd << " --conv_stride_d "
          << sd << " --dilation_d " << dd << " --in_channels_3d " << c;
      h->problem_key = key.str();
    }
  } else if (!data) {
    h = filter_kernel(kid - i_post, true);
    if (!h)
      return nullptr;
  } else if (kid == i_post) {
    RockFoldDepthParams f;
    std::memset(&f, 0, sizeof f);
    if (x_direct) {
      const int64_t st[6] = {is[0], is[1], is[2], is[3], is[4], is[5]};
      std::memcpy(f.dst_stride, st, sizeof st);
    } else {
      // X'[n, d, h, w, g, c]
      const int64_t st[6] = {Di * Hi * Wi * g * c, c, 1, Wi * g * c, g * c, Hi * Wi * g * c};
      std::memcpy(f.dst_stride, st, sizeof st);
    }
    f.t_pix = t_pix;
    f.n = (int)n; f.g = (int)g; f.c = (int)c; f.cp = (int)cp; f.hi = (int)Hi; f.wi = (int)Wi; f.di = (int)Di;
    f.d_out = (int)Do; f.z = (int)Z; f.stride_d = (int)sd; f.dil_d = (int)dd; f.pad_d = (int)pd;
    f.dtype = P.ti;
    h = new Handle;
    h->op = OP_RELAYOUT;
    h->epi = nullptr;
    h->params.assign(sizeof f, 0);
    std::memcpy(h->params.data(), &f, sizeof f);
    h->kernel_name = "rock_fold_depth";
    h->block_size = 256;
    h->grid_size = (uint32_t)((n * Di * Hi * Wi * g * c + 255) / 256);
    h->num_pointers = 2;
    h->perf_config = "";
    h->ptr_map = {{ws, 0}, x_direct ? Handle::PtrSrc{1, 0} : Handle::PtrSrc{ws, x_off}};
    h->problem_key = "fold depth taps into the input gradient";
  } else {
    // X'[n, d, h, w, g, c] -> the caller's layout
    const std::string letters = "ngc012";
    const int64_t isz[6] = {n, g, c, Hi, Wi, Di};
    const int64_t xss[6] = {Di * Hi * Wi * g * c, c, 1, Wi * g * c, g * c, Hi * Wi * g * c};
    std::vector<ViewDim> dims;
    for (char ch : P.il) {
      const size_t idx = letters.find(ch);
      dims.push_back(ViewDim{isz[idx], isz[idx], xss[idx], is[idx]});
    }
    h = new Handle;
    if (!relayout_handle_nd(h, dims, es, "input")) {
      delete h;
      return nullptr;
    }
    h->ptr_map = {{ws, x_off}, {1, 0}};
    h->problem_key = "relayout input gradient " + P.il;
  }
  h->kernel_count = count;
  h->workspace_bytes = (size_t)inner_off + inner_ws;
  h->caller_pointers = 5;
  return h;
}

Handle *make_conv(const OptMap &o) {
  if (o.count("in_d") || o.count("fil_d"))
    return make_conv3d(o);
  // required keys (ConvGenerator.cpp:492-512); rocmlir-gen's "-t" sets all
  // three types at once
  std::string t_all = str_or(o, "t", "");
  std::string in_t = str_or(o, "in_type", t_all), fil_t = str_or(o, "fil_type", t_all),
              out_t = str_or(o, "out_type", str_or(o, "out_datatype", ""));
  static const char *req[] = {"batchsize", "in_channels", "in_h", "in_w", "out_channels",
                              "fil_h", "fil_w", "in_layout", "out_layout", "fil_layout"};
  for (const char *k : req)
    if (!o.count(k)) {
      set_error(std::string("conv: missing --") + k);
      return nullptr;
    }
  int ti = parse_dtype(in_t), tf = parse_dtype(fil_t);
  if (ti < 0 || tf < 0 || ti != tf || ti == ROCK_I32) {
    set_error("conv: input and filter types must be given, known and equal");
    return nullptr;
  }
  int dflt_out = ti == ROCK_I8 ? ROCK_I32 : (ti == ROCK_FP8 || ti == ROCK_BF8) ? ROCK_F32 : ti;
  int to = out_t.empty() ? dflt_out : parse_dtype(out_t);
  if (to < 0) {
    set_error("conv: unknown output type");
    return nullptr;
  }
  std::string fl, il, ol;
  if (!canon_layout(str_or(o, "fil_layout", ""), 'k', "gkcyx", fl) ||
      !canon_layout(str_or(o, "in_layout", ""), 'c', "ngchw", il) ||
      !canon_layout(str_or(o, "out_layout", ""), 'k', "ngkhw", ol)) {
    set_error("conv: unsupported layout string (2-D, five dimensions with g)");
    return nullptr;
  }
  int64_t n = int_or(o, "batchsize", 0), g = int_or(o, "groupsize", 1),
          ct = int_or(o, "in_channels", 0), kt = int_or(o, "out_channels", 0),
          hi = int_or(o, "in_h", 0), wi = int_or(o, "in_w", 0), y = int_or(o, "fil_h", 0),
          x = int_or(o, "fil_w", 0);
  int64_t dh = int_or(o, "dilation_h", 1), dw = int_or(o, "dilation_w", 1),
          sh = int_or(o, "conv_stride_h", 1), sw = int_or(o, "conv_stride_w", 1),
          ph = int_or(o, "padding_h", 0), pw = int_or(o, "padding_w", 0);
  int64_t ph_r = int_or(o, "padding_h_r", ph), pw_r = int_or(o, "padding_w_r", pw);
  ph = int_or(o, "padding_h_l", ph);
  pw = int_or(o, "padding_w_l", pw);
  // ConvGenerator.cpp:136-248
  if (dh <= 0 || dw <= 0 || sh <= 0 || sw <= 0 || ph < 0 || pw < 0 || ph_r < 0 || pw_r < 0) {
    set_error("conv: dilation and stride must be positive, padding non-negative");
    return nullptr;
  }
  if (n <= 0 || g <= 0 || ct <= 0 || kt <= 0 || hi <= 0 || wi <= 0 || y <= 0 || x <= 0 ||
      ct % g != 0 || kt % g != 0) {
    set_error("conv: tensor dimensions must be positive and channels divisible by groups");
    return nullptr;
  }
  if (hi + ph + ph_r < (y - 1) * dh + 1 || wi + pw + pw_r < (x - 1) * dw + 1) {
    set_error("conv: input, including padding, is smaller than the filter");
    return nullptr;
  }
  // output extent (ConvGenerator.h:101-108)
  int64_t ho = (hi + ph + ph_r - (y - 1) * dh - 1) / sh + 1;
  int64_t wo = (wi + pw + pw_r - (x - 1) * dw - 1) / sw + 1;
  int64_t given;
  if ((get_int(o, "out_h", given) && given != ho) || (get_int(o, "out_w", given) && given != wo)) {
    set_error("conv: out_h/out_w do not match the value computed from the other parameters");
    return nullptr;
  }
  std::string opn = str_or(o, "operation", "conv");
  if (opn != "conv" && opn != "conv2d") {
    // the gradients (rocmlir-gen's conv_bwd_data / conv_bwd_weight, Miir's operation key)
    if (ph_r != ph || pw_r != pw) {
      set_error("conv: the backward kernels take symmetric padding only");
      return nullptr;
    }
    if (ti != to || (ti != ROCK_F32 && ti != ROCK_F16 && ti != ROCK_BF16)) {
      set_error("conv: the backward kernels take f32, f16 or bf16 for all three tensors");
      return nullptr;
    }
    ConvProblem cp;
    cp.ti = ti; cp.fl = fl; cp.il = il; cp.ol = ol;
    cp.n = n; cp.g = g; cp.c = ct / g; cp.k = kt / g; cp.hi = hi; cp.wi = wi; cp.y = y; cp.x = x; cp.ho = ho; cp.wo = wo;
    cp.sh = sh; cp.sw = sw; cp.ph = ph; cp.pw = pw; cp.dh = dh; cp.dw = dw;
    const int64_t fsz[5] = {g, cp.k, cp.c, y, x}, isz[5] = {n, g, cp.c, hi, wi}, osz[5] = {n, g, cp.k, ho, wo};
    layout_strides(fl, "gkcyx", fsz, cp.fs);
    layout_strides(il, "ngchw", isz, cp.is);
    layout_strides(ol, "ngkhw", osz, cp.os);
    return opn.find("bwd_data") != std::string::npos ? make_conv_bwd_data(o, cp) : make_conv_bwd_weight(o, cp);
  }
  const int64_t c_problem = ct / g, k = kt / g; // channels per group as the problem states them
  int64_t c = c_problem;                        // ... and as the contraction kernel sees them (may be padded)
  const int64_t Mg = n * ho * wo;
  int64_t Kg = c * y * x;
  if (Mg > INT32_MAX || Kg > INT32_MAX) {
    set_error("conv: problem too large for 32-bit tile indices");
    return nullptr;
  }

  auto *h = new Handle;
  h->op = OP_CONV;
  h->params.assign(sizeof(RockConvParams), 0);
  auto &p = *reinterpret_cast<RockConvParams *>(h->params.data());
  h->epi = &p.epi;
  if (!parse_epilogue(o, ti, to, p.epi)) {
    set_error("conv: illegal input/output type combination or epilogue");
    delete h;
    return nullptr;
  }
  p.n = (int)n; p.g = (int)g; p.c = (int)c; p.k = (int)k;
  p.hi = (int)hi; p.wi = (int)wi; p.y = (int)y; p.x = (int)x; p.ho = (int)ho; p.wo = (int)wo;
  p.stride_h = (int)sh; p.stride_w = (int)sw; p.pad_h = (int)ph; p.pad_w = (int)pw;
  p.dil_h = (int)dh; p.dil_w = (int)dw;
  p.M = (int)Mg; p.N = (int)k; p.K = (int)Kg;
  {
    int64_t fsz[5] = {g, k, c, y, x}, isz[5] = {n, g, c, hi, wi}, osz[5] = {n, g, k, ho, wo};
    int64_t fs[5], is[5], os[5];
    layout_strides(fl, "gkcyx", fsz, fs);
    layout_strides(il, "ngchw", isz, is);
    layout_strides(ol, "ngkhw", osz, os);
    p.fil_gs = fs[0]; p.fil_ks = fs[1]; p.fil_cs = fs[2]; p.fil_ys = fs[3]; p.fil_xs = fs[4];
    p.in_ns = is[0]; p.in_gs = is[1]; p.in_cs = is[2]; p.in_hs = is[3]; p.in_ws = is[4];
    p.out_ns = os[0]; p.out_gs = os[1]; p.out_ks = os[2]; p.out_hs = os[3]; p.out_ws = os[4];
    // a filter dimension of one element is described by any stride: a 1x1 filter stored gkcyx is the
    // channels-last filter as it lies and needs no conversion
    if (x == 1 && p.fil_cs == 1)
      p.fil_xs = c;
    if (y == 1 && p.fil_cs == 1 && p.fil_xs == c)
      p.fil_ys = x * c;
  }
  const int es = dtype_size(ti);
  auto al = [&](int64_t elems) { return (elems * es) % 16 == 0; };
  auto conv_fast = [&](const RockConvParams &q, int64_t cc) {
    return q.in_cs == 1 && al(cc) && al(q.in_ws) && al(q.in_hs) && al(q.in_ns) && al(q.in_gs) &&
           q.fil_cs == 1 && q.fil_xs == cc && q.fil_ys == x * cc && al(q.fil_ks) && al(q.fil_gs) &&
           // byte offsets inside one group's input slice and one filter tile < 2^31
           (n * q.in_ns + hi * q.in_hs + wi * q.in_ws + cc) * es < ((int64_t)1 << 31) &&
           (256 * q.fil_ks + cc * y * x) * es < ((int64_t)1 << 31);
  };
  bool fast = conv_fast(p, c);
  bool planned = false; // the layout-conversion plan fixes the pointer map itself

  // Reduction split over blocks: few output tiles and a long reduction (the 3x3 layers of a UNet at batch 2:
  // 512 pixels x 1280 channels over K = 17280 is 160 tiles of 64 x 64, each with 270 K-steps in a row).  The
  // (taps, channels) range is cut into S equal shares of whole K-steps; the contraction kernel runs them as S
  // groups of the one-group problem (RockConvParams::k_group_stride) into f32 partial results in the
  // workspace (int32 for int8 operands), which rock_reduce_splits adds in split order into the caller's
  // layout.  Only with the identity epilogue, which commutes with the sum (as for the GEMM, and as the reference's split-K,
  // Rock.cpp:167-198); "--split_k false" declines, and a perf_config names the split itself in its splitK field
  // (1 = none), so that the string a split plan reports leads back to it.
  int64_t S = 1, k_part = 0, part_off = 0;
  int conv_kid = 0;
  {
    const RockEpilogue &e = p.epi;
    const bool plain = e.scale == 1.0f && !e.has_bias && e.activation == ROCK_ACT_NONE && !e.chan_flags &&
                       e.residual_op == ROCK_RES_NONE;
    const bool identity = plain && ((to == ti && (ti == ROCK_F32 || ti == ROCK_F16 || ti == ROCK_BF16)) ||
                                    (ti == ROCK_I8 && to == ROCK_I32 && e.zero_point == 0));
    const int64_t c_chunks = (c * es + 15) / 16 * 16 / es, Kfull = c_chunks * y * x, step = 128 / es;
    const int64_t tiles64 = (int64_t)ceil_div(Mg, 64) * ceil_div(k, 64);
    const int64_t s_req = requested_block_splits(o); // a perf_config names the split itself
    auto share_ok = [&](int64_t d) { return Kfull % d == 0 && (Kfull / d) % step == 0; };
    if (g == 1 && identity && Mg * k <= INT32_MAX && bool_or(o, "split_k", true)) {
      if (s_req > 1 && share_ok(s_req))
        S = s_req;
      else if (s_req < 0 && tiles64 <= 2 * kNumCU && Kfull >= 2048) {
        const int64_t want = std::min<int64_t>(4 * kNumCU / tiles64, Kfull / 1024);
        for (int64_t d = want; d >= 2; --d)
          if (share_ok(d)) {
            S = d;
            break;
          }
      }
      if (S > 1)
        k_part = Kfull / S;
    }
  }
  const int64_t part_bytes = S > 1 ? align256(S * Mg * k * 4) : 0;

  auto set_problem_key = [&] {
    std::ostringstream key;
    const char *opname = ti == ROCK_F32 ? "conv" : ti == ROCK_F16 ? "convfp16"
                       : ti == ROCK_BF16 ? "convbfp16" : ti == ROCK_I8 ? "convint8"
                       : ti == ROCK_FP8 ? "convfp8_fp8" : "convbf8_bf8";
    key << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << opname << " -F 1 -f "
        << key_layout(fl, true) << " -I " << key_layout(il, false) << " -O "
        << key_layout(ol, false) << " -n " << n << " -c " << c_problem << " -H " << hi << " -W " << wi
        << " -k " << k << " -y " << y << " -x " << x << " -p " << ph << " -q " << pw << " -u "
        << sh << " -v " << sw << " -l " << dh << " -j " << dw << " -g " << g;
    h->problem_key = key.str();
  };

  // A 1x1 filter with unit stride, no padding and one group over images whose
  // pixels are contiguous (NCHW): image n's output is filter[k, c] x
  // input_n[c, h*w], a batched GEMM with the filter shared by the batch and the
  // second operand stored K-major.  The transposing-read GEMM kernels take it
  // as it lies: no conversion, no workspace.  (A per-channel bias would run
  // along GEMM rows, which the epilogue does not do; such problems convert.)
  if (!fast && y == 1 && x == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && g == 1 && !p.epi.has_bias &&
      !p.epi.chan_flags && p.in_ws == 1 && p.in_hs == wi && p.out_ws == 1 && p.out_hs == wo && hi * wi <= INT32_MAX &&
      bool_or(o, "pointwise_as_gemm", true)) {
    RockGemmParams gp;
    std::memset(&gp, 0, sizeof gp);
    gp.G = (int)n; gp.M = (int)k; gp.N = (int)(hi * wi); gp.K = (int)c;
    gp.a_gs = 0; gp.a_ms = p.fil_ks; gp.a_ks = p.fil_cs;
    gp.b_gs = p.in_ns; gp.b_ns = 1; gp.b_ks = p.in_cs;
    gp.c_gs = p.out_ns; gp.c_ms = p.out_ks; gp.c_ns = 1;
    gp.epi = p.epi;
    if (plan_gemm_kernel(h, gp, operand_code(ti, ti), es, o)) {
      h->op = OP_GEMM;
      h->params.assign(sizeof gp, 0); // p is gone from here on
      std::memcpy(h->params.data(), &gp, sizeof gp);
      h->epi = &reinterpret_cast<RockGemmParams *>(h->params.data())->epi;
      set_problem_key();
      return h;
    }
  }

  // Narrow pixels (the 3-channel first layer of a CNN), one group, no padding or
  // dilation along w.  Both tensors are copied channels-last with the channel
  // run padded to a power of two that divides a 16-byte chunk (3 -> 4 of 16
  // bits, 3 -> 8 of 8 bits); a row of x filter taps then reads x neighbouring
  // pixels, one contiguous run, padded to whole chunks, and the contraction
  // sees "channels" = that run under a filter one tap wide: K = y * run in
  // place of y * x * (c padded to a whole chunk).  The last chunk of a run
  // brings the next pixel along; the "_runs" kernels clear it in LDS (the
  // filter holds zeros there, but zero times an Inf in that pixel would not be
  // zero).  Every window must start on a chunk boundary: stride_w pixels and an
  // image row are whole chunks.
  bool runs_kernel = false, rows_plan = false;
  if (!fast && g == 1 && pw == 0 && pw_r == 0 && dw == 1 && y * x > 1 && ti != ROCK_F32 &&
      bool_or(o, "layout_conversion", true) && bool_or(o, "tap_rows", true)) {
    int64_t cpad = 1;
    while (cpad < c || cpad * es < 4)
      cpad *= 2;
    while ((sw * cpad * es) % 16 != 0 && cpad * es < 16)
      cpad *= 2;
    const int64_t pix_bytes = cpad * es;
    const int64_t run = (x * pix_bytes + 15) / 16 * 16 / es; // elements of a row of taps, in whole chunks
    const int64_t in_bytes = align256(n * hi * wi * pix_bytes + run * es); // the last run reaches past the end
    const int64_t fil_bytes = align256(k * y * run * es);
    if ((c * es) % 16 != 0 && pix_bytes < 16 && (sw * pix_bytes) % 16 == 0 && (wi * pix_bytes) % 16 == 0 &&
        in_bytes < ((int64_t)1 << 31) && (256 * y * run + run) * es < ((int64_t)1 << 31) && y * run <= INT32_MAX) {
      const int ws = p.epi.residual_op ? 5 : 4;
      h->kernel_count = 3;
      h->workspace_bytes = (size_t)(fil_bytes + in_bytes);
      h->caller_pointers = ws + 1;
      planned = true;
      const int kid = (int)int_or(o, "kernel_id", 0);
      if (kid == 0 || kid == 1) {
        const bool is_f = kid == 0;
        // dimensions in destination order: g k y x c ; n h w g c
        const int64_t size_f[5] = {1, k, y, run / cpad, cpad}, from_f[5] = {1, k, y, x, c};
        const int64_t stride_f[5] = {p.fil_gs, p.fil_ks, p.fil_ys, p.fil_xs, p.fil_cs};
        const int64_t size_i[5] = {n, hi, wi, 1, cpad}, from_i[5] = {n, hi, wi, 1, c};
        const int64_t stride_i[5] = {p.in_ns, p.in_hs, p.in_ws, p.in_gs, p.in_cs};
        const int callers = h->caller_pointers;
        if (!fill_relayout_handle(h, is_f ? size_f : size_i, is_f ? from_f : from_i, is_f ? stride_f : stride_i, es)) {
          delete h;
          return nullptr;
        }
        h->caller_pointers = callers;
        h->ptr_map = {{is_f ? 0 : 1, 0}, {ws, is_f ? 0 : fil_bytes}};
        h->problem_key = std::string("relayout ") + (is_f ? "filter " : "input ") + (is_f ? fl : il) + " into rows of taps";
        return h;
      }
      p.c = (int)run; p.x = 1;
      p.in_cs = 1; p.in_gs = 0; p.in_ws = cpad; p.in_hs = wi * cpad; p.in_ns = hi * wi * cpad;
      p.fil_cs = 1; p.fil_xs = run; p.fil_ys = run; p.fil_ks = y * run; p.fil_gs = k * y * run;
      p.run_valid = x * cpad < run ? (int)(x * cpad) : 0;
      c = run;
      Kg = y * run;
      p.K = (int)Kg;
      fast = true;
      rows_plan = true;
      runs_kernel = p.run_valid != 0;
      h->ptr_map = {{ws, 0}, {ws, fil_bytes}, {2, 0}, {3, 0}, {p.epi.residual_op ? 4 : -1, 0}};
    }
  }

  // Layout-conversion plan.  A problem whose filter or input is not
  // channel-contiguous (the reference's default gkcyx / ngchw) would run the
  // element-wise kernel; if the channel-contiguous form qualifies for the
  // vector kernels, the tensors are first copied into that form in a
  // workspace by one relayout kernel each, and the contraction kernel reads
  // the copies (and writes the caller's output layout directly).  This is the
  // reference's multi-kernel protocol (miirGetKernelCount / --kernel_id /
  // miirGetWorkspaceSize, rocmlir-lib.cpp:150-199) which it uses for its
  // backward convolutions with their utility kernels.
  {
    // channel runs that are not whole 16-byte chunks (the 3-channel first layer
    // of a CNN) are zero-padded up to one by the conversion kernels
    const int64_t cp = (c * es + 15) / 16 * 16 / es;
    RockConvParams q = p;
    q.c = (int)cp;
    q.K = (int)(cp * y * x);
    const bool need_i = cp != c || !(p.in_cs == 1 && al(p.in_ws) && al(p.in_hs) && al(p.in_ns) && al(p.in_gs));
    // a strided 1x1 filter without padding reads one pixel in stride_h * stride_w:
    // the conversion copies only those, and the contraction runs with unit stride
    const bool shrink = need_i && y == 1 && x == 1 && ph == 0 && pw == 0 && ph_r == 0 && pw_r == 0 && (sh > 1 || sw > 1);
    const int64_t hi2 = shrink ? ho : hi, wi2 = shrink ? wo : wi;
    if (shrink) {
      q.hi = (int)ho; q.wi = (int)wo;
      q.stride_h = q.stride_w = 1;
    }
    const int64_t fsz[5] = {g, k, cp, y, x}, isz[5] = {n, g, cp, hi2, wi2};        // converted tensors
    const int64_t fsz_src[5] = {g, k, c, y, x}, isz_src[5] = {n, g, c, hi2, wi2};  // the caller's
    int64_t fs[5], is[5];
    layout_strides("gkyxc", "gkcyx", fsz, fs);
    layout_strides("nhwgc", "ngchw", isz, is);
    q.fil_gs = fs[0]; q.fil_ks = fs[1]; q.fil_cs = fs[2]; q.fil_ys = fs[3]; q.fil_xs = fs[4];
    q.in_ns = is[0]; q.in_gs = is[1]; q.in_cs = is[2]; q.in_hs = is[3]; q.in_ws = is[4];
    const bool need_f = cp != c || !(p.fil_cs == 1 && p.fil_xs == c && p.fil_ys == x * c && al(p.fil_ks) && al(p.fil_gs));
    const int64_t fil_bytes = (g * k * cp * y * x * es + 255) / 256 * 256;
    const int64_t in_bytes = (n * g * cp * hi2 * wi2 * es + 255) / 256 * 256;
    if (!fast && cp * y * x <= INT32_MAX && conv_fast(q, cp) && bool_or(o, "layout_conversion", true)) {
      if (!need_f) { // keep the caller's filter
        q.fil_gs = p.fil_gs; q.fil_ks = p.fil_ks; q.fil_cs = p.fil_cs; q.fil_ys = p.fil_ys; q.fil_xs = p.fil_xs;
      }
      if (!need_i) {
        q.in_ns = p.in_ns; q.in_gs = p.in_gs; q.in_cs = p.in_cs; q.in_hs = p.in_hs; q.in_ws = p.in_ws;
      }
      const int n_relayout = (need_f ? 1 : 0) + (need_i ? 1 : 0);
      const int64_t off_f = 0, off_i = need_f ? fil_bytes : 0;
      h->kernel_count = n_relayout + 1;
      h->workspace_bytes = (size_t)((need_f ? fil_bytes : 0) + (need_i ? in_bytes : 0));
      if (S > 1) { // the partial sums behind the converted tensors, the reduction kernel behind the contraction
        conv_kid = n_relayout;
        part_off = (int64_t)h->workspace_bytes;
        h->kernel_count += 1;
        h->workspace_bytes += (size_t)part_bytes;
      }
      // filter, input, output, bias, [residual,] workspace
      const int ws = p.epi.residual_op ? 5 : 4;
      h->caller_pointers = ws + 1;
      planned = true;
      const int kid = (int)int_or(o, "kernel_id", 0);
      const bool is_f = need_f && kid == 0, is_i = need_i && kid == (need_f ? 1 : 0);
      if (is_f || is_i) {
        // this handle is one of the conversion kernels
        const int64_t *sz = is_f ? fsz : isz;             // sizes in the letter order "gkcyx" / "ngchw"
        const int64_t *sz_src = is_f ? fsz_src : isz_src; // the source is shorter along c when padding
        // dimensions listed in destination (channel-contiguous) order
        const int order_f[5] = {0, 1, 3, 4, 2}, order_i[5] = {0, 3, 4, 1, 2}; // g k y x c ; n h w g c
        const int64_t src_f[5] = {p.fil_gs, p.fil_ks, p.fil_cs, p.fil_ys, p.fil_xs};
        const int64_t src_i[5] = {p.in_ns, p.in_gs, p.in_cs, p.in_hs * (shrink ? sh : 1), p.in_ws * (shrink ? sw : 1)};
        int64_t rsize[5], rsrc_size[5], rstride[5];
        for (int d = 0; d < 5; ++d) {
          const int letter = is_f ? order_f[d] : order_i[d];
          rsize[d] = sz[letter];
          rsrc_size[d] = sz_src[letter];
          rstride[d] = is_f ? src_f[letter] : src_i[letter];
        }
        const int callers = h->caller_pointers;
        if (!fill_relayout_handle(h, rsize, rsrc_size, rstride, es)) {
          delete h;
          return nullptr;
        }
        h->caller_pointers = callers;
        h->ptr_map = {{is_f ? 0 : 1, 0}, {ws, is_f ? off_f : off_i}};
        h->problem_key = std::string("relayout ") + (is_f ? "filter " : "input ") + (is_f ? fl : il);
        return h;
      }
      // this handle is the contraction kernel reading the converted tensors
      p = q;
      c = cp;
      Kg = cp * y * x;
      fast = true;
      h->ptr_map = {{need_f ? ws : 0, need_f ? off_f : 0}, {need_i ? ws : 1, need_i ? off_i : 0}, {2, 0}, {3, 0},
                    {p.epi.residual_op ? 4 : -1, 0}};
    }
  }
  p.k_order_yxc = (p.in_cs == 1) ? 1 : 0;
  int64_t groups = g;
  if (S > 1 && fast && !rows_plan) {
    if (!planned) { // the tensors as they lie: the contraction, then the reduction
      planned = true;
      h->kernel_count = 2;
      h->workspace_bytes = (size_t)part_bytes;
      h->caller_pointers = 5;
      h->ptr_map = {{0, 0}, {1, 0}, {2, 0}, {3, 0}, {-1, 0}};
    }
    const int kid = (int)int_or(o, "kernel_id", 0);
    if (kid == conv_kid + 1) {
      RockReduceParams r;
      std::memset(&r, 0, sizeof r);
      r.split_stride = Mg * k;
      r.size[0] = (int)n; r.size[1] = (int)ho; r.size[2] = (int)wo; r.size[3] = (int)k;
      r.dst_stride[0] = p.out_ns; r.dst_stride[1] = p.out_hs; r.dst_stride[2] = p.out_ws; r.dst_stride[3] = p.out_ks;
      r.splits = (int)S;
      r.out_dtype = to;
      r.int_partials = ti == ROCK_I8 ? 1 : 0;
      h->op = OP_RELAYOUT;
      h->epi = nullptr;
      h->params.assign(sizeof r, 0); // p is gone from here on
      std::memcpy(h->params.data(), &r, sizeof r);
      h->kernel_name = "rock_reduce_splits";
      h->block_size = 256;
      h->grid_size = (uint32_t)((Mg * k + 255) / 256);
      h->num_pointers = 2;
      h->perf_config = "";
      h->ptr_map = {{4, part_off}, {2, 0}};
      h->problem_key = "reduction of the split partial sums";
      return h;
    }
    if (kid != conv_kid) {
      set_error("conv: kernel_id out of range");
      delete h;
      return nullptr;
    }
    groups = S;
    p.g = (int)S;
    p.K = (int)k_part;
    p.k_group_stride = (int)k_part;
    p.in_gs = 0;
    p.fil_gs = k_part;
    p.out_ks = 1; p.out_ws = k; p.out_hs = wo * k; p.out_ns = ho * wo * k; p.out_gs = Mg * k;
    p.epi.out_dtype = ti == ROCK_I8 ? ROCK_I32 : ROCK_F32;
    h->ptr_map[2] = Handle::PtrSrc{4, part_off};
  }
  const Tile *tile = runs_kernel ? &kFastTiles[3]
                     : fast      ? pick_tile(Mg, k, (int)groups, true, forced_tile(o))
                                 : nullptr;
  if (!tile)
    tile = fast ? pick_tile(Mg, k, (int)groups, true, "") : &kGenericTile;
  apply_tile_grid(*tile, Mg, k, (int)groups, p.tiles_m, p.tiles_n, p.group_m, p.xcd_remap,
                  h->block_size, h->grid_size);
  h->kernel_name = std::string("rock_conv_") + dtype_name(ti) + tile->suffix + (runs_kernel ? "_runs" : "") +
                   rich_suffix(p.epi, fast, o);
  h->num_pointers = 5;
  if (!planned)
    set_contraction_pointers(h, p.epi);
  h->perf_config = with_block_splits(perf_string(*tile, es, &o), S);

  // Window-resident kernel (conv_direct.h): stride 1, dilation 1, a filter of
  // more than one tap, channel run a power of two of 128..1024 bytes, whole
  // 32-channel blocks of output channels, output rows that fit the tile's
  // pixels and a window of TH + Y - 1 padded rows (Y - 1 more when tiles
  // straddle two images) within 80 KiB of LDS.  Two kernels: a conversion
  // kernel first stores the filter fragment-major in the workspace
  //   F'[g][32-channel block][K-step of 128 bytes][chunk 0..7][channel 0..31][16 B]
  // (every group padded with zero rows to whole 128-channel tiles), then the
  // contraction reads it with coalesced loads straight into registers.  Taken
  // on request ("-perf_config v2:224,128,...") and, for the 16-bit types and int8, by
  // itself where its tiles fill (3x3 layers of 28- and 56-wide images: 1.2-1.3x
  // the implicit-GEMM kernel; "--window_resident false" declines); a request that cannot be met falls back to the
  // table like any other perf_config.
  if (!planned && fast) {
    const WindowPlan w = window_plan(p, ti, ph_r == ph && pw_r == pw, o);
    const bool rows_as_they_lie = p.fil_cs == 1 && p.fil_xs == c && p.fil_ys == x * c;
    if (w.ok && rows_as_they_lie && (requested_tile_is(o, kDirectTilePixels, 128) || w.by_itself)) {
      const int64_t kbytes = Kg * es; // a whole number of 128-byte K-steps
      const int ws = p.epi.residual_op ? 5 : 4;
      const int kid = (int)int_or(o, "kernel_id", 0);
      h->kernel_count = 2;
      h->workspace_bytes = (size_t)w.filter_bytes;
      if (kid == 0) {
        const int64_t e = 16 / es;
        const int64_t size[5] = {g, w.tiles_n * 4, kbytes / 16, 32, e};
        const int64_t src_size[5] = {g, k / 32, kbytes / 16, 32, e};
        const int64_t stride[5] = {p.fil_gs, 32 * p.fil_ks, e, p.fil_ks, 1};
        if (!fill_relayout_handle(h, size, src_size, stride, es)) {
          delete h;
          return nullptr;
        }
        h->kernel_count = 2;
        h->workspace_bytes = (size_t)w.filter_bytes;
        h->caller_pointers = ws + 1;
        h->ptr_map = {{0, 0}, {ws, 0}};
        h->problem_key = "repack filter " + fl;
        return h;
      }
      apply_window_plan(h, p, w, ti, o);
      h->caller_pointers = ws + 1;
      h->ptr_map = {{ws, 0}, {1, 0}, {2, 0}, {3, 0}, {p.epi.residual_op ? 4 : -1, 0}};
    }
  }
  set_problem_key();
  return h;
}

// Attention outside the fused kernel's reach (head dimensions above 256, f32):
// three kernels over a workspace of f32 scores -- the GEMM Q K^T, a row softmax
// that applies scale tensor, scale, bias and mask and narrows the probabilities
// in place, and the GEMM P V.  The reference fuses every shape
// (GridwiseGemmToBlockwise.cpp:1607-2403); its validator computes these same
// three steps (rocmlir-gen.cpp:2565-2620).
// A score matrix that fits the array of rockamdLaunchStaticWorkspace is worked
// on in one piece.  A larger one is worked off in chunks of kScoreChunkBytes --
// whole groups, or query rows of one group -- each with its own kernels in the
// list (kernel_id = kernels per chunk * chunk + step): the workspace holds one
// chunk, small enough for that array and for the scores to stay in the
// memory-side cache between the kernels, instead of G * seq_q * seq_k * 4
// bytes.  A chunk of one group's rows leaves the second GEMM few output tiles
// and a long reduction; that one is split over blocks as a GEMM of its own
// would be (f32 partial sums behind the scores, a fourth kernel adds them up).
constexpr int64_t kScoreWholeBytes = ROCKAMD_STATIC_WORKSPACE_BYTES - ((int64_t)16 << 20); // room for the partial sums
constexpr int64_t kScoreChunkBytes = (int64_t)32 << 20;
Handle *make_attention_unfused(const OptMap &o, int ty, int64_t G, int64_t sq, int64_t sk, int64_t dqk, int64_t dv,
                               bool tQ, bool tK, bool tV, bool tO, bool has_bias, bool has_scale_t, bool has_mask) {
  // "-t i8": Q and K are int8, their product is dequantised before the softmax
  // ((acc - zero_point) * scale, the scalars rocmlir-gen passes as [1,1,1]
  // tensors, rocmlir-gen.cpp:2173-2184, 2353-2367); V, the pre-softmax tensors
  // and O are f16
  const int tq = ty;
  if (ty == ROCK_I8)
    ty = ROCK_F16;
  const int es = dtype_size(ty);
  // chunk = gc groups x rc query rows
  // ("-score_workspace_limit BYTES" moves the bound, e.g. to keep one chunk inside a smaller cache share)
  const int64_t limit =
      std::max<int64_t>(int_or(o, "score_workspace_limit", G * sq * sk * 4 <= kScoreWholeBytes ? kScoreWholeBytes
                                                                                                : kScoreChunkBytes),
                        sk * 4);
  int64_t gc = G, rc = sq;
  if (G * sq * sk * 4 > limit) {
    if (sq * sk * 4 <= limit) {
      gc = limit / (sq * sk * 4);
    } else {
      gc = 1;
      rc = std::max<int64_t>(1, limit / (sk * 4));
      rc = rc >= 128 ? rc / 128 * 128 : rc >= 8 ? rc / 8 * 8 : rc; // chunk boundaries on whole tiles / 16-byte columns
    }
  }
  const int64_t row_chunks = ceil_div(sq, rc), chunks = ceil_div(G, gc) * row_chunks;
  // the second GEMM of a one-group chunk: its reduction over the keys in S shares (as make_gemm splits a GEMM)
  int64_t S = 1;
  if (gc == 1 && bool_or(o, "split_k", true)) {
    const int64_t tiles64 = (int64_t)ceil_div(rc, 64) * ceil_div(dv, 64);
    if (sk >= 2048 && tiles64 * 2 <= kNumCU)
      for (int64_t d = std::min<int64_t>(2 * kNumCU / tiles64, sk / 512); d >= 2 && S == 1; --d)
        if (sk % d == 0 && (sk / d * es) % 64 == 0)
          S = d;
  }
  const int per_chunk = S > 1 ? 4 : 3;
  const int64_t score_bytes = align256(gc * rc * sk * 4), partial_bytes = S > 1 ? align256(S * rc * dv * 4) : 0;
  const int64_t kid_all = int_or(o, "kernel_id", 0);
  if (chunks * per_chunk > INT32_MAX || gc * rc > INT32_MAX) {
    set_error("attention: score matrix too large for the three-kernel form");
    return nullptr;
  }
  if (kid_all < 0 || kid_all >= per_chunk * chunks) {
    set_error("attention: kernel_id out of range");
    return nullptr;
  }
  const int kid = (int)(kid_all % per_chunk);
  const int64_t g0 = kid_all / per_chunk / row_chunks * gc, r0 = kid_all / per_chunk % row_chunks * rc;
  const int64_t gn = std::min(gc, G - g0), rn = std::min(rc, sq - r0); // this chunk
  float scale = 1.0f;
  get_float(o, "scale", scale);
  // caller list: Q, K, V, [scale tensor], bias slot, [mask, other], O, workspace
  const int i_bias = has_scale_t ? 4 : 3, i_mask = has_mask ? i_bias + 1 : -1, i_other = has_mask ? i_bias + 2 : -1,
            i_out = i_bias + 1 + (has_mask ? 2 : 0), i_ws = i_out + 1;
  const int64_t pitch_p = 4 / es; // elements of P per f32 score: P lies in place, rows sk * 4 bytes apart
  auto *h = new Handle;
  if (kid == 1) {
    RockSoftmaxParams r;
    std::memset(&r, 0, sizeof r);
    r.row_pitch = sk;
    r.t_gs = sq * sk; r.t_is = sk; r.t_js = 1;
    r.G = (int)gn; r.seq_q = (int)rn; r.seq_k = (int)sk;
    r.scale = scale;
    r.has_bias = has_bias ? 1 : 0;
    r.has_scale_tensor = has_scale_t ? 1 : 0;
    r.has_mask = has_mask ? 1 : 0;
    r.dtype = ty;
    h->op = OP_RELAYOUT;
    h->epi = nullptr;
    h->params.assign(sizeof r, 0);
    std::memcpy(h->params.data(), &r, sizeof r);
    h->kernel_name = "rock_softmax_rows";
    h->block_size = sk > 4096 ? 1024 : 256; // rows up to 16 scores per thread stay in registers
    h->grid_size = (uint32_t)(gn * rn);
    h->num_pointers = 5;
    h->perf_config = "";
    const int64_t t_off = (g0 * sq * sk + r0 * sk) * es; // the chunk's first row in the [G, seq_q, seq_k] tensors
    h->ptr_map = {{i_ws, 0}, {has_scale_t ? 3 : -1, t_off}, {has_bias ? i_bias : -1, t_off}, {i_mask, t_off / es},
                  {i_other, t_off}};
    h->problem_key = "row softmax of the attention scores";
  } else if (kid == 3) { // O = the sum of the shares' partial results
    RockReduceParams r;
    std::memset(&r, 0, sizeof r);
    r.split_stride = rn * dv;
    r.size[0] = 1; r.size[1] = 1; r.size[2] = (int)rn; r.size[3] = (int)dv;
    r.dst_stride[2] = tO ? 1 : dv; r.dst_stride[3] = tO ? sq : 1;
    r.splits = (int)S;
    r.out_dtype = ty;
    h->op = OP_RELAYOUT;
    h->epi = nullptr;
    h->params.assign(sizeof r, 0);
    std::memcpy(h->params.data(), &r, sizeof r);
    h->kernel_name = "rock_reduce_splits";
    h->block_size = 256;
    h->grid_size = (uint32_t)((rn * dv + 255) / 256);
    h->num_pointers = 2;
    h->perf_config = "";
    h->ptr_map = {{i_ws, score_bytes}, {i_out, (g0 * sq * dv + r0 * (tO ? 1 : dv)) * es}};
    h->problem_key = "reduction of the split partial sums";
  } else {
    RockGemmParams gp;
    std::memset(&gp, 0, sizeof gp);
    gp.G = (int)gn;
    int64_t a_off, b_off, c_off; // bytes from the tensors' starts to the chunk
    if (kid == 0) { // S[g,i,j] = sum_d Q[g,i,d] K[g,j,d], f32
      gp.M = (int)rn; gp.N = (int)sk; gp.K = (int)dqk;
      gp.a_gs = sq * dqk; gp.a_ms = tQ ? 1 : dqk; gp.a_ks = tQ ? sq : 1;
      gp.b_gs = sk * dqk; gp.b_ns = tK ? dqk : 1; gp.b_ks = tK ? 1 : sk;
      gp.c_gs = rn * sk; gp.c_ms = sk; gp.c_ns = 1;
      a_off = (g0 * gp.a_gs + r0 * gp.a_ms) * dtype_size(tq);
      b_off = g0 * gp.b_gs * dtype_size(tq);
      c_off = 0;
      default_epilogue(gp.epi, ROCK_F32);
      gp.epi.zero_point = (int32_t)int_or(o, "zero_point", 0); // i8: scores leave as float(acc) - zero_point
    } else { // O[g,i,e] = sum_j P[g,i,j] V[g,j,e]
      gp.M = (int)rn; gp.N = (int)dv; gp.K = (int)sk;
      gp.a_gs = rn * sk * pitch_p; gp.a_ms = sk * pitch_p; gp.a_ks = 1;
      gp.b_gs = sk * dv; gp.b_ns = tV ? sk : 1; gp.b_ks = tV ? 1 : dv;
      gp.c_gs = sq * dv; gp.c_ms = tO ? 1 : dv; gp.c_ns = tO ? sq : 1;
      default_epilogue(gp.epi, ty);
      a_off = 0;
      b_off = g0 * gp.b_gs * es;
      c_off = (g0 * gp.c_gs + r0 * gp.c_ms) * es;
      if (S > 1) { // share s: keys s * sk / S onwards, f32 partial result s behind the scores
        const int64_t ks = sk / S;
        gp.G = (int)S; gp.K = (int)ks;
        gp.a_gs = ks; gp.b_gs = ks * gp.b_ks;
        gp.c_gs = rn * dv; gp.c_ms = dv; gp.c_ns = 1;
        default_epilogue(gp.epi, ROCK_F32);
        c_off = score_bytes;
      }
    }
    const int tg = kid == 0 ? tq : ty;
    plan_gemm_kernel(h, gp, operand_code(tg, tg), dtype_size(tg), o);
    if (kid == 0)
      h->ptr_map = {{0, a_off}, {1, b_off}, {i_ws, c_off}, {-1, 0}, {-1, 0}};
    else
      h->ptr_map = {{i_ws, a_off}, {2, b_off}, {S > 1 ? i_ws : i_out, c_off}, {-1, 0}, {-1, 0}};
    h->op = OP_GEMM;
    h->params.assign(sizeof gp, 0);
    std::memcpy(h->params.data(), &gp, sizeof gp);
    h->epi = &reinterpret_cast<RockGemmParams *>(h->params.data())->epi;
    std::ostringstream key;
    auto tf = [](bool b) { return b ? "true" : "false"; };
    key << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << "-t " << dtype_name(tq) << " -transQ " << tf(tQ)
        << " -transK " << tf(tK) << " -transV " << tf(tV) << " -transO " << tf(tO) << " -g " << G << " -seq_len_q "
        << sq << " -seq_len_k " << sk << " -head_dim_qk " << dqk << " -head_dim_v " << dv;
    h->problem_key = key.str();
  }
  h->kernel_count = (int)(per_chunk * chunks);
  h->workspace_bytes = (size_t)(partial_bytes ? score_bytes + partial_bytes : gc * rc * sk * 4);
  h->caller_pointers = i_ws + 1;
  return h;
}

// ---- attention --------------------------------------------------------------------
Handle *make_attention(const OptMap &o) {
  std::string t = str_or(o, "t", "f16");
  int ty = parse_dtype(t);
  if (ty != ROCK_F16 && ty != ROCK_BF16 && ty != ROCK_F32 && ty != ROCK_I8) {
    set_error("attention: f16, bf16, f32 and i8 (quantised first GEMM) kernels are built ('" + t + "' requested)");
    return nullptr;
  }
  int64_t G = int_or(o, "g", 1), sq, sk, dqk, dv;
  if (!get_int(o, "seq_len_q", sq) || !get_int(o, "seq_len_k", sk) ||
      !get_int(o, "head_dim_qk", dqk) || !get_int(o, "head_dim_v", dv) || G <= 0 || sq <= 0 ||
      sk <= 0 || dqk <= 0 || dv <= 0) {
    set_error("attention: -seq_len_q, -seq_len_k, -head_dim_qk, -head_dim_v must be positive");
    return nullptr;
  }
  bool tQ = bool_or(o, "transQ", false), tK = bool_or(o, "transK", false),
       tV = bool_or(o, "transV", false), tO = bool_or(o, "transO", false);
  bool has_bias = bool_or(o, "with-attn-bias", false);
  // "-with-attn-scale": a full [G, seq_q, seq_k] tensor multiplied into the
  // scores before the softmax (rocmlir-gen.cpp:2185-2196), besides the scalar "-scale"
  bool has_scale_t = bool_or(o, "with-attn-scale", false);
  // "-with-attn-mask": migraphx.where(mask, scores, other) in front of the softmax (mixr-attn-where.mlir:11) --
  // an int8 mask and a tensor of replacement scores, both [G, seq_q, seq_k], behind the bias in the caller's list.
  // Where the mask is zero the score (after scale tensor, scale and bias) is replaced, not added to.
  const bool has_mask = bool_or(o, "with-attn-mask", false);
  // "-t i8": int8 Q and K (the quantised first GEMM), f16 V, pre-softmax tensors and O
  const bool qk_i8 = ty == ROCK_I8;
  // Transposed Q, V or O ([G, d, seq_q], [G, dv, seq_k], [G, dv, seq_q]): the fused vector kernels want the
  // head dimension contiguous.  Conversion kernels in front copy Q and V into that layout, one behind writes
  // the result as the caller laid it out, and the fused kernel in between runs on the copies -- the
  // multi-kernel protocol of the convolution plans (rocmlir-lib.cpp:150-199).  The reference reaches every
  // storage through its coordinate transforms (rocmlir-gen.cpp:2149-2200).  "-layout_conversion false", or a
  // problem whose untransposed twin has no fused vector kernel, leaves the tensors to the kernels that read
  // them as they lie (element-wise gathers, or the GEMMs of the three-kernel form).
  // K stored [G, d, seq_k] is read as it lies by the "_kt" kernels when its rows of keys are whole 16-byte
  // chunks; otherwise (seq_k = 27; int8 keys) it is copied to [G, seq_k, d] the same way.
  const bool copy_k = !tK && (qk_i8 || sk % 8 != 0);
  if ((tQ || tV || tO || copy_k) && ty != ROCK_F32 && bool_or(o, "layout_conversion", true)) {
    OptMap inner = o;
    inner["transQ"] = inner["transV"] = inner["transO"] = "false";
    if (copy_k)
      inner["transK"] = "true";
    inner.erase("kernel_id");
    const std::string keep_error = g_last_error;
    Handle *core = make_attention(inner);
    const bool usable = core && core->op == OP_ATTENTION && core->kernel_count == 1 &&
                        core->kernel_name.find("_generic") == std::string::npos;
    if (!usable) {
      delete core;
      g_last_error = keep_error;
    } else {
      const int es_q = qk_i8 ? 1 : 2;
      const int64_t q_bytes = tQ ? align256(G * sq * dqk * es_q) : 0, v_bytes = tV ? align256(G * sk * dv * 2) : 0,
                    o_bytes = tO ? align256(G * sq * dv * 2) : 0, k_bytes = copy_k ? align256(G * sk * dqk * es_q) : 0;
      const int64_t q_off = 0, v_off = q_bytes, o_off = q_bytes + v_bytes, k_off = o_off + o_bytes;
      // caller pointers: Q, K, V, [scale tensor,] bias, [mask, other,] O, workspace
      const int i_scale = has_scale_t ? 3 : -1, i_bias = has_scale_t ? 4 : 3, i_mask = has_mask ? i_bias + 1 : -1,
                i_other = has_mask ? i_bias + 2 : -1, i_out = i_bias + 1 + (has_mask ? 2 : 0), i_ws = i_out + 1;
      std::vector<int> kinds; // 0 = Q copy, 1 = V copy, 4 = K copy, 2 = the fused kernel, 3 = O written in the caller's layout
      if (tQ) kinds.push_back(0);
      if (tV) kinds.push_back(1);
      if (copy_k) kinds.push_back(4);
      kinds.push_back(2);
      if (tO) kinds.push_back(3);
      const int kid = (int)int_or(o, "kernel_id", 0);
      if (kid < 0 || kid >= (int)kinds.size()) {
        set_error("attention: kernel_id out of range");
        delete core;
        return nullptr;
      }
      Handle *h = core;
      const std::string problem_key = core->problem_key;
      if (kinds[kid] != 2) {
        h = new Handle;
        h->arch = core->arch;
        bool ok;
        if (kinds[kid] == 0) { // [G, d, seq_q] -> [G, seq_q, d]
          const int64_t size[5] = {1, 1, G, sq, dqk}, stride[5] = {0, 0, sq * dqk, 1, sq};
          ok = fill_relayout_handle(h, size, size, stride, es_q);
          h->ptr_map = {{0, 0}, {i_ws, q_off}};
          h->problem_key = "relayout attention Q";
        } else if (kinds[kid] == 1) { // [G, dv, seq_k] -> [G, seq_k, dv]
          const int64_t size[5] = {1, 1, G, sk, dv}, stride[5] = {0, 0, sk * dv, 1, sk};
          ok = fill_relayout_handle(h, size, size, stride, 2);
          h->ptr_map = {{2, 0}, {i_ws, v_off}};
          h->problem_key = "relayout attention V";
        } else if (kinds[kid] == 4) { // [G, d, seq_k] -> [G, seq_k, d]
          const int64_t size[5] = {1, 1, G, sk, dqk}, stride[5] = {0, 0, sk * dqk, 1, sk};
          ok = fill_relayout_handle(h, size, size, stride, es_q);
          h->ptr_map = {{1, 0}, {i_ws, k_off}};
          h->problem_key = "relayout attention K";
        } else { // [G, seq_q, dv] -> [G, dv, seq_q]
          const int64_t size[5] = {1, 1, G, dv, sq}, stride[5] = {0, 0, sq * dv, 1, dv};
          ok = fill_relayout_handle(h, size, size, stride, 2);
          h->ptr_map = {{i_ws, o_off}, {i_out, 0}};
          h->problem_key = "relayout attention O";
        }
        delete core;
        if (!ok) {
          delete h;
          return nullptr;
        }
      } else {
        h->ptr_map = {tQ ? Handle::PtrSrc{i_ws, q_off} : Handle::PtrSrc{0, 0},
                      copy_k ? Handle::PtrSrc{i_ws, k_off} : Handle::PtrSrc{1, 0},
                      tV ? Handle::PtrSrc{i_ws, v_off} : Handle::PtrSrc{2, 0}, {i_scale, 0}, {i_bias, 0},
                      {i_mask, 0}, {i_other, 0},
                      tO ? Handle::PtrSrc{i_ws, o_off} : Handle::PtrSrc{i_out, 0}};
        // the key names the problem as the caller posed it
        auto tf = [](bool b) { return b ? "true" : "false"; };
        std::ostringstream key;
        key << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << "-t " << dtype_name(ty) << " -transQ " << tf(tQ)
            << " -transK " << tf(tK) << " -transV " << tf(tV) << " -transO " << tf(tO) << " -g " << G << " -seq_len_q "
            << sq << " -seq_len_k " << sk << " -head_dim_qk " << dqk << " -head_dim_v " << dv;
        h->problem_key = key.str();
      }
      h->kernel_count = (int)kinds.size();
      h->workspace_bytes = (size_t)(q_bytes + v_bytes + o_bytes + k_bytes);
      h->caller_pointers = i_ws + 1;
      return h;
    }
  }
  {
    // the fused kernels: head dimensions up to 128, tensors contiguous along the head dimension in
    // whole 16-byte chunks; int8 Q and K only on the vector kernels
    const bool i8_fused = qk_i8 && !tQ && tK && !tV && !tO && dqk % 16 == 0 && dv % 8 == 0 &&
                          sk * dqk < ((int64_t)1 << 31) && sk * dv * 2 < ((int64_t)1 << 31) &&
                          ((!has_bias && !has_scale_t && !has_mask) || sq * sk < ((int64_t)1 << 31)) &&
                          bool_or(o, "fused", true);
    // 16-bit types up to 256 on the vector kernel (head-dimension-contiguous tensors, checked below)
    // (K either way: [seq_k, d], or the reference's default [d, seq_k] with whole 16-byte rows of keys)
    const bool wide_ok = !qk_i8 && !tQ && (tK || sk % 8 == 0) && !tV && !tO && dqk % 8 == 0 && dv % 8 == 0 &&
                         bool_or(o, "fused", true);
    const int64_t dlimit = wide_ok ? 256 : 128;
    if (ty == ROCK_F32 || (qk_i8 && (!i8_fused || dqk > 128 || dv > 128)) || dqk > dlimit || dv > dlimit)
      return make_attention_unfused(o, ty, G, sq, sk, dqk, dv, tQ, tK, tV, tO, has_bias, has_scale_t, has_mask);
  }

  auto *h = new Handle;
  h->op = OP_ATTENTION;
  h->params.assign(sizeof(RockAttentionParams), 0);
  auto &p = *reinterpret_cast<RockAttentionParams *>(h->params.data());
  // storage (rocmlir-gen.cpp:2149-2200): Q [G,sq,d] (transQ: [G,d,sq]);
  // K [G,d,sk] (transK: [G,sk,d]); V [G,sk,dv] (transV: [G,dv,sk]);
  // O [G,sq,dv] (transO: [G,dv,sq])
  p.G = (int)G; p.seq_q = (int)sq; p.seq_k = (int)sk; p.d_qk = (int)dqk; p.d_v = (int)dv;
  p.q_gs = sq * dqk; p.q_is = tQ ? 1 : dqk; p.q_ds = tQ ? sq : 1;
  p.k_gs = sk * dqk; p.k_js = tK ? dqk : 1; p.k_ds = tK ? 1 : sk;
  p.v_gs = sk * dv; p.v_js = tV ? 1 : dv; p.v_es = tV ? sk : 1;
  p.o_gs = sq * dv; p.o_is = tO ? 1 : dv; p.o_es = tO ? sq : 1;
  p.bias_gs = sq * sk; p.bias_is = sk; p.bias_js = 1;
  p.has_bias = has_bias ? 1 : 0;
  p.has_scale_tensor = has_scale_t ? 1 : 0;
  p.has_mask = has_mask ? 1 : 0;
  p.scale = 1.0f;
  get_float(o, "scale", p.scale);
  p.zero_point = qk_i8 ? (int32_t)int_or(o, "zero_point", 0) : 0;
  p.q_blocks = ceil_div(sq, 128);
  int64_t total = G * p.q_blocks;
  if (total > INT32_MAX) {
    set_error("attention: too many blocks");
    delete h;
    return nullptr;
  }
  p.xcd_remap = total >= 2 * kNumXCD ? 1 : 0;
  // K stored [d, seq_k] (no -transK: the reference's default) goes to the "_kt" twins of the vector kernels,
  // which take the S^T row operand out of a [d][64 keys] tile through the transposing LDS read
  const bool kt = !qk_i8 && !tK;
  const bool k_fast = kt ? (p.k_js == 1 && p.k_ds % 8 == 0 && dqk * p.k_ds * 2 < ((int64_t)1 << 31))
                         : (p.k_ds == 1 && p.k_js % 8 == 0 && sk * p.k_js * 2 < ((int64_t)1 << 31));
  const bool fast = qk_i8 || // checked above: there is no element-wise int8 kernel to fall back to
                    p.q_ds == 1 && k_fast && p.v_es == 1 && p.o_es == 1 && dqk % 8 == 0 &&
                    dv % 8 == 0 && p.o_is % 4 == 0 && p.v_js % 8 == 0 &&
                    p.q_is % 8 == 0 &&
                    // byte offsets inside one g slice below 2^31 (buffer descriptors)
                    sk * p.v_js * 2 < ((int64_t)1 << 31) &&
                    // the bias gather indexes one g slice with 32-bit element offsets
                    ((!has_bias && !has_scale_t && !has_mask) || sq * sk < ((int64_t)1 << 31));
  const bool wide = dqk > 128 || dv > 128; // one kernel: vector loads, simple order per tile
  int dmax = (dqk <= 64 && dv <= 64) ? 64 : wide ? 256 : 128;
  const bool plain_ok = !p.has_bias && !has_scale_t && !has_mask && p.scale >= 0.0f && !wide;
  if (wide && !fast) {
    delete h;
    return make_attention_unfused(o, ty, G, sq, sk, dqk, dv, tQ, tK, tV, tO, has_bias, has_scale_t, has_mask);
  }
  const AttnVariant *variant = !fast ? &kAttnVariants[2] : plain_ok ? &kAttnVariants[0] : &kAttnVariants[1];
  {
    // a perf_config that names a kernel this problem can run on selects it;
    // anything else falls back to the table (AffixTuningParameters.cpp:129-141)
    int want_d, want_kpack, want_unroll;
    if (parse_attn_perf(str_or(o, "perf_config", ""), want_d, want_kpack, want_unroll)) {
      if ((want_d == 64 || want_d == 128) && want_d >= dmax)
        dmax = want_d;
      if (wide)
        ; // a single kernel
      else if (want_kpack == 1 && !qk_i8)
        variant = &kAttnVariants[2];
      else if (fast && want_kpack == 8)
        variant = (want_unroll != 0 && plain_ok) ? &kAttnVariants[0] : &kAttnVariants[1];
    }
  }
  char name[96];
  std::snprintf(name, sizeof name, "rock_attention_%s_d%dx%d_%s%s", dtype_name(ty), dmax, dmax, variant->kind,
                (kt && variant != &kAttnVariants[2]) ? "_kt" : "");
  h->kernel_name = name;
  // kernel pointers: Q, K, V, scale tensor, bias, mask, other, O; a caller passes the scale tensor and the
  // mask with its replacement scores only when the problem names them, the bias slot always
  h->num_pointers = 8;
  {
    const int i_bias = has_scale_t ? 4 : 3, i_out = i_bias + 1 + (has_mask ? 2 : 0);
    h->caller_pointers = i_out + 1;
    h->ptr_map = {{0, 0}, {1, 0}, {2, 0}, {has_scale_t ? 3 : -1, 0}, {i_bias, 0}, {has_mask ? i_bias + 1 : -1, 0},
                  {has_mask ? i_bias + 2 : -1, 0}, {i_out, 0}};
  }
  h->block_size = 256;
  h->grid_size = (uint32_t)total;
  // attn:v1:MPB_G0,MPB_G1,NPB_G0,KpackPB,MPW,MnPerXdl,Kpack,forceUnroll
  // (G0 M tiles seq_k, G0 N tiles seq_q)
  h->perf_config = attn_perf_string(*variant, dmax);
  {
    std::ostringstream key;
    auto tf = [](bool b) { return b ? "true" : "false"; };
    key << h->arch << '\t' << int_or(o, "num_cu", kNumCU) << '\t' << "-t " << dtype_name(ty)
        << " -transQ " << tf(tQ) << " -transK " << tf(tK) << " -transV " << tf(tV) << " -transO "
        << tf(tO) << " -g " << G << " -seq_len_q " << sq << " -seq_len_k " << sk
        << " -head_dim_qk " << dqk << " -head_dim_v " << dv;
    h->problem_key = key.str();
  }
  return h;
}

// --------------------------------------------------------------------------
// module cache: one hipModule per (device, code object)
// --------------------------------------------------------------------------
std::mutex g_module_mutex;
std::map<std::pair<int, const Blob *>, hipModule_t> g_modules;

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
  std::lock_guard<std::mutex> lock(g_module_mutex);
  hipModule_t mod;
  auto key = std::make_pair(dev, h->blob);
  auto mit = g_modules.find(key);
  if (mit == g_modules.end()) {
    e = hipModuleLoadData(&mod, h->blob->start);
    if (e != hipSuccess) {
      set_error(std::string("hipModuleLoadData failed for ") + h->blob->name + ": " +
                hipGetErrorString(e));
      return (int)e;
    }
    g_modules[key] = mod;
  } else {
    mod = mit->second;
  }
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

// What the caller's pointers are, for clients that size and check their
// buffers from the handle (the per-argument rank and dimensions MIGraphX reads
// with mlirGetKernelInfo, mlir/lib/CAPI/Dialect/MIGraphX.cpp:54-90).
void describe_arguments(const OptMap &o, Handle *h) {
  using A = Handle::ArgInfo;
  const std::string op = str_or(o, "operation", "");
  // the per-channel quantisation vectors follow the problem's own tensors, the workspace closes the list
  auto with_workspace = [&](int64_t channels = 0) {
    const int flags = channel_vector_flags(o);
    if (flags & ROCK_CHAN_SCALE)
      h->args.push_back(A{ROCK_F32, {channels}});
    if (flags & ROCK_CHAN_ZP)
      h->args.push_back(A{(flags & ROCK_CHAN_ZP_I8) ? ROCK_I8 : ROCK_I32, {channels}});
    if (flags & ROCK_CHAN_QUANT_SCALE)
      h->args.push_back(A{ROCK_F32, {channels}});
    if (flags & ROCK_CHAN_OUT_ZP)
      h->args.push_back(A{(flags & ROCK_CHAN_OUT_ZP_I8) ? ROCK_I8 : ROCK_I32, {channels}});
    if (h->workspace_bytes)
      h->args.push_back(A{-1, {(int64_t)h->workspace_bytes}});
  };
  if (op == "gemm") {
    std::string t = str_or(o, "t", "f32");
    size_t us = t.find('_');
    const int ta = parse_dtype(us == std::string::npos ? t : t.substr(0, us));
    const int tb = parse_dtype(us == std::string::npos ? t : t.substr(us + 1));
    const int tc = h->epi ? h->epi->out_dtype : -1;
    const int64_t G = int_or(o, "g", 1), M = int_or(o, "m", 0), N = int_or(o, "n", 0), K = int_or(o, "k", 0);
    const bool tA = bool_or(o, "transA", false), tB = bool_or(o, "transB", false), tC = bool_or(o, "transC", false);
    std::string outs = str_or(o, "out_datatype", str_or(o, "c_dtype", ""));
    const int dflt = ta == ROCK_I8 ? ROCK_I32 : (ta == ROCK_FP8 || ta == ROCK_BF8) ? ROCK_F32 : ta;
    const int out_t = outs.empty() ? dflt : parse_dtype(outs);
    (void)tc;
    h->args = {A{ta, tA ? std::vector<int64_t>{G, K, M} : std::vector<int64_t>{G, M, K}},
               A{tb, tB ? std::vector<int64_t>{G, N, K} : std::vector<int64_t>{G, K, N}},
               A{out_t, tC ? std::vector<int64_t>{G, N, M} : std::vector<int64_t>{G, M, N}},
               A{out_t == ROCK_I32 ? ROCK_I32 : ROCK_F32, {N}}};
    if (str_or(o, "residual", "none") != "none")
      h->args.push_back(A{out_t, h->args[2].dims});
    with_workspace(N);
  } else if (op == "attention") {
    const int t = parse_dtype(str_or(o, "t", "f16"));
    const int tv = t == ROCK_I8 ? ROCK_F16 : t;
    const int64_t G = int_or(o, "g", 1), sq = int_or(o, "seq_len_q", 0), sk = int_or(o, "seq_len_k", 0),
                  dqk = int_or(o, "head_dim_qk", 0), dv = int_or(o, "head_dim_v", 0);
    auto mat = [&](bool tr, int64_t r, int64_t c) { return tr ? std::vector<int64_t>{G, c, r} : std::vector<int64_t>{G, r, c}; };
    h->args = {A{t, mat(bool_or(o, "transQ", false), sq, dqk)}, A{t, mat(!bool_or(o, "transK", false), sk, dqk)},
               A{tv, mat(bool_or(o, "transV", false), sk, dv)}};
    if (bool_or(o, "with-attn-scale", false))
      h->args.push_back(A{tv, {G, sq, sk}});
    h->args.push_back(A{tv, {G, sq, sk}}); // bias slot
    if (bool_or(o, "with-attn-mask", false)) {
      h->args.push_back(A{ROCK_I8, {G, sq, sk}});
      h->args.push_back(A{tv, {G, sq, sk}});
    }
    h->args.push_back(A{tv, mat(bool_or(o, "transO", false), sq, dv)});
    with_workspace();
  } else if (o.count("in_d") || o.count("fil_d")) { // three spatial dimensions: six-dimensional tensors
    std::string t_all = str_or(o, "t", "");
    const int ti = parse_dtype(str_or(o, "in_type", t_all)), tf = parse_dtype(str_or(o, "fil_type", t_all));
    std::string out_t = str_or(o, "out_type", str_or(o, "out_datatype", ""));
    const int dflt = ti == ROCK_I8 ? ROCK_I32 : (ti == ROCK_FP8 || ti == ROCK_BF8) ? ROCK_F32 : ti;
    const int to = out_t.empty() ? dflt : parse_dtype(out_t);
    std::string fl, il, ol;
    if (!canon_layout3(str_or(o, "fil_layout", ""), 'k', true, fl) || !canon_layout3(str_or(o, "in_layout", ""), 'c', false, il) ||
        !canon_layout3(str_or(o, "out_layout", ""), 'k', false, ol))
      return;
    const int64_t n = int_or(o, "batchsize", 0), g = int_or(o, "groupsize", 1), c = int_or(o, "in_channels", 0) / g,
                  k = int_or(o, "out_channels", 0) / g;
    int64_t fsz[6] = {g, k, c, 0, 0, 0}, isz[6] = {n, g, c, 0, 0, 0}, osz[6] = {n, g, k, 0, 0, 0};
    static const char *ax[3] = {"h", "w", "d"};
    for (int a = 0; a < 3; ++a) {
      const std::string s = ax[a];
      const int64_t in = int_or(o, ("in_" + s).c_str(), 0), fil = int_or(o, ("fil_" + s).c_str(), 0),
                    dil = int_or(o, ("dilation_" + s).c_str(), 1), str = int_or(o, ("conv_stride_" + s).c_str(), 1),
                    both = int_or(o, ("padding_" + s).c_str(), 0), pl = int_or(o, ("padding_" + s + "_l").c_str(), both),
                    pr = int_or(o, ("padding_" + s + "_r").c_str(), both);
      fsz[3 + a] = fil;
      isz[3 + a] = in;
      osz[3 + a] = (in + pl + pr - (fil - 1) * dil - 1) / str + 1;
    }
    auto dims = [](const std::string &layout, const char *letters, const int64_t *sizes) {
      std::vector<int64_t> d;
      for (char ch : layout)
        d.push_back(sizes[std::strchr(letters, ch) - letters]);
      return d;
    };
    h->args = {A{tf, dims(fl, "gkc012", fsz)}, A{ti, dims(il, "ngc012", isz)}, A{to, dims(ol, "ngk012", osz)},
               A{to == ROCK_I32 ? ROCK_I32 : ROCK_F32, {g * k}}};
    if (str_or(o, "residual", "none") != "none")
      h->args.push_back(A{to, h->args[2].dims});
    with_workspace();
  } else { // convolutions: filter, input, output in the order of their layout strings
    std::string t_all = str_or(o, "t", "");
    const int ti = parse_dtype(str_or(o, "in_type", t_all)), tf = parse_dtype(str_or(o, "fil_type", t_all));
    std::string out_t = str_or(o, "out_type", str_or(o, "out_datatype", ""));
    const int dflt = ti == ROCK_I8 ? ROCK_I32 : (ti == ROCK_FP8 || ti == ROCK_BF8) ? ROCK_F32 : ti;
    const int to = out_t.empty() ? dflt : parse_dtype(out_t);
    std::string fl, il, ol;
    if (!canon_layout(str_or(o, "fil_layout", ""), 'k', "gkcyx", fl) || !canon_layout(str_or(o, "in_layout", ""), 'c', "ngchw", il) ||
        !canon_layout(str_or(o, "out_layout", ""), 'k', "ngkhw", ol))
      return;
    const int64_t n = int_or(o, "batchsize", 0), g = int_or(o, "groupsize", 1), c = int_or(o, "in_channels", 0) / g,
                  k = int_or(o, "out_channels", 0) / g, hi = int_or(o, "in_h", 0), wi = int_or(o, "in_w", 0),
                  y = int_or(o, "fil_h", 0), x = int_or(o, "fil_w", 0);
    const int64_t dh = int_or(o, "dilation_h", 1), dw = int_or(o, "dilation_w", 1), sh = int_or(o, "conv_stride_h", 1),
                  sw = int_or(o, "conv_stride_w", 1);
    const int64_t ph = int_or(o, "padding_h_l", int_or(o, "padding_h", 0)), pw = int_or(o, "padding_w_l", int_or(o, "padding_w", 0));
    const int64_t ph_r = int_or(o, "padding_h_r", int_or(o, "padding_h", 0)), pw_r = int_or(o, "padding_w_r", int_or(o, "padding_w", 0));
    const int64_t ho = (hi + ph + ph_r - (y - 1) * dh - 1) / sh + 1, wo = (wi + pw + pw_r - (x - 1) * dw - 1) / sw + 1;
    auto dims = [](const std::string &layout, const char *letters, const int64_t *sizes) {
      std::vector<int64_t> d;
      for (char ch : layout)
        d.push_back(sizes[std::strchr(letters, ch) - letters]);
      return d;
    };
    const int64_t fsz[5] = {g, k, c, y, x}, isz[5] = {n, g, c, hi, wi}, osz[5] = {n, g, k, ho, wo};
    h->args = {A{tf, dims(fl, "gkcyx", fsz)}, A{ti, dims(il, "ngchw", isz)}, A{to, dims(ol, "ngkhw", osz)},
               A{to == ROCK_I32 ? ROCK_I32 : ROCK_F32, {g * k}}};
    if (str_or(o, "residual", "none") != "none")
      h->args.push_back(A{to, h->args[2].dims});
    with_workspace(g * k);
  }
}

// problem description -> resolved kernel; NULL with the error set on failure
Handle *build_handle(const OptMap &o) {
  // arch: "[triple:]gfxNNN[:features]" (ConvGenerator.cpp:538-552); only
  // gfx950 has kernels here
  std::string arch = str_or(o, "arch", "gfx950");
  if (arch.find("gfx950") == std::string::npos) {
    set_error("only gfx950 is supported (got '" + arch + "')");
    return nullptr;
  }
  // Flags of rocmlir-gen that change what a kernel computes and that no kernel here implements are refused
  // rather than ignored (its scheduling and instruction-set toggles -- reverse_grid, mfma, wmma, dot, x2 -- are
  // ignored: they leave the results alone): an accumulating store (rocmlir-gen.cpp:295-331; pass the tensor
  // as "-residual add" instead), and the non-OCP 8-bit float encodings (rocmlir-gen.cpp:772-785; gfx950's
  // matrix cores take e4m3fn / e5m2).
  {
    const std::string store = str_or(o, "store-method", str_or(o, "store_method", "set"));
    if (store != "set") {
      set_error("store-method '" + store + "' is not built: outputs are overwritten (an addend goes in as -residual add)");
      return nullptr;
    }
    const std::string f8 = str_or(o, "force-f8-types", str_or(o, "force_f8_types", "arch"));
    if (f8 != "arch" && f8 != "ocp") {
      set_error("force-f8-types '" + f8 + "': only the OCP encodings (e4m3fn, e5m2) have kernels on gfx950");
      return nullptr;
    }
  }
  std::string op = str_or(o, "operation", "");
  const int chan = channel_vector_flags(o);
  if (chan && !(op == "gemm" || ((op == "conv" || op == "conv2d") && !o.count("in_d") && !o.count("fil_d")))) {
    set_error("per-channel quantisation vectors: GEMM and forward 2-D convolution only");
    return nullptr;
  }
  Handle *h = nullptr;
  try {
    if (op == "gemm")
      h = make_gemm(o);
    else if (op == "attention")
      h = make_attention(o);
    else if (op == "conv" || op == "conv2d" || op == "conv_bwd_data" || op == "conv2d_bwd_data" ||
             op == "conv_bwd_weight" || op == "conv2d_bwd_weight")
      h = make_conv(o);
    else
      set_error("unknown --operation '" + op + "'");
  } catch (...) {
    set_error("internal error while building the problem");
    h = nullptr;
  }
  if (!h)
    return nullptr;
  h->kernel_id = (int)int_or(o, "kernel_id", 0);
  if (h->kernel_id < 0 || h->kernel_id >= h->kernel_count) {
    set_error("kernel_id out of range");
    delete h;
    return nullptr;
  }
  h->num_cu = (int)int_or(o, "num_cu", kNumCU);
  if (chan) {
    // The vectors are further caller tensors between the problem's own and the workspace (which closes
    // every multi-kernel problem's list): every kernel of the plan sees the longer list, and the
    // contraction kernel finds the vectors through pointer fields of its parameter block.
    int nvec = 0;
    for (int bit : {ROCK_CHAN_SCALE, ROCK_CHAN_ZP, ROCK_CHAN_QUANT_SCALE, ROCK_CHAN_OUT_ZP})
      nvec += (chan & bit) ? 1 : 0;
    const int base = h->caller_pointers ? h->caller_pointers : h->num_pointers;
    const int first = h->workspace_bytes ? base - 1 : base;
    if (h->ptr_map.empty())
      for (int i = 0; i < h->num_pointers; ++i)
        h->ptr_map.push_back(Handle::PtrSrc{i, 0});
    for (Handle::PtrSrc &m : h->ptr_map)
      if (m.source >= first)
        m.source += nvec;
    h->caller_pointers = base + nvec;
    if (h->epi && h->epi->chan_flags) {
      const int at = (int)((const char *)h->epi - h->params.data());
      int next = first;
      if (chan & ROCK_CHAN_SCALE)
        h->param_ptrs.push_back({at + (int)offsetof(RockEpilogue, scale_vec), next++});
      if (chan & ROCK_CHAN_ZP)
        h->param_ptrs.push_back({at + (int)offsetof(RockEpilogue, zero_point_vec), next++});
      if (chan & ROCK_CHAN_QUANT_SCALE)
        h->param_ptrs.push_back({at + (int)offsetof(RockEpilogue, quant_scale_vec), next++});
      if (chan & ROCK_CHAN_OUT_ZP)
        h->param_ptrs.push_back({at + (int)offsetof(RockEpilogue, out_zero_point_vec), next++});
    }
  }
  if (h->op == OP_CONV && h->params.size() == sizeof(RockConvParams)) {
    // every plan's convolution kernels leave through here: the division constants of the loader's set-up
    auto &cpar = *reinterpret_cast<RockConvParams *>(h->params.data());
    cpar.div_image = fast_div_of(std::max<int64_t>(1, (int64_t)cpar.ho * cpar.wo));
    cpar.div_row = fast_div_of(std::max<int64_t>(1, cpar.wo));
    cpar.div_c = fast_div_of(std::max<int64_t>(1, cpar.c));
    cpar.div_x = fast_div_of(std::max<int64_t>(1, cpar.x));
  }
  h->blob = find_blob(h->kernel_name);
  if (!h->blob) {
    set_error("no code object for " + h->kernel_name);
    delete h;
    return nullptr;
  }
  h->options = o;
  describe_arguments(o, h);
  return h;
}

// The perf_config strings worth trying for a problem: one per distinct kernel
// the problem can run on (a request that does not fit falls back to the
// table's choice and is dropped as a duplicate).  The reference enumerates
// its parameter grid instead (createGemmTuningRangeBF / the quick lists,
// RockTuningImpl.cpp:461-548); here the grid is the handful of hand-written
// tiles.
std::vector<std::string> tuning_candidates(const Handle &h, int kind) {
  std::vector<std::string> requests;
  requests.push_back(""); // the table's own choice comes first
  if (h.op == OP_ATTENTION) {
    for (int dmax : {64, 128})
      for (const AttnVariant &v : kAttnVariants)
        requests.push_back(attn_perf_string(v, dmax));
  } else {
    for (const Tile &t : kFastTiles)
      requests.push_back(perf_string(t, 1));
    requests.push_back("v2:32,32,4,32,32,16,4,1,1");    // K split over the block's waves (GEMM)
    requests.push_back("v2:224,128,8,224,32,16,1,1,1"); // window-resident convolution
    if (kind == ROCKAMD_TUNING_EXHAUSTIVE) {
      // every tile once more as its twin with the rolled epilogue (forceUnroll 0)
      for (const Tile &t : kFastTiles) {
        std::string pc = perf_string(t, 1);
        pc[pc.size() - 3] = '0';
        requests.push_back(pc);
      }
    }
  }
  std::vector<std::string> out, seen;
  const std::string keep_error = g_last_error;
  for (const std::string &r : requests) {
    OptMap o = h.options;
    o.erase("perf_config");
    if (!r.empty())
      o["perf_config"] = r;
    // the contraction kernel of the plan the request leads to (conversion kernels may run in front of it)
    o.erase("kernel_id");
    Handle *c = build_handle(o);
    for (int id = 1; c && c->op == OP_RELAYOUT && id < c->kernel_count; ++id) {
      const int count = c->kernel_count;
      delete c;
      o["kernel_id"] = std::to_string(id);
      c = build_handle(o);
      if (c && c->kernel_count != count) {
        delete c;
        c = nullptr;
      }
    }
    if (!c)
      continue;
    // one entry per distinct plan: a reduction split over blocks runs the same kernel as the unsplit plan
    const std::string plan = c->kernel_name + "/" + std::to_string(c->kernel_count);
    if (std::find(seen.begin(), seen.end(), plan) == seen.end()) {
      seen.push_back(plan);
      out.push_back(c->perf_config);
    }
    delete c;
  }
  g_last_error = keep_error;
  // Quick: the table's choice and its two nearest alternatives in the order
  // above (largest tiles first), as the reference's quick lists hold a handful
  // of likely winners (RockTuningImpl.cpp:401-459)
  if (kind == ROCKAMD_TUNING_QUICK && out.size() > 3)
    out.resize(3);
  return out;
}

struct TuningSpace {
  std::vector<std::string> params;
};

// problem key -> best perf_config seen and its time (mlirRockTuningUpdateTable keeps only the best)
struct TuningTable {
  std::map<std::string, std::pair<std::string, float>> best;
  std::mutex mutex; // several tuning threads may share one table (RockTuningImpl.cpp:902-931 takes a RW lock)
};

} // namespace

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
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return (int)e;
  hipModule_t mod;
  {
    std::lock_guard<std::mutex> lock(g_module_mutex);
    auto key = std::make_pair(dev, blob);
    auto it = g_modules.find(key);
    if (it == g_modules.end()) {
      e = hipModuleLoadData(&mod, blob->start);
      if (e != hipSuccess)
        return (int)e;
      g_modules[key] = mod;
    } else {
      mod = it->second;
    }
  }
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
