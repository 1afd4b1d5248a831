// Option strings, element types, epilogue options, the perf_config grammar and the table of embedded code
// objects (ConvGenerator.cpp:82-98, 136-248; MIGraphXToTosa.cpp:874-982 for the epilogue's steps).
#include "rock_host.h"

namespace rockhost {

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

RoutePolicy::RoutePolicy(const OptMap &o)
    : layout_conversion(bool_or(o, "layout_conversion", true)), split_k(bool_or(o, "split_k", true)),
      window_resident(bool_or(o, "window_resident", true)), pointwise_as_gemm(bool_or(o, "pointwise_as_gemm", true)),
      merge_phases(bool_or(o, "merge_phases", true)), bwd_weight_gemm(bool_or(o, "bwd_weight_gemm", true)),
      tap_rows(bool_or(o, "tap_rows", true)), fused(bool_or(o, "fused", true)),
      score_workspace_limit(int_or(o, "score_workspace_limit", 0)) {}

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

std::string perf_string(const Tile &t, int es, const OptMap *o) {
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

} // namespace rockhost
