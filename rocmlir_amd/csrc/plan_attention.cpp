// Attention problems: the fused kernels and their perf_config strings, conversion kernels around them, and
// the GEMM / row softmax / GEMM form (GridwiseGemmToBlockwise.cpp:1607-2403; rocmlir-gen.cpp:2149-2200).
#include "rock_host.h"

namespace rockhost {

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

// "-attn_elementwise x,t0,mul,exp,t1,add" with "-attn_inputs f32,f32": the pre-softmax region of rock.attention
// as postfix code (RockOps.td:208-254: any element-wise tree over the scores and further [G, seq_q, seq_k]
// tensors; mixr-attention-padded-scale-bias-exp.mlir and ...-complex-tree-elemwise.mlir are two).  Tokens: x (the
// score), t<i> (input tensor i), c:<number>, add sub mul div max min (a b -> a op b), exp neg tanh sigmoid relu
// abs erf, where (c a b -> c != 0 ? a : b).  Such a problem runs as GEMM, row softmax (which interprets the
// program), GEMM; the fixed chain -with-attn-scale / -scale / -with-attn-bias / -with-attn-mask stays on the
// fused kernels.
struct AttnProgram {
  std::vector<int32_t> code;
  std::vector<float> consts;
  std::vector<int> input_types; // RockDType per input tensor
};

bool parse_attention_program(const OptMap &o, int default_type, AttnProgram &prog) {
  const std::string text = str_or(o, "attn_elementwise", "");
  if (text.empty())
    return true;
  auto split = [](const std::string &t) {
    std::vector<std::string> out;
    std::string cur;
    for (char ch : t) {
      if (ch == ',') {
        out.push_back(cur);
        cur.clear();
      } else {
        cur += ch;
      }
    }
    out.push_back(cur);
    return out;
  };
  static const std::pair<const char *, int> kOps[] = {
      {"add", ROCK_AOP_ADD}, {"sub", ROCK_AOP_SUB}, {"mul", ROCK_AOP_MUL}, {"div", ROCK_AOP_DIV},
      {"max", ROCK_AOP_MAX}, {"min", ROCK_AOP_MIN}, {"exp", ROCK_AOP_EXP}, {"neg", ROCK_AOP_NEG},
      {"tanh", ROCK_AOP_TANH}, {"sigmoid", ROCK_AOP_SIGMOID}, {"relu", ROCK_AOP_RELU}, {"abs", ROCK_AOP_ABS},
      {"erf", ROCK_AOP_ERF}, {"where", ROCK_AOP_WHERE}};
  int depth = 0, inputs_used = 0;
  for (const std::string &tok : split(text)) {
    int op = 0, arg = 0;
    if (tok == "x") {
      op = ROCK_AOP_SCORE;
    } else if (tok.size() >= 2 && tok[0] == 't' && std::isdigit((unsigned char)tok[1])) {
      op = ROCK_AOP_TENSOR;
      arg = std::atoi(tok.c_str() + 1);
      if (arg >= ROCK_ATTN_PROGRAM_INPUTS) {
        set_error("attention: at most 8 pre-softmax input tensors");
        return false;
      }
      inputs_used = std::max(inputs_used, arg + 1);
    } else if (tok.rfind("c:", 0) == 0) {
      char *end = nullptr;
      const float v = std::strtof(tok.c_str() + 2, &end);
      if (end == tok.c_str() + 2 || *end || prog.consts.size() == ROCK_ATTN_PROGRAM_INPUTS) {
        set_error("attention: bad or too many constants in the pre-softmax program ('" + tok + "')");
        return false;
      }
      op = ROCK_AOP_CONST;
      arg = (int)prog.consts.size();
      prog.consts.push_back(v);
    } else {
      for (const auto &k : kOps)
        if (tok == k.first)
          op = k.second;
      if (!op) {
        set_error("attention: unknown token '" + tok + "' in the pre-softmax program");
        return false;
      }
    }
    const int pops = op <= ROCK_AOP_CONST ? 0 : op < ROCK_AOP_EXP ? 2 : op < ROCK_AOP_WHERE ? 1 : 3;
    if (depth < pops) {
      set_error("attention: the pre-softmax program pops an empty stack at '" + tok + "'");
      return false;
    }
    depth += 1 - pops;
    if (depth > 4 || prog.code.size() == ROCK_ATTN_PROGRAM_MAX) {
      set_error("attention: the pre-softmax program is longer than 24 steps or deeper than 4 values");
      return false;
    }
    prog.code.push_back(op | (arg << 8));
  }
  if (depth != 1) {
    set_error("attention: the pre-softmax program must leave exactly one value");
    return false;
  }
  const std::string types = str_or(o, "attn_inputs", "");
  if (!types.empty())
    for (const std::string &t : split(types)) {
      const int ty = parse_dtype(t);
      if (ty != ROCK_F32 && ty != ROCK_F16 && ty != ROCK_BF16 && ty != ROCK_I8) {
        set_error("attention: pre-softmax input tensors are f32, f16, bf16 or i8 ('" + t + "')");
        return false;
      }
      prog.input_types.push_back(ty);
    }
  if ((int)prog.input_types.size() < inputs_used) {
    if (!types.empty()) {
      set_error("attention: the pre-softmax program reads more tensors than -attn_inputs lists");
      return false;
    }
    prog.input_types.assign(inputs_used, default_type);
  }
  if (bool_or(o, "with-attn-scale", false) || bool_or(o, "with-attn-bias", false) || bool_or(o, "with-attn-mask", false)) {
    set_error("attention: -attn_elementwise replaces -with-attn-scale / -with-attn-bias / -with-attn-mask");
    return false;
  }
  float scale = 1.0f;
  if (get_float(o, "scale", scale) && scale != 1.0f) {
    set_error("attention: with -attn_elementwise the scale is a constant of the program (c:<value>), not -scale");
    return false;
  }
  return true;
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
                               bool tQ, bool tK, bool tV, bool tO, bool has_bias, bool has_scale_t, bool has_mask,
                               const AttnProgram &prog = AttnProgram()) {
  // "-t i8": Q and K are int8, their product is dequantised before the softmax
  // ((acc - zero_point) * scale, the scalars rocmlir-gen passes as [1,1,1]
  // tensors, rocmlir-gen.cpp:2173-2184, 2353-2367); V, the pre-softmax tensors
  // and O are f16
  const int tq = ty;
  if (ty == ROCK_I8)
    ty = ROCK_F16;
  const int es = dtype_size(ty);
  // A row of scores is sk f32 values in a pitch of whole 16-byte chunks; P replaces it in place, its tail up to
  // the next chunk written as zeros by the softmax kernel, so that the second GEMM reads P on its vector path
  // whatever sk is.
  const int64_t skp = (sk + 3) / 4 * 4;
  // chunk = gc groups x rc query rows
  // ("-score_workspace_limit BYTES" moves the bound, e.g. to keep one chunk inside a smaller cache share)
  const RoutePolicy route(o);
  const int64_t dflt = G * sq * skp * 4 <= kScoreWholeBytes ? kScoreWholeBytes : kScoreChunkBytes;
  const int64_t limit = std::max<int64_t>(route.score_workspace_limit > 0 ? route.score_workspace_limit : dflt, skp * 4);
  int64_t gc = G, rc = sq;
  if (G * sq * skp * 4 > limit) {
    if (sq * skp * 4 <= limit) {
      gc = limit / (sq * skp * 4);
    } else {
      gc = 1;
      rc = std::max<int64_t>(1, limit / (skp * 4));
      rc = rc >= 128 ? rc / 128 * 128 : rc >= 8 ? rc / 8 * 8 : rc; // chunk boundaries on whole tiles / 16-byte columns
    }
  }
  const int64_t row_chunks = ceil_div(sq, rc), chunks = ceil_div(G, gc) * row_chunks;
  // the second GEMM of a one-group chunk: its reduction over the keys in S shares (as make_gemm splits a GEMM)
  int64_t S = 1;
  if (gc == 1 && route.split_k) {
    const int64_t tiles64 = (int64_t)ceil_div(rc, 64) * ceil_div(dv, 64);
    if (sk >= 2048 && tiles64 * 2 <= kNumCU)
      for (int64_t d = std::min<int64_t>(2 * kNumCU / tiles64, sk / 512); d >= 2 && S == 1; --d)
        if (sk % d == 0 && (sk / d * es) % 64 == 0)
          S = d;
  }
  const int per_chunk = S > 1 ? 4 : 3;
  const int64_t score_bytes = align256(gc * rc * skp * 4), partial_bytes = S > 1 ? align256(S * rc * dv * 4) : 0;
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
  // caller list: Q, K, V, [scale tensor], bias slot, [mask, other], O, workspace;
  // with a pre-softmax program: Q, K, V, the program's input tensors, O, workspace
  const bool programmed = !prog.code.empty();
  const int n_in = (int)prog.input_types.size();
  const int i_bias = has_scale_t ? 4 : 3, i_mask = has_mask ? i_bias + 1 : -1, i_other = has_mask ? i_bias + 2 : -1,
            i_out = programmed ? 3 + n_in : i_bias + 1 + (has_mask ? 2 : 0), i_ws = i_out + 1;
  const int64_t pitch_p = 4 / es; // elements of P per f32 score: P lies in place, rows skp * 4 bytes apart
  auto *h = new Handle;
  if (kid == 1) {
    RockSoftmaxParams r;
    std::memset(&r, 0, sizeof r);
    r.row_pitch = skp;
    r.seq_k_padded = (int)((sk * es + 15) / 16 * 16 / es);
    r.t_gs = sq * sk; r.t_is = sk; r.t_js = 1;
    r.G = (int)gn; r.seq_q = (int)rn; r.seq_k = (int)sk;
    r.scale = scale;
    r.has_bias = has_bias ? 1 : 0;
    r.has_scale_tensor = has_scale_t ? 1 : 0;
    r.has_mask = has_mask ? 1 : 0;
    r.dtype = ty;
    r.prog_len = (int)prog.code.size();
    std::copy(prog.code.begin(), prog.code.end(), r.prog);
    std::copy(prog.consts.begin(), prog.consts.end(), r.consts);
    std::copy(prog.input_types.begin(), prog.input_types.end(), r.tensor_dtype);
    r.t_base = g0 * sq * sk + r0 * sk; // the chunk's first row in the program's [G, seq_q, seq_k] tensors
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
    if (programmed) {
      h->ptr_map = {{i_ws, 0}, {-1, 0}, {-1, 0}, {-1, 0}, {-1, 0}};
      for (int i = 0; i < n_in; ++i) // their pointers ride in the parameter block
        h->param_ptrs.push_back({(int)(offsetof(RockSoftmaxParams, tensors) + i * sizeof(void *)), 3 + i});
    } else {
      h->ptr_map = {{i_ws, 0}, {has_scale_t ? 3 : -1, t_off}, {has_bias ? i_bias : -1, t_off}, {i_mask, t_off / es},
                    {i_other, t_off}};
    }
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
      gp.c_gs = rn * skp; gp.c_ms = skp; gp.c_ns = 1;
      a_off = (g0 * gp.a_gs + r0 * gp.a_ms) * dtype_size(tq);
      b_off = g0 * gp.b_gs * dtype_size(tq);
      c_off = 0;
      default_epilogue(gp.epi, ROCK_F32);
      gp.epi.zero_point = (int32_t)int_or(o, "zero_point", 0); // i8: scores leave as float(acc) - zero_point
    } else { // O[g,i,e] = sum_j P[g,i,j] V[g,j,e]
      gp.M = (int)rn; gp.N = (int)dv; gp.K = (int)sk;
      gp.a_gs = rn * skp * pitch_p; gp.a_ms = skp * pitch_p; gp.a_ks = 1;
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
    plan_gemm_kernel(h, gp, operand_code(tg, tg), dtype_size(tg), o, /*k_padded=*/kid == 2);
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
  h->workspace_bytes = (size_t)(partial_bytes ? score_bytes + partial_bytes : gc * rc * skp * 4);
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
  AttnProgram prog;
  if (!parse_attention_program(o, ty == ROCK_I8 ? ROCK_F16 : ty, prog))
    return nullptr;
  if (!prog.code.empty())
    return make_attention_unfused(o, ty, G, sq, sk, dqk, dv, tQ, tK, tV, tO, false, false, false, prog);
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
  // Head dimensions that are not whole 16-byte chunks (d = 20, 36): the same copies pad every row of Q and K to
  // dqp and of V to dvp elements with zeros, which add nothing to a score; the fused kernel works on the padded
  // problem and the last conversion keeps the dv columns of its result that exist.
  const int64_t unit_qk = qk_i8 ? 16 : 8;
  const int64_t dqp = (dqk + unit_qk - 1) / unit_qk * unit_qk, dvp = (dv + 7) / 8 * 8;
  const bool pad_qk = dqp != dqk, pad_v = dvp != dv;
  const bool copy_k = (!tK && (qk_i8 || sk % 8 != 0)) || pad_qk;
  const bool copy_q = tQ || pad_qk, copy_v = tV || pad_v, copy_o = tO || pad_v;
  if ((copy_q || copy_v || copy_o || copy_k) && ty != ROCK_F32 && RoutePolicy(o).layout_conversion) {
    OptMap inner = o;
    inner["transQ"] = inner["transV"] = inner["transO"] = "false";
    if (copy_k)
      inner["transK"] = "true";
    if (pad_qk)
      inner["head_dim_qk"] = std::to_string(dqp);
    if (pad_v)
      inner["head_dim_v"] = std::to_string(dvp);
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
      const int64_t q_bytes = copy_q ? align256(G * sq * dqp * es_q) : 0, v_bytes = copy_v ? align256(G * sk * dvp * 2) : 0,
                    o_bytes = copy_o ? align256(G * sq * dvp * 2) : 0, k_bytes = copy_k ? align256(G * sk * dqp * es_q) : 0;
      const int64_t q_off = 0, v_off = q_bytes, o_off = q_bytes + v_bytes, k_off = o_off + o_bytes;
      // caller pointers: Q, K, V, [scale tensor,] bias, [mask, other,] O, workspace
      const int i_scale = has_scale_t ? 3 : -1, i_bias = has_scale_t ? 4 : 3, i_mask = has_mask ? i_bias + 1 : -1,
                i_other = has_mask ? i_bias + 2 : -1, i_out = i_bias + 1 + (has_mask ? 2 : 0), i_ws = i_out + 1;
      std::vector<int> kinds; // 0 = Q copy, 1 = V copy, 4 = K copy, 2 = the fused kernel, 3 = O written in the caller's layout
      if (copy_q) kinds.push_back(0);
      if (copy_v) kinds.push_back(1);
      if (copy_k) kinds.push_back(4);
      kinds.push_back(2);
      if (copy_o) kinds.push_back(3);
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
        // (source strides in the order of the destination's dimensions; rows padded with zeros up to dqp / dvp)
        if (kinds[kid] == 0) { // [G, d, seq_q] or [G, seq_q, d] -> [G, seq_q, dqp]
          const int64_t size[5] = {1, 1, G, sq, dqp}, src_size[5] = {1, 1, G, sq, dqk};
          const int64_t stride[5] = {0, 0, sq * dqk, tQ ? 1 : dqk, tQ ? sq : 1};
          ok = fill_relayout_handle(h, size, src_size, stride, es_q);
          h->ptr_map = {{0, 0}, {i_ws, q_off}};
          h->problem_key = "relayout attention Q";
        } else if (kinds[kid] == 1) { // [G, dv, seq_k] or [G, seq_k, dv] -> [G, seq_k, dvp]
          const int64_t size[5] = {1, 1, G, sk, dvp}, src_size[5] = {1, 1, G, sk, dv};
          const int64_t stride[5] = {0, 0, sk * dv, tV ? 1 : dv, tV ? sk : 1};
          ok = fill_relayout_handle(h, size, src_size, stride, 2);
          h->ptr_map = {{2, 0}, {i_ws, v_off}};
          h->problem_key = "relayout attention V";
        } else if (kinds[kid] == 4) { // [G, d, seq_k] or [G, seq_k, d] -> [G, seq_k, dqp]
          const int64_t size[5] = {1, 1, G, sk, dqp}, src_size[5] = {1, 1, G, sk, dqk};
          const int64_t stride[5] = {0, 0, sk * dqk, tK ? dqk : 1, tK ? 1 : sk};
          ok = fill_relayout_handle(h, size, src_size, stride, es_q);
          h->ptr_map = {{1, 0}, {i_ws, k_off}};
          h->problem_key = "relayout attention K";
        } else if (tO) { // [G, seq_q, dvp] -> [G, dv, seq_q]
          const int64_t size[5] = {1, 1, G, dv, sq}, stride[5] = {0, 0, sq * dvp, 1, dvp};
          ok = fill_relayout_handle(h, size, size, stride, 2);
          h->ptr_map = {{i_ws, o_off}, {i_out, 0}};
          h->problem_key = "relayout attention O";
        } else { // [G, seq_q, dvp] -> [G, seq_q, dv]
          const int64_t size[5] = {1, 1, G, sq, dv}, stride[5] = {0, 0, sq * dvp, dvp, 1};
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
        h->ptr_map = {copy_q ? Handle::PtrSrc{i_ws, q_off} : Handle::PtrSrc{0, 0},
                      copy_k ? Handle::PtrSrc{i_ws, k_off} : Handle::PtrSrc{1, 0},
                      copy_v ? Handle::PtrSrc{i_ws, v_off} : Handle::PtrSrc{2, 0}, {i_scale, 0}, {i_bias, 0},
                      {i_mask, 0}, {i_other, 0},
                      copy_o ? Handle::PtrSrc{i_ws, o_off} : Handle::PtrSrc{i_out, 0}};
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
                          RoutePolicy(o).fused;
    // 16-bit types up to 256 on the vector kernel (head-dimension-contiguous tensors, checked below)
    // (K either way: [seq_k, d], or the reference's default [d, seq_k] with whole 16-byte rows of keys)
    const bool wide_ok = !qk_i8 && !tQ && (tK || sk % 8 == 0) && !tV && !tO && dqk % 8 == 0 && dv % 8 == 0 &&
                         RoutePolicy(o).fused;
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

} // namespace rockhost
