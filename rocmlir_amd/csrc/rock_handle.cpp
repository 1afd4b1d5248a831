// From an option string to a handle: dispatch to the planners, the caller's argument list described, the
// tuning space of a problem (rocmlir-lib.cpp:117-199; RockTuningImpl.cpp:401-548).
#include "rock_host.h"

namespace rockhost {

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
    if (!str_or(o, "attn_elementwise", "").empty()) {
      // the program's input tensors (their number: what the plan put into the caller's list between V and O)
      const int total = h->caller_pointers ? h->caller_pointers : h->num_pointers;
      const int n_in = total - 5; // Q, K, V, O, workspace
      std::vector<int> types;
      std::string cur;
      for (char ch : str_or(o, "attn_inputs", "") + ",") {
        if (ch == ',') {
          if (!cur.empty())
            types.push_back(parse_dtype(cur));
          cur.clear();
        } else {
          cur += ch;
        }
      }
      for (int i = 0; i < n_in; ++i)
        h->args.push_back(A{i < (int)types.size() ? types[i] : tv, {G, sq, sk}});
    } else {
      if (bool_or(o, "with-attn-scale", false))
        h->args.push_back(A{tv, {G, sq, sk}});
      h->args.push_back(A{tv, {G, sq, sk}}); // bias slot
      if (bool_or(o, "with-attn-mask", false)) {
        h->args.push_back(A{ROCK_I8, {G, sq, sk}});
        h->args.push_back(A{tv, {G, sq, sk}});
      }
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
    auto without_depth = [&](const char *key) { // a third spatial letter of extent one (make_conv)
      std::string s = str_or(o, key, "");
      s.erase(std::remove(s.begin(), s.end(), '2'), s.end());
      return s;
    };
    if (!canon_layout(without_depth("fil_layout"), 'k', "gkcyx", fl) || !canon_layout(without_depth("in_layout"), 'c', "ngchw", il) ||
        !canon_layout(without_depth("out_layout"), 'k', "ngkhw", ol))
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
Handle *build_handle(const OptMap &given) {
  OptMap planned = given;
  const OptMap &o = planned;
  // "-p": rocmlir-gen's default problem of each operation, assigned over whatever the string gave for these keys
  // (populateDefaults, rocmlir-gen.cpp:996-1069; its regression lists name most problems "-p" and nothing else)
  if (bool_or(given, "p", false)) {
    const std::string op = str_or(given, "operation", "");
    auto set = [&](std::initializer_list<std::pair<const char *, int>> values) {
      for (const auto &kv : values)
        planned[kv.first] = std::to_string(kv.second);
    };
    if (op == "gemm") {
      set({{"g", 1}, {"m", 1024}, {"k", 769}, {"n", 512}});
    } else if (op == "attention") {
      set({{"g", 1}, {"seq_len_q", 1024}, {"seq_len_k", 1024}, {"head_dim_qk", 32}, {"head_dim_v", 32}});
    } else {
      const bool big = str_or(given, "mfma", "infer") == "on"; // the 1x1 problem rocmlir-gen takes when MFMA is forced on
      set({{"groupsize", 1}, {"batchsize", 128}, {"in_channels", big ? 1024 : 8}, {"out_channels", big ? 1024 : 128},
           {"in_h", big ? 14 : 32}, {"in_w", big ? 14 : 32}, {"fil_h", big ? 1 : 3}, {"fil_w", big ? 1 : 3},
           {"dilation_h", 1}, {"dilation_w", 1}, {"conv_stride_h", 1}, {"conv_stride_w", 1}, {"padding_h", 0},
           {"padding_w", 0}});
      for (const char *k : {"padding_h_l", "padding_h_r", "padding_w_l", "padding_w_r", "out_h", "out_w", "in_d", "fil_d",
                            "out_d", "padding_d", "padding_d_l", "padding_d_r", "dilation_d", "conv_stride_d"})
        planned.erase(k);
    }
  }
  // arch: "[triple:]gfxNNN[:features]" (ConvGenerator.cpp:538-552); only
  // gfx950 has kernels here
  std::string arch = str_or(o, "arch", "gfx950");
  if (arch.find("gfx950") == std::string::npos) {
    set_error("only gfx950 is supported (got '" + arch + "')");
    return nullptr;
  }
  // Flags of rocmlir-gen that change what a kernel computes and that no kernel here implements are refused
  // rather than ignored (its scheduling and instruction-set toggles -- reverse_grid, mfma, wmma, dot, x2 -- are
  // ignored: they leave the results alone): the non-OCP 8-bit float encodings (rocmlir-gen.cpp:772-785;
  // gfx950's matrix cores take e4m3fn / e5m2).
  // "-store-method atomic_add" (rocmlir-gen.cpp:295-331: C += A B, what the reference's split-K kernels do to a
  // pre-filled C, RockOps.td:136-181) is the residual epilogue with C itself as the addend: the problem is
  // planned with "-residual add" and the residual's place in every kernel's pointer map is then given to the
  // output, so the caller's list stays A, B, C, bias.  Every element is read by the thread (direct stores) or
  // the wave (staged stores) that afterwards writes it, so reading and writing one tensor is safe; the sum is
  // formed in f32 and rounded once, where an atomic add of a 16-bit partial result rounds twice.
  bool accumulate = false;
  {
    const std::string store = str_or(o, "store-method", str_or(o, "store_method", "set"));
    if (store == "atomic_add") {
      if (str_or(o, "operation", "") != "gemm" || str_or(o, "residual", "none") != "none") {
        set_error("store-method atomic_add: GEMM problems without a residual tensor (C itself is the addend)");
        return nullptr;
      }
      accumulate = true;
      planned["residual"] = "add";
    } else if (store != "set") {
      set_error("store-method '" + store + "': set and atomic_add are the two there are");
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
  if (accumulate) {
    // caller list as planned: A, B, C, bias, residual, [workspace]; the residual goes, C stands in for it
    const int base = h->caller_pointers ? h->caller_pointers : h->num_pointers;
    if (h->ptr_map.empty())
      for (int i = 0; i < h->num_pointers; ++i)
        h->ptr_map.push_back(Handle::PtrSrc{i, 0});
    for (Handle::PtrSrc &m : h->ptr_map)
      m.source = m.source == 4 ? 2 : m.source > 4 ? m.source - 1 : m.source;
    h->caller_pointers = base - 1;
  }
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
  h->options = given;
  if (accumulate)
    planned.erase("residual"); // C stands in for it: no such tensor in the caller's list
  describe_arguments(planned, h);
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

} // namespace rockhost
