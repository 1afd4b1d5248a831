// Forward convolution: layouts, the implicit-GEMM view, the window-resident plan, rows of taps, layout
// conversions and the reduction split (ConvGenerator.cpp:487-749; ConvToGemm.cpp:530-1131).
#include "rock_host.h"

namespace rockhost {

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
  // An output whose pixels are contiguous per channel (NCHW style) leaves the kernel as 16-byte vectors of
  // consecutive pixels only when every tile starts on such a vector, element by element otherwise: tiles of whole
  // vectors first, any tile if there is none.
  const int64_t out_es = std::max(1, dtype_size(p.epi.out_dtype));
  const bool pixels_contiguous = p.out_ws == 1 && p.out_ks != 1;
  for (int pass = 0; pass < 2 && w.rows == 0; ++pass)
    for (int64_t rows = std::min<int64_t>(p.ho, p.wo > 0 ? tile_px / p.wo : 0); rows >= 1; --rows) {
      if (window_rows(rows) * row_pitch > kDirectWindowBytes)
        continue;
      if (pass == 0 && pixels_contiguous && (rows * p.wo * out_es) % 16 != 0)
        continue;
      if (w.rows == 0 || ceil_div(tiles_of(rows), per_round) < ceil_div(tiles_of(w.rows), per_round))
        w.rows = rows;
    }
  w.ok = p.stride_h == 1 && p.stride_w == 1 && p.dil_h == 1 && p.dil_w == 1 && p.y * p.x > 1 && equal_padding &&
         p.k % 32 == 0 && cbytes >= 128 && cbytes <= 1024 && (cbytes & (cbytes - 1)) == 0 && w.rows >= 1 &&
         row_pitch <= 32 * 1024 && p.in_cs == 1;
  // by itself: 16-bit types and int8 (measured: 1.13-1.3x), tiles at least 85 % full in pixels and 75 % in
  // channels, enough of them for every CU, no tile requested
  w.by_itself = w.ok && RoutePolicy(o).window_resident && (ti == ROCK_F16 || ti == ROCK_BF16 || ti == ROCK_I8) &&
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
  // Layouts that name a third spatial dimension ("kc012 / nc012 / nk012" in the reference's regression lists)
  // for a problem that gives none: its extent is 1 (rocmlir-gen's defaults for -in_d, -fil_d), and a unit
  // dimension may be dropped from a dense tensor wherever it stands.
  auto without_depth = [&](const char *key) {
    std::string s = str_or(o, key, "");
    s.erase(std::remove(s.begin(), s.end(), '2'), s.end());
    return s;
  };
  if (!canon_layout(without_depth("fil_layout"), 'k', "gkcyx", fl) ||
      !canon_layout(without_depth("in_layout"), 'c', "ngchw", il) ||
      !canon_layout(without_depth("out_layout"), 'k', "ngkhw", ol)) {
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
    // Unequal top / bottom or left / right padding: the gradients' plans carry the right-hand padding through
    // (it only sets the output's extent, ConvProblem::ph_r / pw_r) and replay correctly on the CPU, but the one
    // GPU run that included such problems (the reference's conv_regression_bwd list: in 4x4, filter 2x2, stride 2,
    // padding 2 / 1 and 2 / 0) ended in a memory fault whose cause has not been shown; until it is, they are refused.
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
    cp.ph_r = ph_r; cp.pw_r = pw_r;
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
    if (g == 1 && identity && Mg * k <= INT32_MAX && RoutePolicy(o).split_k) {
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
      RoutePolicy(o).pointwise_as_gemm) {
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
      RoutePolicy(o).layout_conversion && RoutePolicy(o).tap_rows) {
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
    if (!fast && cp * y * x <= INT32_MAX && conv_fast(q, cp) && RoutePolicy(o).layout_conversion) {
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

} // namespace rockhost
