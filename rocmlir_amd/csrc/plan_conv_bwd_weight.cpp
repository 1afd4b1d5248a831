// Gradient of a convolution with respect to its filter.
#include "rock_host.h"

namespace rockhost {

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
  applies = (!cl_in || !cl_out) && (cp.c * es) % 16 == 0 && (cp.k * es) % 16 == 0 && RoutePolicy(o).layout_conversion;
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
        RoutePolicy(o).bwd_weight_gemm && RoutePolicy(o).layout_conversion))
    return nullptr;
  int64_t cpad = 1;
  while (cpad < cp.c)
    cpad *= 2;
  const int64_t pix_bytes = cpad * es;
  if ((cp.c * es) % 16 == 0 || pix_bytes > 16 || cp.pw != 0 || cp.pw_r != 0 || cp.dw != 1 || (cp.sw * pix_bytes) % 16 != 0 ||
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
  if (cp.y == 1 && cp.x == 1 && cp.unpadded() && (cp.sh > 1 || cp.sw > 1) &&
      RoutePolicy(o).layout_conversion && RoutePolicy(o).pointwise_as_gemm) {
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
      (cp.ti == ROCK_F32 || cp.ti == ROCK_F16 || cp.ti == ROCK_BF16) && RoutePolicy(o).bwd_weight_gemm &&
      RoutePolicy(o).layout_conversion) {
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
    if (cp.y == 1 && cp.x == 1 && cp.sh == 1 && cp.sw == 1 && cp.unpadded() && cp.g == 1 && lin_x && lin_y &&
        RoutePolicy(o).pointwise_as_gemm) {
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
      RoutePolicy(o).bwd_weight_gemm) {
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
  const bool fast = RoutePolicy(o).layout_conversion && conv_view_fast(f, es) &&
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

} // namespace rockhost
