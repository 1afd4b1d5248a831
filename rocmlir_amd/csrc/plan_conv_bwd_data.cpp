// Gradient of a convolution with respect to its input.
#include "rock_host.h"

namespace rockhost {

// ---- backward convolutions ------------------------------------------------------
// Both gradients are forward convolutions over re-labelled views of the
// problem's tensors, so they run on the forward kernels; what the views cannot
// express directly (channel-contiguous operands for the vector kernels,
// flipped filters, a reduction split over blocks) goes through the utility
// kernels and the multi-kernel protocol.  The reference lowers them through
// its own gridwise GEMM with dedicated coordinate transforms
// (ConvToGemm.cpp:530-1131) plus zero-init / converting-copy utility kernels
// (ConvGenerator.cpp:279-344, 434-480).

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
  if (cp.y == 1 && cp.x == 1 && cp.sh == 1 && cp.sw == 1 && cp.unpadded() && cp.g == 1 &&
      cp.hi * cp.wi <= INT32_MAX && cp.n * cp.hi * cp.wi <= INT32_MAX && RoutePolicy(o).pointwise_as_gemm &&
      RoutePolicy(o).layout_conversion) {
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
  bool fast = RoutePolicy(o).layout_conversion;
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
      RoutePolicy(o).merge_phases) {
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
  if (fast && phases.size() == 1 && !win[0].ok && cp.g == 1 && RoutePolicy(o).split_k) {
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

} // namespace rockhost
