// Convolutions over three spatial dimensions, forward and both gradients, on the 2-D plans.
#include "rock_host.h"

namespace rockhost {

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
    if (backward && P.pl[a] != P.pr[a]) { // (see make_conv: refused until the 2-D case has been cleared on a GPU)
      set_error("conv: the backward kernels take symmetric padding only");
      return false;
    }
  }
  if (P.n <= 0 || P.g <= 0 || P.ct <= 0 || P.kt <= 0 || P.ct % P.g != 0 || P.kt % P.g != 0) {
    set_error("conv: tensor dimensions must be positive and channels divisible by groups");
    return false;
  }
  if (!RoutePolicy(o).layout_conversion) {
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
  inner.ph_r = P.pr[0]; inner.pw_r = P.pr[1];
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

} // namespace rockhost
