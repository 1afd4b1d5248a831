// GEMM problems: tile choice, kernel and grid, padded copies of ragged operands, the reduction split over
// blocks (GridwiseGemmParams.cpp:91-103; RockTuningImpl.cpp:962-1008).
#include "rock_host.h"

namespace rockhost {

// pick the tile that minimises rounds * tile_area / efficiency
// `k_major`: the problem has a K-major operand; those kernels exist for the square tiles only
const Tile *pick_tile(int64_t M, int64_t N, int G, bool conv, const std::string &force, bool k_major) {
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
bool plan_gemm_kernel(Handle *h, RockGemmParams &p, int code, int es, const OptMap &o, bool k_padded) {
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
  if (!vector_kernel && RoutePolicy(o).layout_conversion) {
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
    if (G == 1 && is_float_in(ta) && is_float_in(tb) && identity && tiled && RoutePolicy(o).split_k) {
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

} // namespace rockhost
