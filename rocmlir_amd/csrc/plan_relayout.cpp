// Handles of the layout-conversion, fill and reduction kernels that run around the contractions
// (the reference's utility kernels: ConvGenerator.cpp:279-344, 434-480).
#include "rock_host.h"

namespace rockhost {

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

} // namespace rockhost
