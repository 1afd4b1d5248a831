// Layout conversion of a 5-D tensor (RockRelayoutParams in kernel_params.h):
// what one thread of a 256-thread block does, written over explicit thread and
// block indices and an explicit LDS pointer, in two phases with the block's
// barrier between them.  The kernels in relayout_kernels.hip call it with the
// hardware indices; a host build (RK_DEV defined empty) can step the same code
// through every block and thread of a launch to check its indexing.
#pragma once
#include <stdint.h>
#include "kernel_params.h"

#ifndef RK_DEV
#define RK_DEV __device__ __forceinline__
#endif

namespace rock_relayout {

struct alignas(16) Bytes16 { uint32_t w[4]; };
struct alignas(8) Bytes8 { uint32_t w[2]; };

// Geometry of RELAYOUT_TRANSPOSE_VEC per element width.  A tile holds AREA
// elements, tile_d of them along the destination's contiguous dimension and
// AREA / tile_d along the source's (both powers of two, at least two 16-byte
// vectors long); every thread moves VPT vectors in and VPT vectors out.
template <typename T> struct VecGeom {
  static constexpr int ES = (int)sizeof(T);
  static constexpr int V = 16 / ES;           // elements per 16-byte vector
  static constexpr int G = 4 / ES;            // elements per 32-bit word
  static constexpr int VPT = ES == 1 ? 4 : 2; // vectors per thread and phase
  static constexpr int AREA = 256 * VPT * V;
  static constexpr int MIN_SIDE = 2 * V;
  // An LDS row holds one more vector than the tile is wide (rows that do not
  // start on a 16-byte boundary are read from the boundary below them) plus
  // padding chosen so that rows V apart, which the column gather of one wave
  // reads together, start in different banks.
  static constexpr int PAD = ES == 1 ? 20 : ES == 2 ? 12 : 8;
  static constexpr int LDS_ELEMS = AREA + PAD * (AREA / MIN_SIDE);
};

// Workgroups are handed to the eight XCDs round-robin, each with an L2 of its
// own.  Neighbouring tiles share cache lines whenever tensor rows are not
// whole lines, so every XCD is given one contiguous run of tiles: the second
// touch of a line then hits the L2 that fetched it.
RK_DEV unsigned xcd_contiguous(unsigned block, unsigned nblocks) {
  const unsigned per = nblocks / 8;
  return block < per * 8 ? (block % 8) * per + block / 8 : block;
}

RK_DEV unsigned fast_div(unsigned n, const RockFastDiv &d) {
  return (unsigned)(((uint64_t)n * d.mul) >> d.shift);
}

struct TilePos {
  int org_s, org_d;  // tile origin along src_fast / dst_fast
  int64_t so, dof;   // element offsets of the tile origin in source / destination
  bool outer_in;     // the other three coordinates lie inside the source
};

// blockIdx enumerates tiles fastest over the src_fast tiles, then dst_fast
// tiles, then the remaining three dimensions in index order.
RK_DEV TilePos tile_position(const RockRelayoutParams &p, unsigned b) {
  TilePos t;
  unsigned q = fast_div(b, p.div[0]);
  t.org_s = (int)(b - q * (unsigned)p.tiles_s) << p.ts_shift;
  b = q;
  q = fast_div(b, p.div[1]);
  t.org_d = (int)(b - q * (unsigned)p.tiles_d) << p.td_shift;
  b = q;
  t.so = (int64_t)t.org_s * p.ss_s + (int64_t)t.org_d * p.ss_d;
  t.dof = (int64_t)t.org_s * p.ds_s + (int64_t)t.org_d * p.ds_d;
  t.outer_in = true;
  for (int k = 0; k < 3; ++k) {
    q = fast_div(b, p.div[2 + k]);
    const int i = (int)(b - q * (unsigned)p.outer_size[k]);
    b = q;
    t.outer_in = t.outer_in && i < p.outer_src[k];
    t.so += (int64_t)i * p.outer_ss[k];
    t.dof += (int64_t)i * p.outer_ds[k];
  }
  return t;
}

// RELAYOUT_TRANSPOSE: one block moves a tile of tile_d x (1024 / tile_d)
// elements over (dst_fast, src_fast) through LDS element by element, so that
// the source is read along its contiguous dimension and the destination
// written along its own; tile_d is 32, or 16 or 8 when the destination's
// contiguous dimension is that short.
template <typename T>
RK_DEV void transpose_phase(int phase, const T *src, T *dst, const RockRelayoutParams &p, unsigned block, int tid,
                            T *tile) {
  const int td_shift = p.td_shift, ts_shift = p.ts_shift;
  const int td = 1 << td_shift, ts = 1 << ts_shift;
  const int size_s = p.size_s, size_d = p.size_d;
  const int src_s = p.src_s, src_d = p.src_d; // shorter than the destination when padding
  const TilePos t = tile_position(p, block);
  if (phase == 0) {
    const int64_t ss_s = p.ss_s, ss_d = p.ss_d;
    // consecutive threads walk the source's contiguous dimension
    for (int j = 0; j < 4; ++j) {
      const int idx = j * 256 + tid;
      const int r = idx >> ts_shift, cs = idx & (ts - 1); // along dst_fast, along src_fast
      if (t.org_d + r < size_d && t.org_s + cs < size_s)
        tile[r * (ts + 1) + cs] = (t.outer_in && t.org_d + r < src_d && t.org_s + cs < src_s)
                                      ? src[t.so + (int64_t)r * ss_d + (int64_t)cs * ss_s]
                                      : (T)0;
    }
  } else {
    const int64_t ds_s = p.ds_s, ds_d = p.ds_d;
    // consecutive threads walk the destination's contiguous dimension
    for (int j = 0; j < 4; ++j) {
      const int idx = j * 256 + tid;
      const int cs = idx >> td_shift, r = idx & (td - 1);
      if (t.org_s + cs < size_s && t.org_d + r < size_d)
        dst[t.dof + (int64_t)cs * ds_s + (int64_t)r * ds_d] = tile[r * (ts + 1) + cs];
    }
  }
}

template <typename T> RK_DEV void lds_store16(T *at, const Bytes16 &v) {
  if (sizeof(T) == 1) { // rows are 4-byte aligned
    uint32_t *q = (uint32_t *)at;
    q[0] = v.w[0]; q[1] = v.w[1]; q[2] = v.w[2]; q[3] = v.w[3];
  } else if (sizeof(T) == 2) { // 8-byte aligned
    Bytes8 *q = (Bytes8 *)at;
    q[0] = Bytes8{{v.w[0], v.w[1]}};
    q[1] = Bytes8{{v.w[2], v.w[3]}};
  } else {
    *(Bytes16 *)at = v;
  }
}

// RELAYOUT_TRANSPOSE_VEC: the same transposition with 16-byte accesses.  The
// destination's contiguous dimension has unit stride; the source's need not
// (every other pixel of a row, a flipped filter), and is then read element by
// element, or, for a stride of two over rows that start on 16-byte boundaries,
// with aligned vectors of which every other element is kept.
//
// Reading (unit stride): row r of the tile starts m_r elements past a 16-byte
// boundary.  Its lanes load the aligned vectors from that boundary on (one
// more than the tile is wide when m_r != 0) and store them at the start of LDS
// row r, so LDS column j holds tile column j - m_r; the gather adds m_r back.
// An aligned vector that holds at least one element of the row lies in that
// element's page, so the bytes around the row that come along are readable;
// they belong to neighbouring tiles or rows and are never used.
//
// Writing: a lane gathers V elements of one tile column from V consecutive
// rows and stores them as one vector.  When every m_r is a whole number of
// 32-bit words the gather reads words, each holding G neighbouring columns,
// and writes G vectors from them.
template <typename T>
RK_DEV void transpose_vec_phase(int phase, const T *src, T *dst, const RockRelayoutParams &p, unsigned block,
                                unsigned nblocks, int tid, T *tile) {
  using Geo = VecGeom<T>;
  constexpr int V = Geo::V, G = Geo::G, ES = Geo::ES;
  union Vec {
    T e[V];
    Bytes16 v;
  };
  const int td_shift = p.td_shift, ts_shift = p.ts_shift;
  const int ts = 1 << ts_shift;
  const int pitch = ts + Geo::PAD;
  const int size_s = p.size_s, size_d = p.size_d;
  const int src_s = p.src_s, src_d = p.src_d;
  const TilePos t = tile_position(p, xcd_contiguous(block, nblocks));
  const int64_t ss_s = p.ss_s, ss_d = p.ss_d;
  const bool unit = ss_s == 1;
  // element address of the tile's first element, and what a row adds to it, modulo a vector
  const unsigned a0 = unit ? (unsigned)(((uintptr_t)(src + t.so)) / ES) : 0u;
  const unsigned astep = unit ? (unsigned)ss_d : 0u;
  if (phase == 0) {
    if (!t.outer_in)
      return;
    if (unit) {
      const int lim = src_s - t.org_s < ts ? src_s - t.org_s : ts; // tile columns that hold source elements
      if (lim <= 0)
        return;
      const int vpr_shift = ts_shift - __builtin_ctz((unsigned)V), vpr = 1 << vpr_shift;
      for (int j = 0; j < Geo::VPT; ++j) {
        const int vi = j * 256 + tid;
        const int r = vi >> vpr_shift, k = vi & (vpr - 1);
        if (t.org_d + r >= src_d)
          continue;
        const int m = (int)((a0 + (unsigned)r * astep) & (unsigned)(V - 1));
        const T *g = src + t.so + (int64_t)r * ss_d - m + k * V; // 16-byte aligned
        if (k * V - m < lim)
          lds_store16(&tile[r * pitch + k * V], *(const Bytes16 *)g);
        if (k == vpr - 1 && m != 0 && ts - m < lim)
          lds_store16(&tile[r * pitch + ts], *(const Bytes16 *)(g + V));
      }
    } else if (ss_s == 2 && (((uintptr_t)(src + t.so) / ES) & (unsigned)(V - 1)) == 0 &&
               ((unsigned)ss_d & (unsigned)(V - 1)) == 0) {
      // every other element of rows that start on 16-byte boundaries (every other pixel of an image
      // row): aligned vectors, of which every other element is kept -- V/2 tile columns per vector
      const int lim = src_s - t.org_s < ts ? src_s - t.org_s : ts;
      const int vpr_shift = ts_shift - __builtin_ctz((unsigned)(V / 2)), vpr = 1 << vpr_shift;
      for (int j = 0; j < 2 * Geo::VPT; ++j) {
        const int vi = j * 256 + tid;
        const int r = vi >> vpr_shift, k = vi & (vpr - 1);
        if (t.org_d + r >= src_d || k * (V / 2) >= lim)
          continue;
        Vec u;
        u.v = *(const Bytes16 *)(src + t.so + (int64_t)r * ss_d + k * V);
        T *at = &tile[r * pitch + k * (V / 2)];
        for (int e = 0; e < V / 2; ++e)
          at[e] = u.e[2 * e];
      }
    } else {
      for (int j = 0; j < Geo::AREA / 256; ++j) {
        const int idx = j * 256 + tid;
        const int r = idx >> ts_shift, cs = idx & (ts - 1);
        if (t.org_d + r < src_d && t.org_s + cs < src_s)
          tile[r * pitch + cs] = src[t.so + (int64_t)r * ss_d + (int64_t)cs * ss_s];
      }
    }
    return;
  }
  const int64_t ds_s = p.ds_s;
  const int vpd_shift = td_shift - __builtin_ctz((unsigned)V), vpd = 1 << vpd_shift;
  const bool words = ((a0 | astep) & (unsigned)(G - 1)) == 0;
  if (words) {
    for (int j = 0; j < Geo::VPT / G; ++j) {
      const int vi = j * 256 + tid;
      const int cs = (vi >> vpd_shift) * G, d0 = (vi & (vpd - 1)) * V;
      if (t.org_s + cs >= size_s || t.org_d + d0 >= size_d)
        continue;
      uint32_t w[V];
      for (int e = 0; e < V; ++e) {
        const int m = (int)((a0 + (unsigned)(d0 + e) * astep) & (unsigned)(V - 1));
        w[e] = *(const uint32_t *)&tile[(d0 + e) * pitch + cs + m];
      }
      for (int q = 0; q < G; ++q) {
        if (t.org_s + cs + q >= size_s)
          break;
        const bool col_in = t.outer_in && t.org_s + cs + q < src_s;
        Vec u;
        for (int e = 0; e < V; ++e)
          u.e[e] = (col_in && t.org_d + d0 + e < src_d) ? (T)(w[e] >> (8 * ES * q)) : (T)0;
        T *g = dst + t.dof + (int64_t)(cs + q) * ds_s + d0;
        if (t.org_d + d0 + V <= size_d && ((uintptr_t)g & 15) == 0) {
          *(Bytes16 *)g = u.v;
        } else {
          for (int e = 0; e < V; ++e)
            if (t.org_d + d0 + e < size_d)
              g[e] = u.e[e];
        }
      }
    }
  } else {
    for (int j = 0; j < Geo::VPT; ++j) {
      const int vi = j * 256 + tid;
      const int cs = vi >> vpd_shift, d0 = (vi & (vpd - 1)) * V;
      if (t.org_s + cs >= size_s || t.org_d + d0 >= size_d)
        continue;
      const bool col_in = t.outer_in && t.org_s + cs < src_s;
      Vec u;
      for (int e = 0; e < V; ++e) {
        const int m = (int)((a0 + (unsigned)(d0 + e) * astep) & (unsigned)(V - 1));
        u.e[e] = (col_in && t.org_d + d0 + e < src_d) ? tile[(d0 + e) * pitch + cs + m] : (T)0;
      }
      T *g = dst + t.dof + (int64_t)cs * ds_s + d0;
      if (t.org_d + d0 + V <= size_d && ((uintptr_t)g & 15) == 0) {
        *(Bytes16 *)g = u.v;
      } else {
        for (int e = 0; e < V; ++e)
          if (t.org_d + d0 + e < size_d)
            g[e] = u.e[e];
      }
    }
  }
}

// RELAYOUT_COPY: a thread builds one 16-byte chunk of the destination, reading
// zero beyond the source's extent in any dimension.  Either the destination's
// runs along dimension 4 are whole chunks (tile_d == 1), or a run is a fraction
// of a chunk (3 channels padded to 4 of 16 bits) and a chunk holds the runs of
// tile_d consecutive positions of dimension 3, which the destination stores
// back to back; size[3] is then a multiple of tile_d.  Source and destination
// usually share their contiguous dimension; when not (an NCHW image whose
// pixels become such runs), consecutive threads, which take consecutive
// chunks, still read consecutive addresses.  blockIdx.x enumerates groups of
// 256 chunks over the flattened dimensions (2, 3, chunk), then dimensions 1
// and 0.
template <typename T>
RK_DEV void copy_thread(const T *src, T *dst, const RockRelayoutParams &p, unsigned block, int tid) {
  constexpr int EPC = 16 / (int)sizeof(T); // elements per chunk
  const int ppc = p.tile_d;                // positions of dimension 3 per chunk
  const unsigned chunks4 = ppc > 1 ? 1u : (unsigned)p.size[4] / EPC;
  const unsigned groups3 = (unsigned)p.size[3] / (unsigned)ppc;
  const unsigned inner = (unsigned)p.size[2] * groups3 * chunks4;
  const unsigned per = (inner + 255) / 256;
  unsigned b = fast_div(block, p.div[0]);
  unsigned q = (block - b * per) * 256 + (unsigned)tid;
  const unsigned i0 = fast_div(b, p.div[1]), i1 = b - i0 * (unsigned)p.size[1];
  if (q >= inner)
    return;
  unsigned r = fast_div(q, p.div[2]);
  const unsigned ch = q - r * chunks4;
  const unsigned i2 = fast_div(r, p.div[3]), i3 = (r - i2 * groups3) * (unsigned)ppc;
  const int64_t so = (int64_t)i0 * p.src_stride[0] + (int64_t)i1 * p.src_stride[1] +
                     (int64_t)i2 * p.src_stride[2] + (int64_t)i3 * p.src_stride[3];
  const int64_t dof = (int64_t)i0 * p.dst_stride[0] + (int64_t)i1 * p.dst_stride[1] +
                      (int64_t)i2 * p.dst_stride[2] + (int64_t)i3 * p.dst_stride[3] + (int64_t)ch * EPC;
  const bool outer_in = i0 < (unsigned)p.src_size[0] && i1 < (unsigned)p.src_size[1] &&
                        i2 < (unsigned)p.src_size[2];
  const int lim4 = outer_in ? p.src_size[4] : 0;
  const int64_t ss3 = p.src_stride[3], ss4 = p.src_stride[4];
  union {
    T e[EPC];
    Bytes16 v;
  } u;
  if (ppc > 1) {
    const int run_shift = __builtin_ctz((unsigned)p.size[4]); // a run is a power of two of elements
    for (int j = 0; j < EPC; ++j) {
      const int pos = j >> run_shift, e = j & (p.size[4] - 1);
      u.e[j] = (e < lim4 && (int)i3 + pos < p.src_size[3]) ? src[so + (int64_t)pos * ss3 + (int64_t)e * ss4] : (T)0;
    }
  } else {
    const int e0 = (int)ch * EPC, lim = (int)i3 < p.src_size[3] ? lim4 : 0;
    for (int j = 0; j < EPC; ++j)
      u.e[j] = e0 + j < lim ? src[so + (int64_t)(e0 + j) * ss4] : (T)0;
  }
  *(Bytes16 *)(dst + dof) = u.v;
}

// Elements of LDS a block needs, whatever the mode.
template <typename T> constexpr int lds_elems() {
  return VecGeom<T>::LDS_ELEMS > 1024 + 128 ? VecGeom<T>::LDS_ELEMS : 1024 + 128;
}

// phase 0, the block's barrier, phase 1
template <typename T>
RK_DEV void relayout_phase(int phase, const T *src, T *dst, const RockRelayoutParams &p, unsigned block,
                           unsigned nblocks, int tid, T *lds) {
  if (p.mode == RELAYOUT_COPY) {
    if (phase == 0)
      copy_thread<T>(src, dst, p, block, tid);
  } else if (p.mode == RELAYOUT_TRANSPOSE_VEC) {
    transpose_vec_phase<T>(phase, src, dst, p, block, nblocks, tid, lds);
  } else {
    transpose_phase<T>(phase, src, dst, p, block, tid, lds);
  }
}

} // namespace rock_relayout
