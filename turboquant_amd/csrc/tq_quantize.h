// Pieces shared by the vector-ALU and the matrix-core key quantise kernels: where a
// tile of 16 vectors comes from, where its codes go, and the two writers.
#pragma once

#include <type_traits>

#include "tq_common.h"

namespace tq {

constexpr int TILE = TQ_PAGE_TOKENS;

// ------------------------------------------------------------------------------------
// tile sources: where the 16 vectors of a tile come from and which are valid
// ------------------------------------------------------------------------------------

// What the staging code of the matrix-core kernels needs to know about a tile, all of it uniform: slot s
// of the tile exists iff lo <= s < hi, and its row starts `base + s * slot_stride()` elements into the
// tensor.  A source hands it out for consecutive tiles through a walk (begin at a tile, step to the next),
// so that the index arithmetic of a tile number (divisions by run-time sizes) is done once per group.
struct TileAddr { int64_t base; int lo, hi; };

// N uniform 32-bit loads p[at[k]] through the scalar cache with one wait (read-only inputs only: the
// scalar cache does not see what vector stores of the same launch write)
template <int N>
__device__ __forceinline__ void sload(const int32_t* p, const int (&at)[N], int32_t (&v)[N]) {
  static_assert(N == 1 || N == 2 || N == 4, "one, two or four at a time");
  const int32_t* q[N];
#pragma unroll
  for (int k = 0; k < N; ++k) q[k] = p + __builtin_amdgcn_readfirstlane(at[k]);
  if constexpr (N == 4) {
    asm volatile("s_load_dword %0, %4, 0x0\n\ts_load_dword %1, %5, 0x0\n\ts_load_dword %2, %6, 0x0\n\t"
                 "s_load_dword %3, %7, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(v[0]), "=&s"(v[1]), "=&s"(v[2]), "=&s"(v[3])
                 : "s"(q[0]), "s"(q[1]), "s"(q[2]), "s"(q[3])
                 : "memory");
  } else if constexpr (N == 1) {
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=&s"(v[0]) : "s"(q[0]) : "memory");
  } else {
    asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(v[0]), "=&s"(v[1])
                 : "s"(q[0]), "s"(q[1])
                 : "memory");
  }
}

struct FlatSource {          // (n_vec, d) with a row stride
  int64_t n_vec, row_stride;
  __device__ int64_t slot_stride() const { return row_stride; }
  __device__ TileAddr tile_addr(int64_t tile) const {
    const int64_t left = n_vec - tile * TILE;
    return TileAddr{tile * TILE * row_stride, 0, (int)(left < 0 ? 0 : (left > TILE ? TILE : left))};
  }
  struct TileRef { int64_t v0; };
  __device__ TileRef tile_ref(int64_t tile) const { return TileRef{tile * TILE}; }
  __device__ bool slot_off(const TileRef& r, int slot, int64_t& elem_off) const {
    elem_off = (r.v0 + slot) * row_stride;
    return r.v0 + slot < n_vec;
  }
  __device__ bool locate(int tile, int slot, int64_t& elem_off) const {
    int64_t v = (int64_t)tile * TILE + slot;
    elem_off = v * row_stride;
    return v < n_vec;
  }
};

__device__ const int32_t k_zero_i32 = 0;
__device__ const int32_t k_max_i32 = 0x7fffffff;

struct PagedSource {         // (b, t, h, :) strided, tokens mapped onto 16-token pages
  int B, T, H, tiles_per_seq;
  int64_t stride_b, stride_t, stride_h;
  const int32_t* start_pos;
  // Optional block-gather mode: the tokens sit in a paged exact cache (blocks of 16 tokens).  Token at
  // absolute position p of sequence b is slot p % 16 of block src_table[b * src_stride + p / 16]; blocks
  // are stride_blk elements apart and stride_b is unused.  run_len (optional) bounds the run of each
  // sequence separately (<= T).
  const int32_t* src_table = nullptr;
  int src_stride = 0;
  int64_t stride_blk = 0;
  const int32_t* run_len = nullptr;
  // Optional ragged mode: the rows of all sequences lie one after another in one (rows, H, :) tensor; the
  // run of sequence b begins at row row0[b] (stride_b is unused, run_len gives its length).
  const int32_t* row0 = nullptr;
  // (sequence, page slot window, head) of a tile, and of the tile after it (a walk that leaves the last
  // sequence stays on its last tile): the divisions by run-time sizes are done once per group of tiles
  struct Coord { int b, pg, h; };
  __device__ Coord coord(int64_t tile) const {
    Coord c;
    c.h = (int)tile % H;
    const int r = (int)tile / H;
    c.pg = r % tiles_per_seq;
    c.b = r / tiles_per_seq;
    return c;
  }
  __device__ void next(Coord& c) const {
    if (c.h + 1 < H) ++c.h;
    else if (c.pg + 1 < tiles_per_seq) { c.h = 0; ++c.pg; }
    else if (c.b + 1 < B) { c.h = 0; c.pg = 0; ++c.b; }
  }
  __device__ int64_t slot_stride() const { return stride_t; }
  // Addresses of N tiles.  The per-sequence words come through the scalar cache, N at a time (they are
  // inputs of the launch that no kernel writes; as ordinary loads they would be vector-memory loads with
  // a full wait each, one after the other, in every pass of a persistent workgroup).
  template <int N>
  __device__ void tile_addrs(const Coord (&c)[N], TileAddr (&ta)[N], int (&lpage)[N]) const {
    int32_t s0[N], lim[N], r0[N], blk[N], at[N];
#pragma unroll
    for (int m = 0; m < N; ++m) { at[m] = c[m].b; s0[m] = 0; lim[m] = k_max_i32; r0[m] = 0; blk[m] = 0; }
    if (start_pos) sload<N>(start_pos, at, s0);
    if (run_len) sload<N>(run_len, at, lim);
    if (row0) sload<N>(row0, at, r0);
#pragma unroll
    for (int m = 0; m < N; ++m) {
      lpage[m] = s0[m] / TILE + c[m].pg;
      at[m] = c[m].b * src_stride + min(lpage[m], src_stride - 1);
    }
    if (src_table) sload<N>(src_table, at, blk);
#pragma unroll
    for (int m = 0; m < N; ++m) {
      const int t0 = lpage[m] * TILE - s0[m];
      const int64_t base = src_table ? (int64_t)blk[m] * stride_blk - (int64_t)t0 * stride_t
                                     : (row0 ? (int64_t)r0[m] * stride_t : c[m].b * stride_b);
      // slot s is token t0 + s of the run: it exists iff 0 <= t0 + s < min(run length, T)
      ta[m] = TileAddr{base + c[m].h * stride_h + (int64_t)t0 * stride_t, -t0, min(lim[m], T) - t0};
    }
  }
  // tile index -> (b, page slot window, head)
  __device__ void decode(int tile, int& b, int& lpage, int& h) const {
    h = tile % H;
    int r = tile / H;
    int pg = r % tiles_per_seq;
    b = r / tiles_per_seq;
    int s0 = start_pos ? start_pos[b] : 0;
    lpage = s0 / TILE + pg;
  }
  // the part of locate() that is the same for the 16 slots of a tile
  struct TileRef { int64_t base; int t0; int lim; };
  __device__ TileRef tile_ref(int64_t tile) const {
    int h = (int)tile % H;
    int r = (int)tile / H;
    int pg = r % tiles_per_seq;
    int b = r / tiles_per_seq;
    // unconditional loads (no branch on the null pointers): a load under a branch makes the
    // compiler wait for every outstanding load at the join
    int s0 = *(start_pos ? start_pos + b : &k_zero_i32);
    const int lpage = s0 / TILE + pg, t0 = lpage * TILE - s0;
    const int lim = min(*(run_len ? run_len + b : &k_max_i32), T);
    const int64_t blk = *(src_table ? src_table + (int64_t)b * src_stride + min(lpage, src_stride - 1) : &k_zero_i32);
    const int64_t r0 = *(row0 ? row0 + b : &k_zero_i32);
    const int64_t base = src_table ? blk * stride_blk - (int64_t)t0 * stride_t : (row0 ? r0 * stride_t : b * stride_b);
    return TileRef{base + h * stride_h, t0, lim};
  }
  __device__ bool slot_off(const TileRef& r, int slot, int64_t& elem_off) const {
    int t = r.t0 + slot;
    elem_off = r.base + (int64_t)t * stride_t;
    return t >= 0 && t < r.lim;
  }
  __device__ bool locate(int tile, int slot, int64_t& elem_off) const {
    return slot_off(tile_ref(tile), slot, elem_off);
  }
};

// ------------------------------------------------------------------------------------
// key tile
// ------------------------------------------------------------------------------------

struct KeyFlatSink {
  uint8_t* idx;
  uint8_t* sign;
  void* norm;
  float* rnorm;
  float* y_dbg;
  float* p_dbg;
};

struct KeyPagedSink {
  uint8_t* pool;
  const int32_t* block_table;
  int max_pages;
  int num_pages;           // pages of the pool: a table entry outside [0, num_pages) is never written through
  tq_page_layout L;
};

// Physical page of logical page `lpage` of sequence b, or -1 when the logical page lies outside the block
// table or the table entry outside the pool (a stale or poisoned entry): the writers then store nothing.
// The table load itself is unconditional and clamped into the table.
__device__ __forceinline__ int64_t checked_page(const int32_t* block_table, int max_pages, int num_pages, int b,
                                                int lpage) {
  const int raw = block_table[(int64_t)b * max_pages + min(max(lpage, 0), max_pages - 1)];
  return (lpage >= 0 && lpage < max_pages && (unsigned)raw < (unsigned)num_pages) ? (int64_t)raw : (int64_t)-1;
}


// ------------------------------------------------------------------------------------
// writers for one tile of 16 vectors, run by `nthreads` cooperating threads (tid = 0..nthreads-1).
// sidx / ssgn hold one byte per (slot, coordinate): the Lloyd-Max index and the sign bit;
// snorm / srn the key norm (as fp32) and the residual norm; svalid which slots exist.
// ------------------------------------------------------------------------------------

template <int DT>
__device__ __forceinline__ void write_key_tile_flat(const KeyFlatSink& sink, int64_t tile, int d, int mb, int mse_only,
                                                    const uint8_t* sidx, const uint8_t* ssgn, const float* snorm,
                                                    const float* srn, const int* svalid, int tid, int nthreads) {
  using E = Elem<DT>;
  const int eff = eff_bits(mb), per = 8 / eff, row = idx_row_bytes(d, mb), srow = d >> 3;
  for (int o = tid; o < TILE * row; o += nthreads) {
    int t = o / row, k = o - t * row;
    if (!svalid[t]) continue;
    unsigned byte = 0;
    for (int s = 0; s < per; ++s) {
      int c = k * per + s;
      if (c < d) byte |= (unsigned)sidx[t * d + c] << (eff * s);
    }
    sink.idx[(tile * TILE + t) * row + k] = (uint8_t)byte;
  }
  if (!mse_only) {
    for (int o = tid; o < TILE * srow; o += nthreads) {
      int t = o / srow, k = o - t * srow;
      if (!svalid[t]) continue;
      unsigned byte = 0;
      for (int s = 0; s < 8; ++s) byte |= (unsigned)ssgn[t * d + k * 8 + s] << s;
      sink.sign[(tile * TILE + t) * srow + k] = (uint8_t)byte;
    }
  }
  if (tid < TILE && svalid[tid]) {
    int64_t v = tile * TILE + tid;
    E::store(sink.norm, v, snorm[tid]);
    if (!mse_only) sink.rnorm[v] = srn[tid];
  }
}

__device__ __forceinline__ void write_key_tile_paged(const KeyPagedSink& sink, const PagedSource& src, int tile, int d,
                                                     int mb, const uint8_t* sidx, const uint8_t* ssgn,
                                                     const float* snorm, const float* srn, const int* svalid, int tid,
                                                     int nthreads) {
  int b, lpage, h;
  src.decode(tile, b, lpage, h);
  const tq_page_layout& L = sink.L;
  const int64_t page = checked_page(sink.block_table, sink.max_pages, sink.num_pages, b, lpage);
  if (page < 0) return;                                   // the same for every thread of the tile
  uint8_t* pg = sink.pool + (page * src.H + h) * (int64_t)L.page_bytes;
  const int words = d >> 5, planes = mb + 1;
  for (int o = tid; o < planes * words * TILE; o += nthreads) {
    int n = o % TILE, r = o / TILE;
    int w = r % words, p = r / words;
    if (!svalid[n]) continue;
    uint32_t bits = 0;
    if (p < mb) {
      int sh = mb - 1 - p;
      for (int i = 0; i < 32; ++i) bits |= (uint32_t)((sidx[n * d + w * 32 + i] >> sh) & 1) << i;
    } else {
      for (int i = 0; i < 32; ++i) bits |= (uint32_t)ssgn[n * d + w * 32 + i] << i;
    }
    *(uint32_t*)(pg + key_word_off(L, p, w, n)) = bits;
  }
  if (tid < TILE && svalid[tid]) {
    ((float*)(pg + L.off_meta))[2 * tid] = snorm[tid];
    ((float*)(pg + L.off_meta))[2 * tid + 1] = srn[tid];
  }
}

// matrix-core de-quantiser (tq_quantize_mfma.hip); TQ_EUNSUPPORTED = use the vector-ALU kernel
int launch_dequant_mfma(const uint8_t* idx, const uint8_t* signs, const void* norms, int norm_dtype, const float* rnorms,
                        int64_t n_vec, const tq_layer& ly, float* out, hipStream_t st);

}  // namespace tq
