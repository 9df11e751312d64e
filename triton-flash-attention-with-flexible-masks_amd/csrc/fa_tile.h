// LDS tile staging, MFMA fragment readers and the tile-skip iterator shared by
// the forward, dq and dk/dv kernels.
#pragma once

#include "fa_common.h"

namespace fa {

// ---------------------------------------------------------------------------
// LDS tile layout.  A tile is ROWS rows of D elements (2 bytes each), row pitch
// D*2 bytes, split into 16-byte chunks.  The chunk index is XOR-swizzled with a
// function of the row chosen so that both access patterns used by the kernels
// spread over all banks:
//   row reads : MFMA A/B operands, 16 bytes per lane, 16 consecutive rows at the
//               same logical chunk per LDS cycle   -> 16 distinct physical chunks
//   tr reads  : ds_read_b64_tr_b16, a half wave touches 4 consecutive rows x 64
//               contiguous bytes                    -> 4 distinct 64-byte windows
// For D = 128 (16 chunks per row) the 4-bit swizzle ((row & 3) << 2) | ((row >> 2) & 3)
// is a bijection on 16 consecutive rows and puts row & 3 in the window bits.
// ---------------------------------------------------------------------------
enum { SWZ_ROW = 0, SWZ_TR = 1 };  // kept as a tag of the intended access; same map

template <int D, int SWZ>
FA_DEV int swz(int row) {
  constexpr int CPR = D / 8;  // 16-byte chunks per row
  if (CPR == 16) return ((row & 3) << 2) | ((row >> 2) & 3);
  if (CPR == 8) return ((row & 1) << 2) | ((row >> 1) & 3);
  if (CPR == 4) return (row >> 2) & 3;
  return 0;
}

// Asynchronously copy ROWS x D elements (rows row0 .. row0+ROWS-1 of a [*, D]
// matrix with row stride `rs` elements, rows clamped to nrows-1) from global
// memory straight into LDS, all 256 threads cooperating.  Completion is
// observed with s_waitcnt vmcnt(0) followed by a workgroup barrier.
template <typename T, int D, int ROWS, int SWZ>
FA_DEV void tile_load_async(const T* __restrict__ g, int64_t rs, int row0, int nrows, char* lds) {
  constexpr int CPR = D / 8;          // chunks per row
  constexpr int RPI = 64 / CPR;       // rows per wave instruction
  constexpr int NI = ROWS / RPI;      // wave instructions per tile
  static_assert(NI % 4 == 0, "tile must split evenly over 4 waves");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < NI / 4; ++i) {
    const int inst = i * 4 + wave;
    const int row = inst * RPI + lane / CPR;
    const int pc = lane % CPR;
    const int c = pc ^ swz<D, SWZ>(row);
    int grow = row0 + row;
    grow = grow < nrows ? grow : nrows - 1;
    const T* src = g + int64_t(grow) * rs + c * 8;
    __builtin_amdgcn_global_load_lds(FA_GLB(src), FA_LDS(lds + inst * 1024), 16, 0, 0);
  }
}

// Same, with an explicit list of row indices (gathered rows), idx[r] already clamped.
template <typename T, int D, int ROWS, int SWZ>
FA_DEV void tile_load_async_rows(const T* __restrict__ g, int64_t rs, const int* __restrict__ idx, char* lds) {
  constexpr int CPR = D / 8;
  constexpr int RPI = 64 / CPR;
  constexpr int NI = ROWS / RPI;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < NI / 4; ++i) {
    const int inst = i * 4 + wave;
    const int row = inst * RPI + lane / CPR;
    const int pc = lane % CPR;
    const int c = pc ^ swz<D, SWZ>(row);
    const T* src = g + int64_t(idx[row]) * rs + c * 8;
    __builtin_amdgcn_global_load_lds(FA_GLB(src), FA_LDS(lds + inst * 1024), 16, 0, 0);
  }
}

FA_DEV void wait_async_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// 8 consecutive elements of row `row` starting at element 8*chunk (A or B operand).
template <typename E, int D, int SWZ>
FA_DEV typename E::vec8 frag_row(const char* lds, int row, int chunk) {
  const int pc = chunk ^ swz<D, SWZ>(row);
  return *reinterpret_cast<const typename E::vec8*>(lds + row * (D * 2) + pc * 16);
}

// Transposed operand: for the 16 rows rbase .. rbase+15 of the tile and the 32
// columns 32*db .. 32*db+31, returns for lane l (col = 32*db + (l & 31), g = l >> 5)
// the 8 values of rows rbase + {4g..4g+3, 8+4g..8+4g+3} at that column, which is the
// k-slot order of an accumulator block reused as the other MFMA operand.
template <typename E, int D, int SWZ>
FA_DEV typename E::vec8 frag_tr(const char* lds, int rbase, int db) {
  const int l = threadIdx.x & 63;
  const int i = l & 15, e = i >> 2, c4 = i & 3, hd = (l >> 4) & 1, g = l >> 5;
  const int chunk = 4 * db + 2 * hd + (c4 >> 1);
  const int sub = (c4 & 1) * 8;
  const int r0 = rbase + 4 * g + e;
  const int r1 = r0 + 8;
  typename E::vec4 lo = E::lds_tr(lds + r0 * (D * 2) + ((chunk ^ swz<D, SWZ>(r0)) * 16) + sub);
  typename E::vec4 hi = E::lds_tr(lds + r1 * (D * 2) + ((chunk ^ swz<D, SWZ>(r1)) * 16) + sub);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Buffer resource and buffer -> LDS load.  The resource type and the builtins exist
// only in the device pass; the host pass (which still parses the kernels to emit
// their launch stubs) sees a plain struct and empty bodies.
#if defined(__HIP_DEVICE_COMPILE__)
typedef __amdgpu_buffer_rsrc_t buf_rsrc_t;
FA_DEV buf_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
// 16 bytes per lane from base + voff + soff into lds + 16 * lane
FA_DEV void buf_load_lds16(buf_rsrc_t r, char* lds, int voff, int soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, FA_LDS(lds), 16, voff, soff, 0, 0);
}
#else
struct buf_rsrc_t { int w[4]; };
FA_DEV buf_rsrc_t make_rsrc(const void*, unsigned) { return buf_rsrc_t(); }
FA_DEV void buf_load_lds16(buf_rsrc_t, char*, int, int) {}
#endif

// Global -> LDS tile streamer built on buffer loads with the LDS destination
// (buffer_load_dwordx4 ... lds).  The per-lane byte offsets are computed once;
// a tile is then addressed with one scalar offset, and rows past the end of the
// matrix read as zero through the buffer's range check instead of being clamped.
// D is the row width of the LDS tile, GD (<= D) the width of the rows in memory; chunks past GD
// are fetched from beyond the buffer's range, i.e. zero filled.
constexpr int kOobOffset = (int)0x80000000;  // beyond any buffer this library accepts (< 2 GiB)

template <int D, int ROWS, int GD = D>
struct TileLoader {
  static constexpr int CPR = D / 8;      // 16-byte chunks per row
  static constexpr int RPI = 64 / CPR;   // rows per wave instruction
  static constexpr int NI = ROWS / RPI;  // wave instructions per tile
  static constexpr int PER = NI / 4;     // per wave
  static_assert(NI % 4 == 0, "tile must split evenly over 4 waves");
  buf_rsrc_t rsrc;
  int voff[PER];
  int row_bytes;

  // base: first row of the (batch, head) slice; rs: row stride in elements
  FA_DEV void init(const void* base, int64_t rs, int nrows) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned bytes = (unsigned)((int64_t(nrows - 1) * rs + GD) * 2);
    rsrc = make_rsrc(base, bytes);
    row_bytes = int(rs) * 2;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int row = (i * 4 + wave) * RPI + lane / CPR;
      const int c = (lane % CPR) ^ swz<D, SWZ_ROW>(row);
      voff[i] = c < GD / 8 ? row * row_bytes + c * 16 : kOobOffset;
    }
  }
  // stream rows row0 .. row0+ROWS-1 into the tile at `lds`
  FA_DEV void issue(int row0, char* lds) const {
    const int wave = threadIdx.x >> 6;
    const int soff = row0 * row_bytes;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      buf_load_lds16(rsrc, lds + (i * 4 + wave) * 1024, voff[i], soff);
  }
};

// Byte offsets (inside one tile) of the operand reads of one lane, computed once.
//   row[ks]     : 16 bytes of row (l & 31) at logical chunk 2*ks + (l >> 5); add
//                 32*rows*D*2 for the next 32-row block
//   tr[db][hh]  : the ds_read_b64_tr_b16 source of frag_tr for rows {4g+e (+8*hh)} of a
//                 16-row group and columns 32*db..; add 16*D*2 per 16-row group
template <int D>
struct LdsOffsets {
  static constexpr int KS = D / 16, DBN = D / 32;
  int row[KS];
  int tr[DBN][2];
  FA_DEV void init() {
    const int l = threadIdx.x & 63;
    const int lq = l & 31, g = l >> 5;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) row[ks] = lq * (D * 2) + (((2 * ks + g) ^ swz<D, SWZ_ROW>(lq)) << 4);
    const int i = l & 15, e = i >> 2, c4 = i & 3, hd = (l >> 4) & 1;
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int r = 4 * g + e + 8 * hh;
        const int chunk = 4 * db + 2 * hd + (c4 >> 1);
        tr[db][hh] = r * (D * 2) + ((chunk ^ swz<D, SWZ_TR>(r)) << 4) + (c4 & 1) * 8;
      }
  }
};

template <typename E>
FA_DEV typename E::vec8 lds_row8(const char* p) { return *reinterpret_cast<const typename E::vec8*>(p); }

template <typename E>
FA_DEV typename E::vec8 lds_tr8(const char* p0, const char* p1) {
  typename E::vec4 lo = E::lds_tr(p0);
  typename E::vec4 hi = E::lds_tr(p1);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// ---------------------------------------------------------------------------
// Iterator over the 64-entry tiles of the other side of the score matrix that may
// hold a kept element for this workgroup's rows.  All state is wave-uniform: each
// lane tests one candidate tile and a ballot turns 64 tests into a bit mask.
//   keys mode   : own side = query tile (lo, hi, glob), candidates = key tiles
//                 [first, last) in natural order
//   query mode  : own side = key tile (lo, hi), candidates = tiles of the permuted
//                 query order; a tile is a candidate if it holds rows and, with a
//                 causal mask, its largest row index reaches the own keys
// With sum == nullptr (no document ids) every tile of the range is visited.
// ---------------------------------------------------------------------------
struct TileIter {
  unsigned long long mask;
  int base, last;
  int o_lo, o_hi, o_glob;
  int min_rmax;            // query mode: candidates need rmax >= min_rmax
  bool keys_mode;
  const IdSummary* sum;

  FA_DEV void init_keys(int first, int last_, const IdSummary* ksum, int q_lo, int q_hi, int q_glob) {
    sum = ksum; o_lo = q_lo; o_hi = q_hi; o_glob = q_glob; keys_mode = true; min_rmax = 0;
    start(first, last_);
  }
  FA_DEV void init_queries(int first, int last_, const IdSummary* qsum, int k_lo, int k_hi, int min_rmax_) {
    sum = qsum; o_lo = k_lo; o_hi = k_hi; o_glob = 0; keys_mode = false; min_rmax = min_rmax_;
    start(first, last_);
  }
  FA_DEV void start(int first, int last_) {
    last = last_;
    base = (first / 64) * 64;
    mask = chunk_mask(base) & (~0ull << (first - base));
  }
  FA_DEV unsigned long long chunk_mask(int b) const {
    const int t = b + (threadIdx.x & 63);
    bool v = t < last;
    if (sum != nullptr && v) {
      const IdSummary s = sum[t];
      v = keys_mode ? doc_may_keep(o_lo, o_hi, o_glob, s.lo, s.hi)
                    : (s.nvalid > 0 && s.rmax >= min_rmax && doc_may_keep(s.lo, s.hi, s.glob, o_lo, o_hi));
    }
    return __builtin_amdgcn_ballot_w64(v);
  }
  // next tile index, or -1
  FA_DEV int next() {
    while (mask == 0) {
      base += 64;
      if (base >= last) return -1;
      mask = chunk_mask(base);
    }
    const int j = base + __builtin_ctzll(mask);
    mask &= mask - 1;
    return j;
  }
};

// ---------------------------------------------------------------------------
// Query-side tile context shared by the forward and dq kernels: which original
// row this lane owns, its id, the id / row-index summaries of the wave's 32 rows
// and of the workgroup's 128 rows, and the mask decisions per key tile.
// ---------------------------------------------------------------------------
template <bool CAUSAL, bool DOC>
struct QTileCtx {
  int row;    // original row index of this lane's query (lanes l and l^32 share it), -1 if none
  int rowc;   // row clamped into [0, M) for loads
  int eq_i;
  int w_lo, w_hi, w_glob, w_rmin, w_rmax;  // this wave's 32 rows
  int g_lo, g_hi, g_glob, g_rmax;          // the workgroup's 128 rows
  const int* ekp;
  const IdSummary* ksum;

  // tile: index of the 128-row tile (natural order, or permuted order with ids).
  // Returns false when the tile holds no row.
  FA_DEV bool init(const KArgs& a, int b, int h, int tile) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lq = lane & 31;
    eq_i = 0; ekp = nullptr; ksum = nullptr;
    w_lo = 0; w_hi = -1; w_glob = 1; g_lo = 0; g_hi = -1; g_glob = 1;
    if (!DOC) {
      const int m0 = tile * 128, mw = m0 + wave * 32;
      row = mw + lq < a.M ? mw + lq : -1;
      w_rmin = mw; w_rmax = min(mw + 31, a.M - 1);
      if (w_rmax < w_rmin) w_rmax = -1;
      g_rmax = min(m0 + 127, a.M - 1);
    } else {
      const QHeader hd = a.qhdr[b * a.qh_bs + h * a.qh_hs];
      if (tile >= hd.nT128) return false;
      row = a.perm[b * a.pm_bs + h * a.pm_hs + tile * 128 + wave * 32 + lq];
      const IdSummary* qs = a.qsum + b * a.qs_bs + h * a.qs_hs + 2 * tile;
      const IdSummary s0 = qs[0], s1 = qs[1];
      g_lo = min(s0.lo, s1.lo); g_hi = max(s0.hi, s1.hi); g_glob = s0.glob | s1.glob;
      g_rmax = max(s0.rmax, s1.rmax);
      ekp = a.ek32 + b * a.ek_bs + h * a.ek_hs;
      ksum = a.ksum + b * a.ks_bs + h * a.ks_hs;
      eq_i = row >= 0 ? a.eq32[b * a.eq_bs + h * a.eq_hs + row] : 0;
      const bool local = (eq_i < 0) && (row >= 0);
      int lo = local ? eq_i : 0x7fffffff, hi = local ? eq_i : (int)0x80000000;
      int rmin = row >= 0 ? row : 0x7fffffff, rmax = row;
#pragma unroll
      for (int off = 16; off >= 1; off >>= 1) {
        lo = min(lo, __shfl_xor(lo, off));
        hi = max(hi, __shfl_xor(hi, off));
        rmin = min(rmin, __shfl_xor(rmin, off));
        rmax = max(rmax, __shfl_xor(rmax, off));
      }
      w_lo = lo; w_hi = hi; w_rmin = rmin; w_rmax = rmax;
      w_glob = __builtin_amdgcn_ballot_w64(eq_i >= 0 && row >= 0) != 0;
    }
    rowc = row >= 0 ? row : 0;
    return true;
  }
  // one past the last key any row of the workgroup can see
  FA_DEV int hi_key(const KArgs& a) const { return CAUSAL ? min(a.N, a.gap + g_rmax + 1) : a.N; }

  // wave-level decisions for key tile `cur` (keys n0 .. n0+BN-1)
  FA_DEV void decide(const KArgs& a, int cur, int n0, int BN, bool& skip, bool& need_mask) const {
    skip = (w_rmax < 0) || (CAUSAL && (n0 > a.gap + w_rmax));
    need_mask = (n0 + BN > a.N) || (CAUSAL && (n0 + BN - 1 > a.gap + w_rmin));
    if (DOC) {
      const IdSummary ks = ksum[cur];
      skip = skip || !doc_may_keep(w_lo, w_hi, w_glob, ks.lo, ks.hi);
      need_mask = need_mask || !doc_all_keep(w_lo, w_hi, ks.lo, ks.hi);
    }
  }
};

// blockIdx -> (tile, batch*head) for grids of `ntile` tiles per (batch, head):
// consecutive workgroup ids land on different XCDs, so every XCD is given whole
// heads (its L2 then keeps that head's K/V or Q/dO).  Returns false for padding ids.
FA_DEV bool block_to_tile(int ntile, int BH, int& tile_slot, int& bh) {
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  bh = (idx / ntile) * 8 + xcd;
  tile_slot = idx % ntile;
  return bh < BH;
}

}  // namespace fa
