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

// ---------------------------------------------------------------------------
// Iterator over the tiles (of kSumRows rows each) on the other side of the
// score matrix that may hold a kept element for this workgroup's rows.
// All state is wave-uniform.  `first`/`last` bound the range from the causal
// structure; inside it a tile is visited iff doc_may_keep() of its summary.
// ---------------------------------------------------------------------------
struct TileIter {
  unsigned long long mask;
  int base, last;  // tiles [.., last)
  int q_lo, q_hi, q_glob;
  const IdSummary* sum;  // summaries of the iterated side, or nullptr (visit all)
  bool iter_keys;        // true: own side is the query side, iterated side is keys

  FA_DEV void init(int first, int last_, const IdSummary* s, int lo, int hi, int glob, bool keys) {
    sum = s; q_lo = lo; q_hi = hi; q_glob = glob; iter_keys = keys;
    last = last_;
    base = (first / 64) * 64;
    mask = chunk_mask(base) & (~0ull << (first - base));
  }
  FA_DEV unsigned long long chunk_mask(int b) const {
    const int t = b + (threadIdx.x & 63);
    bool v = t < last;
    if (sum != nullptr && v) {
      const IdSummary s = sum[t];
      v = iter_keys ? doc_may_keep(q_lo, q_hi, q_glob, s.lo, s.hi)
                    : doc_may_keep(s.lo, s.hi, s.glob, q_lo, q_hi);
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

}  // namespace fa
