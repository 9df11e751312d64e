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

// ---------------------------------------------------------------------------
// Asynchronous global -> LDS copies (the data never passes through registers).
// They are issued from inline assembly on purpose: written with the compiler's
// builtins, every later LDS read is preceded by s_waitcnt vmcnt(0), because the
// compiler cannot tell that the tile being filled is not the tile being read, and
// the copy of the next tile then no longer overlaps the arithmetic on this one.
// Completion is observed explicitly: wait_async_loads() followed by a workgroup
// barrier, before the first read of the tile.
// ---------------------------------------------------------------------------
// Raw buffer resource (stride 0): base address, byte range, gfx9 data-format word.
typedef i32x4 buf_rsrc_t;

FA_DEV buf_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  const unsigned long long p = reinterpret_cast<unsigned long long>(base);
  // wave-uniform by construction; readfirstlane tells the compiler so (the words must sit in SGPRs)
  buf_rsrc_t r = {__builtin_amdgcn_readfirstlane((int)(unsigned)p), __builtin_amdgcn_readfirstlane((int)((p >> 32) & 0xffff)),
                  __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
  return r;
}

// LDS byte address of a pointer into the workgroup's dynamic shared memory
FA_DEV unsigned lds_addr(const char* p) {
  return (unsigned)(unsigned long long)(p);  // the low 32 bits of a generic LDS address are the LDS offset
}

// 16 bytes per lane from base + voff + soff into lds + 16 * lane (out of range reads give 0)
FA_DEV void buf_load_lds16(buf_rsrc_t r, const char* lds, int voff, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :: "s"(__builtin_amdgcn_readfirstlane(lds_addr(lds))), "v"(voff), "s"(r), "s"(__builtin_amdgcn_readfirstlane(soff))
               : "memory", "m0");
}

// 4 bytes per lane from the lane's own address into lds + 4 * lane
FA_DEV void glb_load_lds4(const void* src, const char* lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
               :: "s"(__builtin_amdgcn_readfirstlane(lds_addr(lds))), "v"(src) : "memory", "m0");
}

FA_DEV void wait_async_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// A word in LDS used as a flag between two waves of a workgroup.  Explicit LDS instructions: a
// volatile access through a generic pointer would become a flat access whose completion is
// counted together with (and so waits for) the asynchronous global -> LDS loads in flight.
// LDS operations of one wave execute in issue order, so a flag stored after data is never
// visible before the data.
FA_DEV void lds_flag_store(const char* p, int v) {
  asm volatile("ds_write_b32 %0, %1" :: "v"(lds_addr(p)), "v"(v) : "memory");
}
FA_DEV int lds_flag_load(const char* p) {
  int v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_addr(p)) : "memory");
  return v;
}

// Global -> LDS tile streamer built on buffer loads with the LDS destination
// (buffer_load_dwordx4 ... lds).  The per-lane byte offsets are computed once;
// a tile is then addressed with one scalar offset, and rows past the end of the
// matrix read as zero through the buffer's range check instead of being clamped.
// D is the row width of the LDS tile, GD (<= D) the width of the rows in memory; chunks past GD
// are fetched from beyond the buffer's range, i.e. zero filled.
constexpr int kOobOffset = (int)0x80000000;  // beyond any buffer this library accepts (< 2 GiB)

template <int D, int ROWS, int GD = D, int NW = 4>
struct TileLoader {
  static constexpr int CPR = D / 8;      // 16-byte chunks per row
  static constexpr int RPI = 64 / CPR;   // rows per wave instruction
  static constexpr int NI = ROWS / RPI;  // wave instructions per tile
  static constexpr int PER = (NI + NW - 1) / NW;  // per wave (NW waves share the tile)
  buf_rsrc_t rsrc;
  int voff;       // this lane's byte offset inside the first group of NW * RPI rows
  int row_bytes;

  // base: first row of the (batch, head) slice; rs: row stride in elements
  FA_DEV void init(const void* base, int64_t rs, int nrows) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned bytes = (unsigned)((int64_t(nrows - 1) * rs + GD) * 2);
    rsrc = make_rsrc(base, bytes);
    row_bytes = int(rs) * 2;
    // The swizzle of a row depends on the row modulo NW * RPI only (see swz), so the lanes of wave
    // instruction i address the rows of instruction 0 moved down by i * NW * RPI rows: one vector
    // offset serves every instruction, the rest is a scalar offset.
    static_assert((NW * RPI) % 16 == 0, "swizzle period");
    const int row = wave * RPI + lane / CPR;
    const int c = (lane % CPR) ^ swz<D, SWZ_ROW>(row);
    voff = c < GD / 8 ? row * row_bytes + c * 16 : kOobOffset;
  }
  // stream rows row0 .. row0+ROWS-1 into the tile at `lds`
  FA_DEV void issue(int row0, char* lds) const {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: LDS targets stay in SGPRs
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (NI % NW == 0 || i * NW + wave < NI)
        buf_load_lds16(rsrc, lds + (i * NW + wave) * 1024, voff, (row0 + i * NW * RPI) * row_bytes);
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
//                 causal mask, its largest row index reaches the own keys (and, with a sliding
//                 window, its smallest row index is not past them)
// With sum == nullptr (no document ids) every tile of the range is visited.
// ---------------------------------------------------------------------------
// Wave-level decisions for one tile, taken when the candidates are tested (dec(tile, summary) is
// evaluated by the lane that tests the tile) and handed out with the tile index, so that the tile
// loop itself reads nothing from global memory.
// dec() returns the TF_ bits in its low word and, optionally, one value in its high word
// (tile_value(): handed out as `value`, e.g. the single id of a tile).
enum { TF_SKIP = 1, TF_LIM = 2, TF_DOC = 4, TF_GLOB = 8, TF_COL = 16, TF_NBITS = 5 };
// Returned by dec() next to those, not handed out: no wave of the workgroup needs this candidate
// (block mask), so it is not visited at all.
enum { TF_NONE = 32 };
FA_DEV long long tile_value(int flags, int value) { return (long long)(unsigned)flags | ((long long)value << 32); }

struct TileIter {
  unsigned long long mask;
  unsigned long long fm[TF_NBITS];   // per candidate: the TF_ bits of dec()
  int c_val;                  // per lane: the value dec() attached to this lane's candidate
  int value;                  // that value for the tile returned by the last next()
  int base, last;
  int flags;                  // TF_ bits of the tile returned by the last next()
  int o_lo, o_hi, o_glob;
  int min_rmax, max_rmin;  // query mode: candidates need rmax >= min_rmax and rmin <= max_rmin
  bool keys_mode;
  const IdSummary* sum;

  template <class Dec>
  FA_DEV void init_keys(int first, int last_, const IdSummary* ksum, int q_lo, int q_hi, int q_glob, const Dec& dec) {
    sum = ksum; o_lo = q_lo; o_hi = q_hi; o_glob = q_glob; keys_mode = true; min_rmax = 0; max_rmin = 0x7fffffff;
    start(first, last_, dec);
  }
  template <class Dec>
  FA_DEV void init_queries(int first, int last_, const IdSummary* qsum, int k_lo, int k_hi, int min_rmax_, int max_rmin_,
                           const Dec& dec) {
    sum = qsum; o_lo = k_lo; o_hi = k_hi; o_glob = 0; keys_mode = false; min_rmax = min_rmax_; max_rmin = max_rmin_;
    start(first, last_, dec);
  }
  template <class Dec>
  FA_DEV void start(int first, int last_, const Dec& dec) {
    last = last_; flags = 0; c_val = 0; value = 0;
    base = (first / 64) * 64;
    mask = chunk_mask(base, dec) & (~0ull << (first - base));
  }
  template <class Dec>
  FA_DEV unsigned long long chunk_mask(int b, const Dec& dec) {
    const int t = b + (threadIdx.x & 63);
    bool v = t < last;
    IdSummary s;
    s.lo = 0; s.hi = -1; s.glob = 0; s.rmin = 0; s.rmax = -1; s.nvalid = 0; s.kfirst = 0; s.klast = 0;
    if (sum != nullptr && v) {
      s = sum[t];
      v = keys_mode ? doc_may_keep(o_lo, o_hi, o_glob, s.lo, s.hi)
                    : (s.nvalid > 0 && s.rmax >= min_rmax && s.rmin <= max_rmin && doc_may_keep(s.lo, s.hi, s.glob, o_lo, o_hi));
    }
    const long long fv = dec(t, s);
    const int f = (int)fv;
    v = v && (f & TF_NONE) == 0;
    c_val = (int)(fv >> 32);
#pragma unroll
    for (int i = 0; i < TF_NBITS; ++i) fm[i] = __builtin_amdgcn_ballot_w64(((f >> i) & 1) != 0);
    return __builtin_amdgcn_ballot_w64(v);
  }
  // next tile index, or -1
  template <class Dec>
  FA_DEV int next(const Dec& dec) {
    while (mask == 0) {
      base += 64;
      if (base >= last) return -1;
      mask = chunk_mask(base, dec);
    }
    const int jl = __builtin_ctzll(mask);
    mask &= mask - 1;
    flags = 0;
#pragma unroll
    for (int i = 0; i < TF_NBITS; ++i) flags |= int((fm[i] >> jl) & 1) << i;
    value = __builtin_amdgcn_readlane(c_val, jl);
    return base + jl;
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
  // Causal terms are written in key positions: the diagonal of row i sits at key gp + r, where without ids
  // r is the row index and gp = gap, and with ids r is the position the mask plan stored for the row
  // (gap + row, or the caller's per-row position) and gp = 0.
  int gp;
  int w_lo, w_hi, w_glob, w_rmin, w_rmax;  // this wave's 32 rows (rmin / rmax: smallest / largest r)
  int g_lo, g_hi, g_glob, g_rmin, g_rmax;  // the workgroup's 128 rows
  int g_kfirst, g_klast;                   // key tiles (of 64) those rows can need, from the mask plan
  int lim_i;                               // last key this lane's row may see (causal / prefix and length limit)
  int w_limmin;                            // smallest such limit among the wave's rows
  int low_i;                               // first key this lane's row may see (sliding window; very negative: none)
  int w_lowmin, w_lowmax;                  // smallest / largest such bound among the wave's rows
  bool glob_i;                             // this lane's row has an id >= 0 (sees every id)
  // A tile with at most 64 rows (the last tile of the global rows, a short query block) would leave two of
  // the four waves without rows.  Then waves 2, 3 take the rows of waves 0, 1 as well (rb = row block of the
  // wave) and the pair splits every key tile between them: wave `sub` computes the 32-key half `sub` with a
  // softmax state (or dQ sum) of its own, and the two are merged once, after the tile loop.
  int rb, sub;
  bool halved;
  const int* ekp;
  const IdSummary* ksum;

  // tile: index of the 128-row tile (natural order, or permuted order with ids).
  // Returns false when the tile holds no row.
  // wave: index (0..3) of this wave inside the 128-row tile.
  FA_DEV bool init(const KArgs& a, int b, int h, int tile, int wave) {
    const int lane = threadIdx.x & 63;
    const int lq = lane & 31;
    eq_i = 0; ekp = nullptr; ksum = nullptr;
    w_lo = 0; w_hi = -1; w_glob = 1; g_lo = 0; g_hi = -1; g_glob = 1;
    g_kfirst = 0; g_klast = 0x3fffffff;
    gp = DOC ? 0 : a.gap;
    int posc;   // r of this lane's row, 0 if none
    rb = wave; sub = 0; halved = false;
    if (!DOC) {
      const int m0 = tile * 128;
      if (a.M - m0 <= 64 && a.bmask == nullptr) { halved = true; rb = wave & 1; sub = wave >> 1; }
      const int mw = m0 + rb * 32;
      row = mw + lq < a.M ? mw + lq : -1;
      w_rmin = mw; w_rmax = min(mw + 31, a.M - 1);
      if (w_rmax < w_rmin) w_rmax = -1;
      g_rmin = m0; g_rmax = min(m0 + 127, a.M - 1);
      posc = row >= 0 ? row : 0;
    } else {
      ekp = a.ek32 + b * a.ek_bs + h * a.ek_hs;
      ksum = a.ksum + b * a.ks_bs + h * a.ks_hs;
      const IdSummary* qs = a.qsum + b * a.qs_bs + h * a.qs_hs + 2 * tile;
      const IdSummary s0 = qs[0], s1 = qs[1];
      // (the rows of a tile sit at its front: padding only follows the last local and the last global row)
      if (s0.nvalid + s1.nvalid <= 64) { halved = true; rb = wave & 1; sub = wave >> 1; }
      const int64_t pos = b * a.pm_bs + h * a.pm_hs + tile * 128 + rb * 32 + lq;
      row = a.perm[pos];     // issued together with the summaries: no dependent load chain
      eq_i = a.peq[pos];
      const int ps = a.ppos[pos];
      if (s0.nvalid + s1.nvalid == 0) {  // no rows: every decision below says "skip"
        row = -1; rowc = 0; eq_i = 0; w_rmin = 0x7fffffff; w_rmax = -1; w_glob = 0;
        g_lo = 0x7fffffff; g_hi = (int)0x80000000; g_glob = 0; g_rmin = 0x7fffffff; g_rmax = -1;
        return false;
      }
      g_lo = min(s0.lo, s1.lo); g_hi = max(s0.hi, s1.hi); g_glob = s0.glob | s1.glob;
      g_rmin = min(s0.rmin, s1.rmin); g_rmax = max(s0.rmax, s1.rmax);
      g_kfirst = min(s0.kfirst, s1.kfirst); g_klast = max(s0.klast, s1.klast);
      const bool local = (eq_i < 0) && (row >= 0);
      int lo = local ? eq_i : 0x7fffffff, hi = local ? eq_i : (int)0x80000000;
      int rmin = row >= 0 ? ps : 0x7fffffff, rmax = row >= 0 ? ps : -1;
      posc = row >= 0 ? ps : 0;
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
    lim_i = CAUSAL ? min(max(gp + posc, a.pfx_m1), a.N - 1) : a.N - 1;
    w_limmin = CAUSAL ? min(max(gp + w_rmin, a.pfx_m1), a.N - 1) : a.N - 1;
    low_i = CAUSAL ? gp + posc - a.win + 1 : -0x3fffffff;
    w_lowmin = CAUSAL && w_rmax >= 0 ? gp + w_rmin - a.win + 1 : -0x3fffffff;
    w_lowmax = CAUSAL && w_rmax >= 0 ? gp + w_rmax - a.win + 1 : -0x3fffffff;
    glob_i = eq_i >= 0;
    return true;
  }
  // range [first, last) of 64-key tiles the workgroup has to look at
  FA_DEV int first_tile(const KArgs& a) const {
    const int f = g_kfirst < 0x3fffffff ? g_kfirst : 0;
    return CAUSAL && g_rmax >= 0 ? max(f, max(0, gp + g_rmin - a.win + 1) / 64) : f;   // sliding window
  }
  FA_DEV int last_tile(const KArgs& a) const {
    const int hi_key = CAUSAL ? min(a.N, max(gp + g_rmax, a.pfx_m1) + 1) : a.N;
    return min((hi_key + 63) / 64, g_klast + 1);
  }

  // Wave-level decisions (TF_ bits) for the key tile n0 .. n0+BN-1 whose ids span [k_lo, k_hi]:
  //   TF_SKIP : no (row, key) pair of the wave's rows is kept
  //   TF_LIM  : some pair fails the causal / length limit  -> mask_lim
  //   TF_DOC  : some pair may fail the id test             -> mask_doc
  FA_DEV int decide(const KArgs& a, int n0, int BN, int k_lo, int k_hi) const {
    bool skip = (w_rmax < 0) || (CAUSAL && (n0 > max(gp + w_rmax, a.pfx_m1) || n0 + BN - 1 < w_lowmin));
    const bool need_lim = n0 + BN - 1 > w_limmin || n0 < w_lowmax;
    bool need_doc = false;
    if (DOC) {
      skip = skip || !doc_may_keep(w_lo, w_hi, w_glob, k_lo, k_hi);
      need_doc = !doc_all_keep(w_lo, w_hi, k_lo, k_hi);
    }
    return (skip ? TF_SKIP : 0) | (need_lim ? TF_LIM : 0) | (need_doc ? TF_DOC : 0);
  }
};

// Element masks of one 32-key block held in the transposed-score layout: register 4*q4 + t of a
// lane is key 8*q4 + 4*(lane >> 5) + t of the block.  Both are called under wave-uniform branches.
//   rel    : (last key the lane's row may see) - (first key of the block) - 4*(lane >> 5)
//   rel_lo : (first key the lane's row may see) - (first key of the block) - 4*(lane >> 5); both
//            bounds in one unsigned compare (rel_lo is very negative without a sliding window)
FA_DEV void mask_lim(f32x16& s, int rel, int rel_lo, float fill) {
  const bool none = rel < rel_lo;   // empty interval: nothing may pass
  const unsigned span = none ? 0u : (unsigned)(rel - rel_lo);
  if (none) rel_lo = 0x3fffffff;
#pragma unroll
  for (int q4 = 0; q4 < 4; ++q4)
#pragma unroll
    for (int t = 0; t < 4; ++t) s[4 * q4 + t] = ((unsigned)(8 * q4 + t - rel_lo) <= span) ? s[4 * q4 + t] : fill;
}
//   ids  : LDS copy of the block's 32 key ids, already offset by 16*(lane >> 5) bytes
// The four id vectors are requested together (one LDS round trip instead of four serial ones:
// left alone, the compiler reuses one register quad and waits after every read).
FA_DEV void mask_doc(f32x16& s, const char* ids, int eq_i, bool glob_i, float fill) {
  i32x4 ekv[4];
#pragma unroll
  for (int q4 = 0; q4 < 4; ++q4) ekv[q4] = *reinterpret_cast<const i32x4*>(ids + 32 * q4);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int q4 = 0; q4 < 4; ++q4) {
#pragma unroll
    for (int t = 0; t < 4; ++t) s[4 * q4 + t] = (glob_i || ekv[q4][t] == eq_i) ? s[4 * q4 + t] : fill;
  }
}

// Block mask seen from a 128-row query tile of the forward / dq kernels (natural row order): the two
// rows of 64 x 64 blocks the tile covers.  flags(t) are the TF_ bits the mask adds for key tile t
// (64 keys = one block column): TF_SKIP when the block of this wave's rows is off, TF_NONE when
// both are.  A wave's 32 rows and a tile's 64 keys lie inside one block, so no element mask is needed.
struct QBlockMask {
  const unsigned char* r0;   // null: no block mask
  const unsigned char* r1;   // null: the tile's second half lies past the last row
  int ncol;
  FA_DEV void init(const KArgs& a, int b, int h, int tile) {
    r0 = r1 = nullptr; ncol = a.nBc;
    if (a.bmask == nullptr) return;
    const unsigned char* base = a.bmask + b * a.bm_bs + h * a.bm_hs;
    r0 = base + int64_t(2 * tile) * a.bm_rs;
    if (2 * tile + 1 < a.nBr) r1 = base + int64_t(2 * tile + 1) * a.bm_rs;
  }
  FA_DEV int flags(int t) const {
    if (r0 == nullptr) return 0;
    const bool in = t < ncol;
    const unsigned b0 = in ? r0[t] : 0u, b1 = (in && r1 != nullptr) ? r1[t] : 0u;
    const unsigned mine = (threadIdx.x >> 7) ? b1 : b0;   // waves 0, 1: first half; waves 2, 3: second half
    return (mine == 0 ? TF_SKIP : 0) | ((b0 | b1) == 0 ? TF_NONE : 0);
  }
};

// ---------------------------------------------------------------------------
// Work assignment of one workgroup of the forward / dq kernels, including the split of the
// key range of global-row tiles (SplitCfg, fa_common.h).
//   slots [0, nE)          : chunks 1 .. split_k-1 of the first split_tiles global-row tiles
//   slots [nE, nE + nQt)   : every tile, last tile first (chunk 0 when the tile is split)
// ---------------------------------------------------------------------------
// Extra workgroup slots per (batch, head): chunks 1 .. split_k-1 of every splittable tile.
FA_HD int split_extra(const KArgs& a) { return a.split_tiles * (a.split_k - 1); }

struct QWork {
  int tile;    // 128-row tile (natural order, or permuted order with ids)
  int gt;      // index among the splittable global-row tiles, or -1
  int split;   // chunk of the key range handled by this workgroup
};

// The header of the (batch, head) is requested by the caller before this call and, for the common
// slots [nE, ...), not looked at until q_work_finish: the tile's own summaries and row indices are
// requested in between, so the two loads overlap instead of forming a dependent chain.
constexpr int kGtPending = -2;
template <bool DOC>
FA_DEV bool q_work(const KArgs& a, const QHeader& hd, int nQt, int slot, QWork& w) {
  if (!DOC) { w.tile = nQt - 1 - slot; w.gt = -1; w.split = 0; return true; }
  const int nE = split_extra(a);
  if (slot < nE) {
    const int g0 = hd.nLp / 128;   // first global-row tile
    w.gt = slot / (a.split_k - 1);
    w.split = 1 + slot % (a.split_k - 1);
    w.tile = g0 + w.gt;
    return w.tile < hd.nT128;
  }
  w.tile = nQt - 1 - (slot - nE);
  w.split = 0;
  w.gt = kGtPending;
  return true;
}
FA_DEV void q_work_finish(const KArgs& a, const QHeader& hd, QWork& w) {
  if (w.gt != kGtPending) return;
  const int g0 = hd.nLp / 128;
  w.gt = (w.tile >= g0 && w.tile - g0 < a.split_tiles) ? w.tile - g0 : -1;
}

// Cut the key-tile range [first, last) of a splittable tile into chunks; returns the number of
// chunks in use (1: not split) and narrows [first, last) to this workgroup's chunk.
FA_DEV int split_range(const KArgs& a, const QWork& w, int& first, int& last) {
  if (w.gt < 0) return 1;
  const int n = max(0, last - first);
  const int ns = min(a.split_k, max(1, n / kSplitMinTiles));
  const int c = (n + ns - 1) / ns;
  first = min(last, first + w.split * c);
  last = min(last, first + c);
  return ns;
}

// A wave's 32 result rows on their way out.  The accumulators hold a row (or key) per lane and 4 consecutive
// columns per register quad: stored from there, a wave instruction writes 64 pieces of 8 bytes, a row apart, and
// every 128-byte line of the result fills up over sixteen instructions -- measured at 5-13 % of the id
// workloads' kernel times.  So the rows pass through a patch of LDS that belongs to the wave (32 rows of
// D * 2 + 16 bytes; LDS operations of one wave execute in issue order, so no barrier sits between the writes
// and the reads) and leave as 16 bytes per lane, D / 8 lanes to a row: whole lines per instruction.
// row_ptr(r) gives the address of row r of the wave (0..31) in memory, or nullptr for a row that does not exist.
template <int D>
constexpr int row_patch_bytes() { return 32 * (D * 2 + 16); }
template <typename E, int D, int DBN, typename F>
FA_DEV void store_rows_through_lds(char* patch, const f32x16 (&v)[DBN], const float sc, F&& row_ptr) {
  using T = typename E::scalar;
  using vec8 = typename E::vec8;
  constexpr int PITCH = D * 2 + 16, CPR = D / 8, RPI = 64 / CPR, NI = 32 / RPI;
  const int lane = threadIdx.x & 63, lq = lane & 31, g = lane >> 5;
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      if (32 * db + 8 * q4 >= D) continue;  // padded columns of the D = 16 layout
      const typename E::vec2 x0 = E::cvt2(v[db][4 * q4 + 0] * sc, v[db][4 * q4 + 1] * sc);
      const typename E::vec2 x1 = E::cvt2(v[db][4 * q4 + 2] * sc, v[db][4 * q4 + 3] * sc);
      typename E::vec4 x = {x0[0], x0[1], x1[0], x1[1]};
      *reinterpret_cast<typename E::vec4*>(patch + lq * PITCH + (32 * db + 8 * q4 + 4 * g) * 2) = x;
    }
  asm volatile("" ::: "memory");   // (order only)
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int r = RPI * i + lane / CPR, cc = lane % CPR;
    const vec8 x = *reinterpret_cast<const vec8*>(patch + r * PITCH + cc * 16);
    T* p = row_ptr(r);
    // (streaming stores: no kernel of the step reads these lines again soon, and the K / V tiles that the other
    // workgroups are fetching keep their place in the L2: 1-2.5 % of the id workloads' kernel times)
    if (p != nullptr) __builtin_nontemporal_store(x, reinterpret_cast<vec8*>(p + cc * 8));
  }
  asm volatile("" ::: "memory");
}

// Partial results travel between workgroups through device-scope accesses (they pass the
// non-coherent cache levels access by access), so no cache-wide write-back or invalidate is needed.
FA_DEV void store_dev(float* p, float x0, float x1) {
  typedef unsigned long long u64;
  const u64 v = (u64)__float_as_uint(x0) | ((u64)__float_as_uint(x1) << 32);
  __hip_atomic_store(reinterpret_cast<u64*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 bytes with the same cache policy as the 8-byte device-scope store above (the `sc1` bit); not atomic as
// a whole, which the partial results do not need: they are read after the arrival counter says so.
// The wait states behind it are part of the instruction as far as this code is concerned: a vector instruction that
// writes the data registers of a store wider than 8 bytes must not follow it directly, and the compiler, which
// keeps that distance for its own stores, does not look inside inline assembly (it placed an address computation
// into the first data register right behind the store).
FA_DEV void store_dev(float* p, f32x4 x) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" :: "v"(p), "v"(x) : "memory");
}
// A partial [128 rows x D] fp32 tile lies in the scratch in the accumulator order of the waves that own the
// rows, not row by row: float4 number i = (rb * (D / 8) + grp) * 64 + lane holds the columns 8 * grp +
// 4 * (lane >> 5) .. + 3 of row 32 * rb + (lane & 31).  A wave's store instruction then writes 1 KB in one
// piece (row by row it was 64 pieces of 16 bytes), and the merging workgroup reads float4 i with thread i.
template <int D>
FA_DEV int part_index(int rb, int grp, int lane) { return (rb * (D / 8) + grp) * 64 + lane; }
template <int D>
FA_DEV void part_coords(int i, int& r, int& c) {   // row of the tile and float4 of that row
  const int rbq = i >> 6, lane = i & 63, rb = rbq / (D / 8), grp = rbq % (D / 8);
  r = rb * 32 + (lane & 31);
  c = 2 * grp + (lane >> 5);
}
FA_DEV void load_dev(const float* p, float& x0, float& x1) {
  typedef unsigned long long u64;
  const u64 v = __hip_atomic_load(reinterpret_cast<const u64*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  x0 = __uint_as_float((unsigned)v);
  x1 = __uint_as_float((unsigned)(v >> 32));
}
FA_DEV f32x4 load_dev4(const float* p) {
  float a, b, c, d;
  load_dev(p, a, b);
  load_dev(p + 2, c, d);
  const f32x4 x = {a, b, c, d};
  return x;
}

// Arrival protocol of the chunks of one tile: every workgroup calls this after it has issued the
// stores of its partial result (store_dev); returns true in exactly one of them, the last to
// arrive, which then merges (load_dev).
FA_DEV bool split_arrive(int* counter, int nsplit) {
  __shared__ int sk_last;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's partial stores have landed
  __syncthreads();
  if (threadIdx.x == 0) {
    const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sk_last = (old == nsplit - 1) ? 1 : 0;
    // ready for the next kernel that uses the same scratch
    if (sk_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  return sk_last != 0;
}

// Which leading keys of (batch b, key head hk) the column kernel of dk/dv takes (see kGcolTilesMax): `ncols`
// keys, a multiple of 128 (0: none), seen by `tiles` 64-row tiles of global rows in all.  Both kernels of a
// launch evaluate this, so the key range is cut in the same place.
struct GcolInfo { int ncols, tiles; };
FA_DEV GcolInfo gcol_info(const KArgs& a, int b, int hk) {
  int k0 = 0x7fffffff, tiles = 0;
  for (int gi = 0; gi < a.G; ++gi) {
    const QHeader hd = a.qhdr[b * a.qh_bs + (hk * a.G + gi) * a.qh_hs];
    k0 = min(k0, hd.k0);
    tiles += (hd.nG + 63) / 64;
  }
  GcolInfo r;
  r.tiles = tiles;
  r.ncols = k0 >= a.nKs ? (a.N + 127) / 128 * 128 : (k0 * kSumRows) / 128 * 128;
  if (tiles > kGcolTilesMax) r.ncols = 0;
  return r;
}

// blockIdx -> (tile, batch*head) for grids of `ntile` tiles per (batch, head); grid_blocks() is the
// matching grid size.  Consecutive workgroup ids land on different XCDs (8 of them, each with its
// own L2), so the map decides which XCD's L2 sees which head:
//   BH a multiple of 8 : every XCD is given whole heads (its L2 keeps that head's K/V or Q/dO).
//        Inside an XCD the order is
//          head-major (tile_major = false): one head after the other -- best L2 reuse when every
//               tile streams most of the head (no ids);
//          tile-major (tile_major = true): tile slot 0 of all the XCD's heads, then slot 1, ... --
//               with ids the few heavy tiles (global rows) of EVERY head start at once instead of
//               queueing behind the light tiles of the heads before them.
//   BH = 1, 2, 4      : a head is shared by 8 / BH XCDs, its tile slots dealt round-robin among them
//                       (heavy and light slots alternate, so the XCDs stay balanced).
//   otherwise          : (slot, head) pairs dealt round-robin over the XCDs, slot-major: balanced for
//                       any BH, at the price of every L2 seeing every head.
// Returns false for padding ids.
FA_HD int grid_blocks(int ntile, int BH) {
  if (BH % 8 == 0) return BH * ntile;
  if (BH < 8 && 8 % BH == 0) { const int k = 8 / BH; return 8 * ((ntile + k - 1) / k); }
  return (BH * ntile + 7) / 8 * 8;
}

// bid: index of the workgroup (blockIdx.x, unless several forms share one grid).
FA_DEV bool block_to_tile(int ntile, int BH, bool tile_major, int& tile_slot, int& bh, int bid) {
  const int xcd = bid & 7, idx = bid >> 3;
  if (BH % 8 == 0) {
    const int heads = BH / 8;  // heads per XCD
    if (tile_major) {
      bh = (idx % heads) * 8 + xcd;
      tile_slot = idx / heads;
    } else {
      bh = (idx / ntile) * 8 + xcd;
      tile_slot = idx % ntile;
    }
    return true;
  }
  if (BH < 8 && 8 % BH == 0) {
    const int k = 8 / BH;
    bh = xcd / k;
    tile_slot = idx * k + xcd % k;
    return tile_slot < ntile;
  }
  tile_slot = bid / BH;
  bh = bid % BH;
  return tile_slot < ntile;
}
FA_DEV bool block_to_tile(int ntile, int BH, bool tile_major, int& tile_slot, int& bh) {
  return block_to_tile(ntile, BH, tile_major, tile_slot, bh, (int)blockIdx.x);
}

}  // namespace fa
