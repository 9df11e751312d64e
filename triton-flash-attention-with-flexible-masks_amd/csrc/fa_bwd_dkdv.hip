// dK/dV kernel of the split backward.  Replaces _bwd_kv_kernel of the reference
// (flash_triton.py:175-321).
//
// One workgroup = 128 keys (64 in the role-split form with document ids, two workgroups per CU).
// D = 128: two waves per 32 keys; they share a SIMD, own the SAME 32 keys and split the work by role, so that each needs only one operand fragment set and one accumulator
// set (two waves per SIMD fit in the register file, and one role's vector work overlaps the
// other role's matrix work):
//   role 0 ("score" wave)                       role 1 ("gradient" wave)
//   S  = Q K^T      A = Q rows, B = K^T (regs)  dP = dO V^T     A = dO rows, B = V^T (regs)
//   P  = exp2(S*c - L), masked -> 0             ---------------- barrier ----------------
//   P (rounded) -> LDS                          dS = P * (dP - delta)      (P read from LDS)
//   dV^T += dO^T P  A = dO^T (transposed read)  dK^T += Q^T dS  A = Q^T (transposed read)
// (flash_triton.py:265-308; dK is scaled by sm_scale at the end, :313).  In the accumulator
// layout each lane owns ONE key column and 16 query rows of every 32-row block, so LSE / delta /
// eq / row index are read as broadcast 16-byte LDS loads, and P travels between the two roles in
// exactly the register layout both of them use.  D <= 64: 4 waves, each doing both roles in turn.
// Query-side tiles (Q, dO, LSE, delta, eq, row index; 64 rows) are streamed through LDS, two
// buffers.  With document ids the query side is walked in the permuted (local rows first) order
// of the mask plan: tiles are gathered row by row through the permutation (row indices fetched
// one tile ahead), and only tiles whose id interval and row range can meet this workgroup's keys
// are visited.  The query heads of a grouped-query group are walked inside the kernel, so dK, dV
// are written once, already summed (the reference sums afterwards, flash_triton.py:635-637).
#include "fa_tile.h"

namespace fa {

// Operand fragments requested ahead of the MFMA that consumes them, in program order (measured
// optimum of a sweep over 2..6): row-wise reads of the first products, transposed reads of the second.
constexpr int kKvPre = 4;
constexpr int kKvPre2 = 3;

constexpr int kColsRun = 8;   // key tiles per workgroup when the column form shares the launch

// SPLIT = true : two waves per block of 32 keys, NKB key blocks per workgroup, roles split over the
//                wave pairs as described above (D = 128: one wave cannot hold both operand sets and
//                both accumulator sets next to a second wave on its SIMD).
// SPLIT = false: 4 waves, every wave does both roles for its 32 keys (D <= 64: everything fits), so P
//                never leaves the registers and the only barrier is the one of the tile stream; two
//                workgroups share a CU.
// Pair waits that expired (role-split form) since the library was loaded, per device: the NaN a wave writes
// into its dK rows says where, this says that it happened at all (fa_pair_wait_expired).
__device__ unsigned long long g_pair_expired = 0;

#ifdef FA_TRACE
// words: 0 start, 1 shader clocks the first gradient wave waited for P (role-split form), 2 first query tile chosen, 3 first query tile in LDS, 4 after the tile loop, 5 end, 6 query tiles computed, 7 key tile | (batch, kv head) << 16 (-1: left at once)
FA_TRACE_ARRAY(g_trace_dkdv);
#endif

}  // namespace fa
#include "fa_dkdv_cols.h"   // the column form; its workgroups stamp the same array: 0 start, 3 tiles resident, 4 after the key loop, 5 end, 6 key blocks of wave 0, 7 chunk | 1 << 40
namespace fa {

// COLS = true : the grid carries, behind the workgroups of this form, those of the column form
//                (fa_dkdv_cols.h) for the leading key columns that only a few global rows see; the workgroups
//                of this form whose keys lie there leave at once.  One launch, so the column form's memory
//                traffic overlaps the set-up latencies of this one.
template <typename Tag, int D, bool CAUSAL, bool DOC, bool SPLIT, int NKB, bool COLS>
__global__ __launch_bounds__(SPLIT ? 128 * NKB : 64 * NKB)
__attribute__((amdgpu_waves_per_eu((D <= 32 && !COLS) ? 3 : 2, (D <= 32 && !COLS) ? 3 : 2)))
void bwd_dkdv_kernel(const KArgs a) {
  using E = Elem<Tag>;
  using T = typename E::scalar;
  using vec8 = typename E::vec8;
  constexpr int BK = 32 * NKB, BQ = 64, KS = D / 16;
  constexpr int DL = D < 32 ? 32 : D;  // LDS row width: D = 16 is staged as 32 columns, the upper 16 zero
  constexpr int DBN = DL / 32;
  constexpr int TILE_BYTES = BQ * DL * 2;
  constexpr int AUX_OFF = 4 * TILE_BYTES;      // [2 buffers][4 arrays][64] x 4 bytes
  constexpr int AUX_BYTES = 1024;
  constexpr int P_OFF = AUX_OFF + 2 * AUX_BYTES;  // [2 (block parity)][NKB key blocks][2 x 1024]: P as fp16
  constexpr int P_BYTES = 2048;
  constexpr int FLAG_OFF = P_OFF + 2 * NKB * P_BYTES;   // [2 (block parity)][NKB] sequence numbers of the published P
  // Polls of the pair flag before the gradient wave gives up (kPairSpinDefault, about a millisecond:
  // orders of magnitude above a legitimate wait; 0 with FA_FLAG_DEBUG_NO_PAIR_WAIT).  A wave that
  // gave up has used a P it cannot trust: it says so by writing NaN into its dK rows at the end.
  const int pair_spin_max = a.pair_spin;
  int pair_lost = 0;
  constexpr int NW = SPLIT ? 2 * NKB : NKB;
  static_assert(NW >= 4, "the four auxiliary arrays of a tile are loaded by waves 0..3");
  using Loader = TileLoader<DL, BQ, D, NW>;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int nKt = (a.N + BK - 1) / BK;
  // With the column form in the launch, most key tiles of this form may have nothing to do here (their keys
  // belong to the column form): a workgroup then takes kColsRun key tiles, nSlots tiles apart, and steps over
  // those -- a workgroup that only finds out that it is not needed costs the dispatcher as much as a short
  // useful one (8192 of them: 50 us), a skipped tile of a run costs a comparison.
  const int nSlots = COLS ? (nKt + kColsRun - 1) / kColsRun : nKt;
  int bid = (int)blockIdx.x;   // index of the workgroup among those of its form
  if constexpr (COLS) {
    static_assert(DOC && (SPLIT ? 128 * NKB : 64 * NKB) == 256, "the column form runs with ids, 4 waves per workgroup");
    // the column form's workgroups come first: few, long, one round of them
    const int nC = dkdv_cols_blocks(a);
    const bool cols = bid < nC;
    if (!cols) bid -= nC;
    if (cols) { dkdv_cols_body<Tag, D, CAUSAL>(a, bid, smem); return; }
  }

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar
  const int role = SPLIT ? wave / NKB : 0, kb = wave % NKB;
  const int lq = lane & 31, g = lane >> 5;
  FA_STAMP(g_trace_dkdv, 0, FA_CLOCK()); FA_STAMP(g_trace_dkdv, 5, 0); FA_STAMP(g_trace_dkdv, 7, -1);
  FA_TRACE_ONLY(int tr_tiles = 0; bool tr_first = false; long long tr_wait = 0;)

  // one workgroup per (key tile, batch, kv head) -- or per run of key tiles, see above
  int kt0, bhk;
  if (!block_to_tile(nSlots, a.B * a.Hk, false, kt0, bhk, bid)) return;  // causal: the first key tiles see the most rows
  const int b = bhk / a.Hk, hk = bhk % a.Hk;
  const int ncols = COLS ? gcol_info(a, b, hk).ncols : 0;   // leading keys that belong to the column form of this launch
  bool ran = false;
  for (int rr = 0; rr < (COLS ? kColsRun : 1); ++rr) {
  const int kt = kt0 + rr * nSlots;
  const int n0 = kt * BK;
  if (COLS && (kt >= nKt || n0 + BK <= ncols)) continue;
  if (COLS && ran) __syncthreads();   // the previous key tile's last reads of LDS are done
  ran = true;
  pair_lost = 0;
  const int nw = n0 + kb * 32;
  const int key = nw + lq;
  const int keyc = key < a.N ? key : a.N - 1;

  // B operand held for the whole kernel: K^T for the score wave, V^T for the gradient wave.
  // Lane holds d = 16*ks + 8*g .. +7 of its key row.
  const T* srcp = role == 0 ? reinterpret_cast<const T*>(a.k) + b * a.k_bs + hk * a.k_hs + int64_t(keyc) * a.k_rs
                            : reinterpret_cast<const T*>(a.v) + b * a.v_bs + hk * a.v_hs + int64_t(keyc) * a.v_rs;
  vec8 frag[KS];
  vec8 frag2[KS];   // V^T next to K^T when one wave does both roles
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) frag[ks] = *reinterpret_cast<const vec8*>(srcp + ks * 16 + g * 8);
  if (!SPLIT) {
    const T* vsrc = reinterpret_cast<const T*>(a.v) + b * a.v_bs + hk * a.v_hs + int64_t(keyc) * a.v_rs;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) frag2[ks] = *reinterpret_cast<const vec8*>(vsrc + ks * 16 + g * 8);
  }
  // Where to wait for these fragments.  The 64-key role-split form serves short tile streams: only
  // right before the tile loop, so that the set-up below overlaps their flight (3 % of the kernel at
  // 16 query tiles per workgroup, under 1 % at a dozen).  The other forms wait here: for the
  // 128-key form, which serves long streams, that gave the faster loop (4.24 against 4.39 ms, plain
  // causal 16K); at D <= 64 the difference stayed inside the run-to-run spread.
  constexpr bool LATE_SETTLE = SPLIT && NKB == 2;
  FA_STAMP(g_trace_dkdv, 1, 0); FA_STAMP(g_trace_dkdv, 7, (long long)kt | ((long long)bhk << 16));
  if (!LATE_SETTLE) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { settle(frag[ks]); if (!SPLIT) settle(frag2[ks]); }
  }
  const float c = a.scale_log2e;
  // rows that may see this lane's key: [row_lo, row_lo + row_span)
  // (causal: from the diagonal on, or from row 0 for a key of the prefix; sliding window: `win` rows)
  // Without ids a row is named by its index r and its diagonal sits at key gap + r; with ids rows are
  // named by the diagonal position the mask plan stored for them (gap + row, or the caller's per-row
  // position), so the offset is 0 and the names run up to kPosMax.
  const int gk = DOC ? 0 : a.gap;
  const int rcap = DOC ? kPosMax : a.M - 1;
  const int row_lo = CAUSAL ? (key <= a.pfx_m1 ? 0 : max(0, key - gk)) : 0;
  const int row_hi = CAUSAL ? min(rcap, key - gk + a.win - 1) : rcap;
  const unsigned row_span = (key < a.N && row_hi >= row_lo) ? (unsigned)(row_hi - row_lo + 1) : 0u;

  // per query head state (set at the top of the head loop)
  const float* lsep = nullptr;
  const float* delp = nullptr;
  int ek_j = 0;
  int wk_lo = 0, wk_hi = 0;   // id interval of this wave's 32 keys
  const int* eqp = nullptr;
  const int* pmp = nullptr;
  const int* ppp = nullptr;   // diagonal positions in the permuted order
  const IdSummary* qsum = nullptr;

  Loader ldQ, ldO;
  LdsOffsets<DL> lo;
  lo.init();
  // gathered loads: byte offset of the lane's chunk inside its row, and the tile rows it fetches
  int g_coff[Loader::PER], g_rit[Loader::PER];
#pragma unroll
  for (int i = 0; i < Loader::PER; ++i) {
    g_rit[i] = ((i * NW + wave) * Loader::RPI + lane / Loader::CPR) % BQ;
    const int gc = (lane % Loader::CPR) ^ swz<DL, SWZ_ROW>(g_rit[i]);
    g_coff[i] = gc < D / 8 ? gc * 16 : kOobOffset;
  }

  // dV^T (score wave) or dK^T (gradient wave): lane = key column, registers = d rows
  // (one wave doing both roles: acc = dV^T, acc2 = dK^T)
  f32x16 acc[DBN], acc2[DBN];
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc[db][r] = 0.f; acc2[db][r] = 0.f; }

  // row indices of a permuted tile this lane needs: PER tile rows for Q/dO, one for the aux arrays
  int ri_t[Loader::PER] = {};
  int ri_aux = 0;
  auto fetch_idx = [&](int tile) {
#pragma unroll
    for (int i = 0; i < Loader::PER; ++i) ri_t[i] = pmp[tile * BQ + g_rit[i]];
    ri_aux = pmp[tile * BQ + lane];
  };
  auto load_tile = [&](int tile, int bufi) {
    const char* aux = smem + AUX_OFF + bufi * AUX_BYTES;
    if (!DOC) {
      const int m0 = tile * BQ;
      ldQ.issue(m0, smem + bufi * TILE_BYTES);
      ldO.issue(m0, smem + (2 + bufi) * TILE_BYTES);
      const int r = m0 + lane < a.M ? m0 + lane : a.M - 1;
      if (wave == 0) glb_load_lds4(lsep + r, aux);
      if (wave == 1) glb_load_lds4(delp + r, aux + 256);
    } else {
      // The row indices were fetched a tile ago and have arrived (the caller waited for every
      // outstanding load before the barrier).  Tell the compiler so here: the wait it would place
      // at their first use would otherwise land between / behind the asynchronous loads issued
      // below and, counting in order, would wait for THOSE as well.
#pragma unroll
      for (int i = 0; i < Loader::PER; ++i) settle(ri_t[i]);
      settle(ri_aux);
#pragma unroll
      for (int i = 0; i < Loader::PER; ++i) {
        if (Loader::NI % NW == 0 || i * NW + wave < Loader::NI) {
          const int r = ri_t[i] >= 0 ? ri_t[i] : 0;
          buf_load_lds16(ldQ.rsrc, smem + bufi * TILE_BYTES + (i * NW + wave) * 1024, r * ldQ.row_bytes + g_coff[i], 0);
          buf_load_lds16(ldO.rsrc, smem + (2 + bufi) * TILE_BYTES + (i * NW + wave) * 1024, r * ldO.row_bytes + g_coff[i], 0);
        }
      }
      const int r = ri_aux >= 0 ? ri_aux : 0;
      if (wave == 0) glb_load_lds4(lsep + r, aux);
      if (wave == 1) glb_load_lds4(delp + r, aux + 256);
      if (wave == 2) glb_load_lds4(eqp + r, aux + 512);
      if (wave == 3) glb_load_lds4(ppp + tile * BQ + lane, aux + 768);
    }
  };

  int pair_seq = 0;   // non-skipped tiles so far: identical in the two waves of a pair
  if (SPLIT && threadIdx.x < 2 * NKB) *reinterpret_cast<int*>(smem + FLAG_OFF + threadIdx.x * 4) = 0;  // visible after the first tile's barrier
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // Masks on P of one 32-row block (lane = key column, register 4*q4 + t = row 8*q4 + 4*g + t of the
  // block); every part sits under a wave-uniform branch.
  auto mask_p = [&](f32x16& x, const int qb, const int flags, const int tile_id, const int m0, const char* aux)
                    __attribute__((always_inline)) {
    const bool need_lim = (flags & TF_LIM) != 0, need_doc = (flags & TF_DOC) != 0, has_glob = (flags & TF_GLOB) != 0;
    if (need_lim) {
      // row name (index, or diagonal position with ids) inside [first that may see this key, last]; padding rows are -1.  The four index
      // vectors are requested together: one LDS round trip instead of four serial ones.
      asm volatile("" ::: "memory");  // keep this a real (wave-uniform) branch: never if-converted
      i32x4 rowv[4];
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int i0 = 32 * qb + 8 * q4 + 4 * g;
        if (DOC) rowv[q4] = *reinterpret_cast<const i32x4*>(aux + 768 + i0 * 4);
        else rowv[q4] = i32x4{m0 + i0, m0 + i0 + 1, m0 + i0 + 2, m0 + i0 + 3};
      }
      if (DOC) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          x[4 * q4 + t] = (unsigned)(rowv[q4][t] - row_lo) < row_span ? x[4 * q4 + t] : 0.f;
    }
    if (DOC && (flags & TF_COL)) {
      // every row of the tile carries the same local id: the id test depends on the key alone,
      // i.e. on the lane -- whole columns of the block are kept or dropped
      asm volatile("" ::: "memory");
      const bool col_keep = ek_j == tile_id;
#pragma unroll
      for (int r = 0; r < 16; ++r) x[r] = col_keep ? x[r] : 0.f;
    }
    if (DOC && need_doc) {
      asm volatile("" ::: "memory");
      i32x4 eqv[4];
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) eqv[q4] = *reinterpret_cast<const i32x4*>(aux + 512 + (32 * qb + 8 * q4 + 4 * g) * 4);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        if (!has_glob) {
#pragma unroll
          for (int t = 0; t < 4; ++t) x[4 * q4 + t] = eqv[q4][t] == ek_j ? x[4 * q4 + t] : 0.f;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) x[4 * q4 + t] = (eqv[q4][t] >= 0 || eqv[q4][t] == ek_j) ? x[4 * q4 + t] : 0.f;
        }
      }
    }
  };

  // One query tile, D > 64 (BUF is a compile-time constant so every LDS address is base + immediate).
  // The two roles are synchronised pairwise, not by workgroup barriers: the
  // score wave publishes P of a 32-row block in LDS and then a sequence number; the gradient wave of
  // the pair polls that number.  LDS operations of one wave are executed in issue order, so the
  // number is never visible before P.  Waves of different key blocks drift apart inside a tile
  // (LDS-heavy and MFMA-heavy phases of different waves overlap); the gradient wave computes dP of
  // both blocks before it needs the first P.  The wait is bounded, so every wave reaches the end
  // of the kernel whatever happens.
  auto compute_flag = [&](const int BUF, const int cur, const int flags, const int tile_id) __attribute__((always_inline)) {
    const char* lqt = smem + BUF * TILE_BYTES;
    const char* ldo = smem + (2 + BUF) * TILE_BYTES;
    const char* aux = smem + AUX_OFF + BUF * AUX_BYTES;
    const int m0 = cur * BQ;  // natural order only
    if (flags & TF_SKIP) return;   // decided per wave pair: both roles agree
    ++pair_seq;
    auto first_product = [&](const char* rows, const int qb) __attribute__((always_inline)) {
      f32x16 x = zero;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const vec8 ra = lds_row8<E>(rows + lo.row[ks] + qb * 32 * DL * 2);
        x = E::mfma32(ra, frag[ks], x);
      }
      {
        constexpr int PRE = KS < kKvPre ? KS : kKvPre;
        __builtin_amdgcn_sched_group_barrier(0x100, PRE, 0);
#pragma unroll
        for (int i = 0; i < KS - PRE; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, PRE, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      return x;
    };
    auto second_product = [&](const char* tr, const vec8 (&yf)[2], const int qb) __attribute__((always_inline)) {
      // NM transposed fragments (two LDS reads each), requested PRE fragments ahead of their MFMA
      // in program order
      constexpr int NM = 2 * DBN, PRE = NM < kKvPre2 ? NM : kKvPre2;
      auto fetch = [&](const int i) __attribute__((always_inline)) {
        const int half = i / DBN, db = i % DBN;
        const int goff = (2 * qb + half) * 16 * DL * 2;
        return lds_tr8<E>(tr + lo.tr[db][0] + goff, tr + lo.tr[db][1] + goff);
      };
      __builtin_amdgcn_sched_barrier(0);
      vec8 tf[NM];
#pragma unroll
      for (int i = 0; i < PRE; ++i) tf[i] = fetch(i);
#pragma unroll
      for (int i = 0; i < NM; ++i) {
        if (i + PRE < NM) tf[i + PRE] = fetch(i + PRE);
        __builtin_amdgcn_sched_barrier(0);
        acc[i % DBN] = E::mfma32(tf[i], yf[i / DBN], acc[i % DBN]);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // Both roles run the same MFMA streams (the accumulators never cross a role branch):
    //   first(0) | score: P0 -> LDS | first(1) | score: P1 -> LDS | gradient: dS0 | second(0) | gradient: dS1 | second(1)
    // so the gradient wave's first product of block 1 falls into the score wave's exponentials and
    // the score wave's second products into the gradient wave's waits.  (Running dV0 before exp1 in
    // the score wave, or dS1 before dK0 in the gradient wave, measured the same or slightly worse.)
    const char* rows = role == 0 ? lqt : ldo;   // rows operand of the first product
    const char* trp = role == 0 ? ldo : lqt;    // transposed operand of the second product
    f32x16 x[2];
    vec8 yf[2][2];   // P (score wave) or dS (gradient wave) per block, rounded to the element type
    f32x4 Lv[2][4];  // LSE of this lane's 16 query rows of a block (row 8*q4 + 4*g + t)
    // requested ahead of the product so that the LDS round trip is hidden
    auto lse_load = [&](const int qb) __attribute__((always_inline)) {
      if (role == 0) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) Lv[qb][q4] = *reinterpret_cast<const f32x4*>(aux + (32 * qb + 8 * q4 + 4 * g) * 4);
      }
    };
    auto score_part = [&](const int qb) __attribute__((always_inline)) {   // S -> P, published
      if (role != 0) return;
      char* pbuf = smem + P_OFF + (qb * NKB + kb) * P_BYTES + lane * 16;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
#pragma unroll
        for (int t = 0; t < 4; ++t) x[qb][4 * q4 + t] = fast_exp2(__builtin_fmaf(x[qb][4 * q4 + t], c, -Lv[qb][q4][t]));
      }
      mask_p(x[qb], qb, flags, tile_id, m0, aux);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int t = 0; t < 8; t += 2) {
          const typename E::vec2 pr = E::cvt2(x[qb][8 * half + t], x[qb][8 * half + t + 1]);
          yf[qb][half][t] = pr[0]; yf[qb][half][t + 1] = pr[1];
        }
        // P crosses to the gradient wave as fp16 whatever the element type: P <= 1, so fp16 keeps 11
        // significant bits of it (anything below 6e-8 becomes 0, far under the rounding of dS itself) and
        // dS = P (dP - delta) is formed from a P that is as good as the fp32 one; the bf16 copy above is
        // the operand of this wave's own dV product only.
        if constexpr (sizeof(typename E::scalar) == 2 && !__is_same(typename E::scalar, _Float16)) {
          f16x8 ph;
#pragma unroll
          for (int t = 0; t < 8; t += 2) {
            const f32x2 pp = {x[qb][8 * half + t], x[qb][8 * half + t + 1]};
            const f16x2 hh = __builtin_convertvector(pp, f16x2);
            ph[t] = hh[0]; ph[t + 1] = hh[1];
          }
          *reinterpret_cast<f16x8*>(pbuf + half * 1024) = ph;
        } else {
          *reinterpret_cast<vec8*>(pbuf + half * 1024) = yf[qb][half];
        }
      }
      lds_flag_store(smem + FLAG_OFF + (qb * NKB + kb) * 4, pair_seq);
    };
    auto grad_part = [&](const int qb) __attribute__((always_inline)) {    // dS = P * (dP - delta)
      if (role != 1) return;
      const char* pbuf = smem + P_OFF + (qb * NKB + kb) * P_BYTES + lane * 16;
      // LDS round trips are long under load: delta is requested before the wait, both halves of
      // P together after it
      f32x4 dl[4];
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) dl[q4] = *reinterpret_cast<const f32x4*>(aux + 256 + (32 * qb + 8 * q4 + 4 * g) * 4);
      const char* fl = smem + FLAG_OFF + (qb * NKB + kb) * 4;
      bool arrived = false;
      FA_TRACE_ONLY(const long long tr_t0 = __builtin_readcyclecounter();)
      for (int spin = 0; spin <= pair_spin_max; ++spin) {
        if (__builtin_amdgcn_readfirstlane(lds_flag_load(fl)) == pair_seq) { arrived = true; break; }
        __builtin_amdgcn_s_sleep(1);
      }
      if (!arrived) pair_lost = 1;
      FA_TRACE_ONLY(tr_wait += __builtin_readcyclecounter() - tr_t0;)
      f16x8 pr8[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) pr8[half] = *reinterpret_cast<const f16x8*>(pbuf + half * 1024);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const f32x8 pv = __builtin_convertvector(pr8[half], f32x8);
#pragma unroll
        for (int q2 = 0; q2 < 2; ++q2) {
#pragma unroll
          for (int t = 0; t < 4; t += 2) {
            const int e = 4 * q2 + t;
            const typename E::vec2 pr = E::cvt2(pv[e] * (x[qb][8 * half + e] - dl[2 * half + q2][t]), pv[e + 1] * (x[qb][8 * half + e + 1] - dl[2 * half + q2][t + 1]));
            yf[qb][half][e] = pr[0]; yf[qb][half][e + 1] = pr[1];
          }
        }
      }
    };
    lse_load(0); x[0] = first_product(rows, 0); score_part(0);
    lse_load(1); x[1] = first_product(rows, 1); score_part(1);
    grad_part(0); second_product(trp, yf[0], 0);
    grad_part(1); second_product(trp, yf[1], 1);
  };

  // One query tile, both roles in one wave: S and dP are accumulated alternately, P and dS stay in
  // registers, then dV^T += dO^T P and dK^T += Q^T dS.
  auto compute_both = [&](const int BUF, const int cur, const int flags, const int tile_id) __attribute__((always_inline)) {
    const char* lqt = smem + BUF * TILE_BYTES;
    const char* ldo = smem + (2 + BUF) * TILE_BYTES;
    const char* aux = smem + AUX_OFF + BUF * AUX_BYTES;
    const int m0 = cur * BQ;  // natural order only
    if (flags & TF_SKIP) return;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      f32x16 x = zero, dp = zero;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const vec8 rq = lds_row8<E>(lqt + lo.row[ks] + qb * 32 * DL * 2);
        x = E::mfma32(rq, frag[ks], x);
        const vec8 ro = lds_row8<E>(ldo + lo.row[ks] + qb * 32 * DL * 2);
        dp = E::mfma32(ro, frag2[ks], dp);
      }
      {
        constexpr int NM = 2 * KS, PRE = NM < kKvPre ? NM : kKvPre;
        __builtin_amdgcn_sched_group_barrier(0x100, PRE, 0);
#pragma unroll
        for (int i = 0; i < NM - PRE; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, PRE, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // S -> P, masks, dS = P * (dP - delta) for this lane's 16 query rows of the block
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int i0 = 32 * qb + 8 * q4 + 4 * g;  // row inside the tile
        const f32x4 Lv = *reinterpret_cast<const f32x4*>(aux + i0 * 4);
#pragma unroll
        for (int t = 0; t < 4; ++t) x[4 * q4 + t] = fast_exp2(__builtin_fmaf(x[4 * q4 + t], c, -Lv[t]));
      }
      mask_p(x, qb, flags, tile_id, m0, aux);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int i0 = 32 * qb + 8 * q4 + 4 * g;
        const f32x4 dl = *reinterpret_cast<const f32x4*>(aux + 256 + i0 * 4);
#pragma unroll
        for (int t = 0; t < 4; ++t) dp[4 * q4 + t] = x[4 * q4 + t] * (dp[4 * q4 + t] - dl[t]);
      }
      // dV^T += dO^T P and dK^T += Q^T dS alternately: transposed fragments (two LDS reads each) are
      // requested PRE MFMAs ahead in program order, P and dS are converted just in time; the
      // scheduling barriers pin that order.
      {
        constexpr int NM = 4 * DBN, PRE = NM < kKvPre2 + 1 ? NM : kKvPre2 + 1;
        auto fetch = [&](const int i) __attribute__((always_inline)) {
          const int half = i / (2 * DBN), db = (i % (2 * DBN)) / 2;
          const char* t = (i & 1) ? lqt : ldo;
          const int goff = (2 * qb + half) * 16 * DL * 2;
          return lds_tr8<E>(t + lo.tr[db][0] + goff, t + lo.tr[db][1] + goff);
        };
        __builtin_amdgcn_sched_barrier(0);
        vec8 tf[NM];
#pragma unroll
        for (int i = 0; i < PRE; ++i) tf[i] = fetch(i);
        vec8 pf, dsf;
#pragma unroll
        for (int i = 0; i < NM; ++i) {
          if (i + PRE < NM) tf[i + PRE] = fetch(i + PRE);
          if (i % (2 * DBN) == 0) {
            const int half = i / (2 * DBN);
#pragma unroll
            for (int t = 0; t < 8; t += 2) {
              const typename E::vec2 pr = E::cvt2(x[8 * half + t], x[8 * half + t + 1]);
              pf[t] = pr[0]; pf[t + 1] = pr[1];
              const typename E::vec2 dr = E::cvt2(dp[8 * half + t], dp[8 * half + t + 1]);
              dsf[t] = dr[0]; dsf[t + 1] = dr[1];
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          const int db = (i % (2 * DBN)) / 2;
          if (i & 1) acc2[db] = E::mfma32(tf[i], dsf, acc2[db]);
          else acc[db] = E::mfma32(tf[i], pf, acc[db]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  auto compute = [&](const int BUF, const int cur, const int flags, const int tile_id) __attribute__((always_inline)) {
    if constexpr (SPLIT) compute_flag(BUF, cur, flags, tile_id);
    else compute_both(BUF, cur, flags, tile_id);
  };

  for (int gi = 0; gi < a.G; ++gi) {
    const int h = hk * a.G + gi;
    lsep = a.lse + (int64_t(b) * a.H + h) * a.M;
    delp = a.delta + (int64_t(b) * a.H + h) * a.M;
    ldQ.init(reinterpret_cast<const T*>(a.q) + b * a.q_bs + h * a.q_hs, a.q_rs, a.M);
    ldO.init(reinterpret_cast<const T*>(a.dout) + b * a.do_bs + h * a.do_hs, a.do_rs, a.M);
    int gk_lo = 0, gk_hi = 0;   // id interval of the workgroup's 128 keys
    int nQtiles = (a.M + BQ - 1) / BQ;
    int first = CAUSAL ? (n0 <= a.pfx_m1 ? 0 : max(0, n0 - gk) / BQ) : 0;
    // sliding window: the last row that sees a key of this workgroup
    const int wg_rhi = CAUSAL ? min(rcap, n0 + BK - 1 - gk + a.win - 1) : rcap;
    if (CAUSAL && !DOC) nQtiles = min(nQtiles, max(0, wg_rhi + 1 + BQ - 1) / BQ);
    if (DOC) {
      ek_j = a.ek32[b * a.ek_bs + h * a.ek_hs + keyc];
      eqp = a.eq32 + b * a.eq_bs + h * a.eq_hs;
      pmp = a.perm + b * a.pm_bs + h * a.pm_hs;
      ppp = a.ppos + b * a.pm_bs + h * a.pm_hs;
      qsum = a.qsum + b * a.qs_bs + h * a.qs_hs;
      const IdSummary* ks = a.ksum + b * a.ks_bs + h * a.ks_hs;
      const IdSummary s0 = ks[n0 / kSumRows];
      gk_lo = s0.lo; gk_hi = s0.hi;
      if (BK > kSumRows && n0 / kSumRows + 1 < a.nKs) {
        const IdSummary s1 = ks[n0 / kSumRows + 1];
        gk_lo = min(gk_lo, s1.lo); gk_hi = max(gk_hi, s1.hi);
      }
      const bool valid = key < a.N;
      int lo_ = valid ? ek_j : 0x7fffffff, hi_ = valid ? ek_j : (int)0x80000000;
#pragma unroll
      for (int off = 16; off >= 1; off >>= 1) {
        lo_ = min(lo_, __shfl_xor(lo_, off));
        hi_ = max(hi_, __shfl_xor(hi_, off));
      }
      wk_lo = lo_; wk_hi = hi_;
      nQtiles = a.nQs;
      first = 0;
    }
    // decisions of this wave pair (keys nw .. nw+31) for query tile t, evaluated by the lane that tests the tile
    // block mask: the byte column(s) of the workgroup's one or two 64-key blocks; a query tile is one
    // row of blocks, a wave's 32 keys lie inside one block (no element mask needed)
    const unsigned char* bmk = (!DOC && a.bmask != nullptr) ? a.bmask + b * a.bm_bs + h * a.bm_hs + n0 / 64 : nullptr;
    auto dec = [&](int t, const IdSummary& qs) {
      bool skip, lim, doc = false, glob = false, col = false, none = false;
      if (!DOC) {
        const int m0 = t * BQ;
        const int rmin = m0, rmax = min(m0 + BQ - 1, a.M - 1);
        skip = (nw >= a.N) || (CAUSAL && ((a.gap + rmax < nw && nw > a.pfx_m1) || a.gap + rmin - a.win + 1 > nw + 31));
        lim = (m0 + BQ > a.M) || (nw + 32 > a.N) ||
              (CAUSAL && ((a.gap + rmin < nw + 31 && nw + 31 > a.pfx_m1) || a.gap + rmax - a.win + 1 > nw));
        if (bmk != nullptr) {
          const bool in = t < a.nBr;
          const unsigned char* r = bmk + int64_t(t) * a.bm_rs;
          const unsigned b0 = in ? r[0] : 0u;
          const unsigned b1 = (in && BK > 64 && n0 / 64 + 1 < a.nBc) ? r[1] : 0u;
          const unsigned mine = (BK > 64 && kb >= 2) ? b1 : b0;
          skip = skip || mine == 0;
          none = (b0 | b1) == 0;
        }
      } else {
        skip = (nw >= a.N) || (CAUSAL && ((qs.rmax < nw && nw > a.pfx_m1) || qs.rmin - a.win + 1 > nw + 31)) ||
               !doc_may_keep(qs.lo, qs.hi, qs.glob, wk_lo, wk_hi);
        lim = (qs.nvalid < BQ) || (nw + 32 > a.N) ||
              (CAUSAL && ((qs.rmin < nw + 31 && nw + 31 > a.pfx_m1) || qs.rmax - a.win + 1 > nw));
        doc = !doc_all_keep(qs.lo, qs.hi, wk_lo, wk_hi);
        glob = qs.glob != 0;
        // one local id for the whole tile (padding rows aside, which the row-range mask drops):
        // the cheap column form of the id mask replaces the element form
        col = doc && !glob && qs.lo == qs.hi;
        if (col) doc = false;
      }
      return tile_value((skip ? TF_SKIP : 0) | (lim ? TF_LIM : 0) | (doc ? TF_DOC : 0) | (glob ? TF_GLOB : 0) | (col ? TF_COL : 0) |
                        (none ? TF_NONE : 0), qs.lo);
    };
    TileIter it;
    it.init_queries(first, nQtiles, qsum, gk_lo, gk_hi, CAUSAL && n0 > a.pfx_m1 ? n0 - gk : (int)0x80000000,
                    CAUSAL ? wg_rhi : 0x7fffffff, dec);
    if (gi > 0) __syncthreads();  // the previous head's last tile may still be read from LDS

    // software pipeline: tile `cur` is computed while `nxt` streams into the other buffer and
    // the row indices of the tile after that are fetched
    int cur = it.next(dec), cur_fl = it.flags, cur_id = it.value;
    int nxt = -1, nxt_fl = 0, nxt_id = 0;
    if (cur >= 0) { nxt = it.next(dec); nxt_fl = it.flags; nxt_id = it.value; }
    FA_TRACE_ONLY(if (gi == 0) FA_STAMP(g_trace_dkdv, 2, FA_CLOCK());)
    if (cur >= 0) {
      if (DOC) fetch_idx(cur);
      load_tile(cur, 0);
      if (DOC && nxt >= 0) fetch_idx(nxt);
    }
    if (LATE_SETTLE && gi == 0) {
      // the K / V fragments are complete before the tile loop (their wait would otherwise sit at the
      // first use inside it)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) settle(frag[ks]);
    }
    while (cur >= 0) {
      int nxt2 = -1, nxt2_fl = 0, nxt2_id = 0;
      if (nxt >= 0) { nxt2 = it.next(dec); nxt2_fl = it.flags; nxt2_id = it.value; }
      wait_async_loads();
      __syncthreads();
      FA_TRACE_ONLY(if (!tr_first) { FA_STAMP(g_trace_dkdv, 3, FA_CLOCK()); tr_first = true; })
      if (nxt >= 0) load_tile(nxt, 1);
      if (DOC && nxt2 >= 0) fetch_idx(nxt2);
      compute(0, cur, cur_fl, cur_id);
      FA_TRACE_ONLY(++tr_tiles;)
      cur = nxt; cur_fl = nxt_fl; cur_id = nxt_id; nxt = nxt2; nxt_fl = nxt2_fl; nxt_id = nxt2_id;
      if (cur < 0) break;
      nxt2 = -1;
      if (nxt >= 0) { nxt2 = it.next(dec); nxt2_fl = it.flags; nxt2_id = it.value; }
      wait_async_loads();
      __syncthreads();
      if (nxt >= 0) load_tile(nxt, 0);
      if (DOC && nxt2 >= 0) fetch_idx(nxt2);
      compute(1, cur, cur_fl, cur_id);
      FA_TRACE_ONLY(++tr_tiles;)
      cur = nxt; cur_fl = nxt_fl; cur_id = nxt_id; nxt = nxt2; nxt_fl = nxt2_fl; nxt_id = nxt2_id;
    }
  }

  FA_STAMP(g_trace_dkdv, 4, FA_CLOCK()); FA_STAMP(g_trace_dkdv, 6, tr_tiles);
  // shader clocks the first gradient wave spent at the pair flag (role-split form)
  FA_TRACE_ONLY(if (SPLIT && threadIdx.x == 64 * NKB && blockIdx.x < fa::kTraceWgs) g_trace_dkdv[blockIdx.x * 8 + 1] = tr_wait;)
  {
    // dK / dV rows leave through LDS (store_rows_through_lds), once every wave is done with the last query tile
    T* dvp = reinterpret_cast<T*>(a.dv) + b * a.dv_bs + hk * a.dv_hs;
    T* dkp = reinterpret_cast<T*>(a.dk) + b * a.dk_bs + hk * a.dk_hs;
    __syncthreads();
    char* patch = smem + wave * row_patch_bytes<D>();
    auto store = [&](T* base, const int64_t rs, const f32x16 (&v)[DBN], const float sc) __attribute__((always_inline)) {
      store_rows_through_lds<E, D, DBN>(patch, v, sc, [&](const int r) -> T* {
        return nw + r < a.N ? base + int64_t(nw + r) * rs : nullptr;
      });
    };
    if (SPLIT) {
      if (role == 1 && pair_lost) {   // the bounded wait expired somewhere: this wave's dK is not to be trusted
        if (lane == 0) __hip_atomic_fetch_add(&g_pair_expired, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int db = 0; db < DBN; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[db][r] = __builtin_nanf("");
      }
      if (role == 0) store(dvp, a.dv_rs, acc, 1.0f); else store(dkp, a.dk_rs, acc, a.scale);
    } else {
      store(dvp, a.dv_rs, acc, 1.0f);
      store(dkp, a.dk_rs, acc2, a.scale);
    }
  }
  }   // run of key tiles
  FA_STAMP(g_trace_dkdv, 5, FA_CLOCK());
}

// Query tiles per workgroup (no ids) below which the 64-key role-split form is launched.
constexpr int kKvShortTiles = 32;
template <typename Tag, int D, bool CAUSAL, bool DOC, int NKB, bool COLS = false>
static int launch_nkb(const KArgs& a, hipStream_t s) {
  constexpr bool SPLIT = D > 64;
  constexpr int BK = 32 * NKB, BQ = 64;
  const int nKt = (a.N + BK - 1) / BK;
  size_t lds = 4 * BQ * (D < 32 ? 32 : D) * 2 + 2 * 1024 + (SPLIT ? 2 * NKB * 2048 + 64 : 0);
  if (COLS && dkdv_cols_lds(D) > lds) lds = dkdv_cols_lds(D);
  auto kern = bwd_dkdv_kernel<Tag, D, CAUSAL, DOC, SPLIT, NKB, COLS>;
  static bool lds_allowed[64] = {};   // per kernel instantiation and device
  if (int e = allow_lds(kern, lds, lds_allowed)) return e;
  const int blocks = COLS ? grid_blocks((nKt + kColsRun - 1) / kColsRun, a.B * a.Hk) + dkdv_cols_blocks(a) : grid_blocks(nKt, a.B * a.Hk);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(SPLIT ? 128 * NKB : 64 * NKB), lds, s, a);
  return (int)hipGetLastError();
}

template <typename Tag, int D, bool CAUSAL, bool DOC>
static int launch_one(const KArgs& a, hipStream_t s) {
  // Role-split form (D = 128): a workgroup that visits few query tiles spends a sizeable part of its
  // life in set-up and drain, and two 64-key workgroups per CU cover each other's there; a long tile
  // stream is better served by the 128-key form, which reads every query tile half as often.  With
  // ids a workgroup visits about a dozen tiles at 16K tokens in documents of ~512 (64-key form 9 %
  // faster); without ids the number of tiles is known here: all of them, half on average under a
  // causal mask, at most a window's worth under a sliding window.  Under a block mask the 64-key
  // form is one column of blocks: no wave waits at a tile that only the other column needs
  // (diagonal + 25 % random blocks at 16K tokens: 1.81 -> 1.24 ms).
  // A key prefix without a diagonal of its own (more keys than queries), per-row positions or no causal
  // mask at all: local rows may need none of the leading keys, and the column form takes those (it decides
  // on the device, from the mask plan, how many they are -- possibly none).  Square causal problems with the
  // same ids on both sides always have a local row on the first keys' diagonal: nothing to gain there.
  if constexpr (DOC) {
    if (a.gap >= kGcolMinGap || a.qpos != nullptr || !CAUSAL) return launch_nkb<Tag, D, CAUSAL, DOC, (D > 64 ? 2 : 4), true>(a, s);
  }
  if constexpr (D > 64) {
    if (DOC || a.bmask != nullptr) return launch_nkb<Tag, D, CAUSAL, DOC, 2>(a, s);
    int tiles = (a.M + 63) / 64;
    if (CAUSAL) tiles = a.win < 0x3fffffff ? min(tiles, a.win / 64 + 3) : (tiles + 1) / 2;
    tiles *= a.G;
    return tiles < kKvShortTiles ? launch_nkb<Tag, D, CAUSAL, DOC, 2>(a, s) : launch_nkb<Tag, D, CAUSAL, DOC, 4>(a, s);
  } else {
    return launch_nkb<Tag, D, CAUSAL, DOC, 4>(a, s);
  }
}

template <typename Tag, int D>
static int launch_cd(const KArgs& a, bool causal, bool doc, hipStream_t s) {
  if (causal) return doc ? launch_one<Tag, D, true, true>(a, s) : launch_one<Tag, D, true, false>(a, s);
  return doc ? launch_one<Tag, D, false, true>(a, s) : launch_one<Tag, D, false, false>(a, s);
}

template <typename Tag>
static int launch_d(const KArgs& a, int D, bool causal, bool doc, hipStream_t s) {
  switch (D) {
    case 128: return launch_cd<Tag, 128>(a, causal, doc, s);
    case 64: return launch_cd<Tag, 64>(a, causal, doc, s);
    case 32: return launch_cd<Tag, 32>(a, causal, doc, s);
    case 16: return launch_cd<Tag, 16>(a, causal, doc, s);
    default: return -1;
  }
}

#ifdef FA_TRACE
int trace_read_dkdv(long long* host, int n) { return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_trace_dkdv), size_t(n) * 8); }
#endif

int read_pair_wait_expired(unsigned long long* n) {
  hipError_t e = hipDeviceSynchronize();
  if (e != hipSuccess) return (int)e;
  return (int)hipMemcpyFromSymbol(n, HIP_SYMBOL(g_pair_expired), sizeof(*n));
}

int launch_bwd_dkdv(const KArgs& a, int dtype, int D, bool causal, bool doc, hipStream_t s) {
  return dtype == FA_DTYPE_BF16 ? launch_d<bf16_t>(a, D, causal, doc, s) : launch_d<fp16_t>(a, D, causal, doc, s);
}

}  // namespace fa
