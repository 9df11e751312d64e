// dK/dV of the key columns that only a few global rows see (the second form of _bwd_kv_kernel,
// flash_triton.py:175-321, for the rectangular case :214-216,521).
//
// With document ids, keys that no local row (eq < 0) can need -- the keys before QHeader::k0: a long
// key sequence whose queries are its tail, a prompt prefix under packed decoding -- are seen by the
// global rows (eq >= 0) alone.  When those are few, the general kernel spends its life setting up:
// one workgroup per 64 keys, each building a tile stream for one or two query tiles.  Here the roles
// of the two sides are swapped: the global rows' Q / dO tiles (at most kGcolTilesMax tiles of 64 rows,
// gathered through the permutation of the mask plan, with their LSE / delta / diagonal positions)
// are loaded into LDS ONCE per workgroup, and the workgroup then walks its share of the columns.  Every wave
// takes 32 keys at a time, K and V rows straight from global memory into registers (the B operands),
// and does both roles for them:
//   pass 1, per resident tile and 32-row block:  S = Q K^T, dP = dO V^T (two interleaved MFMA chains),
//           P = exp2(S c - L) masked, dS = P (dP - delta); P and dS kept as packed 16-bit fragments
//   (the K / V rows of the wave's next 32 keys are requested here: their registers are free again)
//   pass 2: dV^T = sum dO^T P    -> stored        pass 3: dK^T = sum Q^T dS, times sm_scale -> stored
// One accumulator set is live at a time, so two waves per SIMD fit and nothing is exchanged between
// waves: after the one barrier behind the resident tiles the waves run free.  A column no row sees
// gets zeros.  The kernel is bound by HBM: every K / V row is read once and every dK / dV row written once.
//
// Which columns these are is decided on the device by both kernels of the launch (gcol_info).
#pragma once

#include "fa_tile.h"

namespace fa {

// Workgroups of this form per (batch, key head): the columns of a head are dealt evenly among them on the
// device (how many columns there are is only known there).  About two resident workgroups per CU over the
// whole launch, so that the resident tiles are loaded once per workgroup slot and the launch ends without a
// ragged second round; never less than 128 keys each.
constexpr int kColsWgs = 256;
FA_HD int dkdv_cols_per_head(const KArgs& a) {
  const int bh = a.B * a.Hk, most = (a.N + 127) / 128;
  const int p = bh >= kColsWgs ? 1 : kColsWgs / bh;
  return p < most ? p : most;
}
// Grid blocks this form needs next to those of the general form (they share one launch).
FA_HD int dkdv_cols_blocks(const KArgs& a) { return grid_blocks(dkdv_cols_per_head(a), a.B * a.Hk); }
// Dynamic LDS of this form: the resident tiles with their row data, and a patch per wave for the stores.
constexpr size_t dkdv_cols_lds(int D) { return size_t(kGcolTilesMax) * (2 * 64 * (D < 32 ? 32 : D) * 2 + 1024) + 4 * 16 * 144; }

// bid: index of the workgroup among those of this form; 256 threads.
template <typename Tag, int D, bool CAUSAL>
FA_DEV void dkdv_cols_body(const KArgs& a, const int bid, char* smem) {
  using E = Elem<Tag>;
  using T = typename E::scalar;
  using vec8 = typename E::vec8;
  constexpr int BQ = 64, KS = D / 16, NW = 4;
  constexpr int DL = D < 32 ? 32 : D;
  constexpr int DBN = DL / 32;
  constexpr int TILE_BYTES = BQ * DL * 2;
  constexpr int TMAX = kGcolTilesMax;
  constexpr int AUX_OFF = TMAX * 2 * TILE_BYTES;   // per resident tile: Q, dO; then [TMAX][LSE, delta, position][64]
  constexpr int AUX_BYTES = 1024;
  // per wave: 16 key rows x 64 columns (16-bit; 32 columns at D <= 32) of a result on their way out
  constexpr int XP_OFF = AUX_OFF + TMAX * AUX_BYTES;
  constexpr int XP_DB = DBN >= 2 ? 2 : 1;          // column blocks of 32 per round
  constexpr int XP_CPR = XP_DB * 4;                // 16-byte chunks per patch row
  constexpr int XP_RPI = 64 / XP_CPR;              // rows per wave instruction on the way out
  constexpr int XP_NI = 16 / XP_RPI;
  constexpr int kXpPitch = XP_DB * 64 + 16;
  constexpr int XP_BYTES = 16 * 144;
  using Loader = TileLoader<DL, BQ, D, NW>;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lq = lane & 31, g = lane >> 5;

  const int nCh = dkdv_cols_per_head(a);
  int ch, bhk;
  if (!block_to_tile(nCh, a.B * a.Hk, false, ch, bhk, bid)) return;
  const int b = bhk / a.Hk, hk = bhk % a.Hk;
  const GcolInfo info = gcol_info(a, b, hk);
  const int chunk = ((info.ncols + nCh - 1) / nCh + 127) / 128 * 128;   // keys per workgroup of this head
  const int key0 = ch * chunk;
  if (key0 >= info.ncols) return;
  FA_STAMP(g_trace_dkdv, 0, FA_CLOCK()); FA_STAMP(g_trace_dkdv, 5, 0); FA_STAMP(g_trace_dkdv, 7, (long long)ch | (1ll << 40));
  FA_TRACE_ONLY(int tr_blocks = 0;)
  const int kend = min(min(info.ncols, key0 + chunk), a.N);
  const int nblk = (kend - key0 + 31) / 32;

  // the resident tiles: every 64-row tile of global rows of every query head of the group
  int r_h[TMAX], r_t[TMAX];
  int nres = 0;
#pragma unroll
  for (int r = 0; r < TMAX; ++r) { r_h[r] = 0; r_t[r] = 0; }
  for (int gi = 0; gi < a.G; ++gi) {
    const int h = hk * a.G + gi;
    const QHeader hd = a.qhdr[b * a.qh_bs + h * a.qh_hs];
    const int n = (hd.nG + 63) / 64;
    for (int i = 0; i < n; ++i) {
#pragma unroll
      for (int r = 0; r < TMAX; ++r)
        if (r == nres) { r_h[r] = h; r_t[r] = hd.nLp / 64 + i; }
      ++nres;
    }
  }
  // (gcol_info has refused more than TMAX tiles: ncols = 0 and the workgroup is gone)

  // Operand read offsets of this lane (LdsOffsets): the swizzle is an XOR on the 16-byte chunk index, so the
  // offset of k-step ks is the one of step 0 with ks XOR-ed into bits 5.., and of column block db the one of
  // block 0 with db XOR-ed into bits 6..: three registers instead of KS + 2 * DBN.
  int row0, tr0[2];
  {
    LdsOffsets<DL> lo;
    lo.init();
    row0 = lo.row[0]; tr0[0] = lo.tr[0][0]; tr0[1] = lo.tr[0][1];
  }
  // (the copies below are made opaque where they are used, so that the derived offsets are formed next to
  // their reads instead of all being kept in registers for the whole kernel)
  int r_rmin[TMAX], r_rmax[TMAX];
#pragma unroll
  for (int r = 0; r < TMAX; ++r) {
    r_rmin[r] = 0x7fffffff; r_rmax[r] = -1;
    if (r < nres) {
      const int h = r_h[r];
      const IdSummary qs = a.qsum[b * a.qs_bs + h * a.qs_hs + r_t[r]];
      r_rmin[r] = qs.nvalid > 0 ? qs.rmin : 0x7fffffff;
      r_rmax[r] = qs.nvalid > 0 ? qs.rmax : -1;
      // gather the tile: rows through the permutation, LSE / delta of those rows, their diagonal positions
      const int* pmp = a.perm + b * a.pm_bs + h * a.pm_hs + r_t[r] * BQ;
      const int* ppp = a.ppos + b * a.pm_bs + h * a.pm_hs + r_t[r] * BQ;
      Loader ldQ, ldO;
      ldQ.init(reinterpret_cast<const T*>(a.q) + b * a.q_bs + h * a.q_hs, a.q_rs, a.M);
      ldO.init(reinterpret_cast<const T*>(a.dout) + b * a.do_bs + h * a.do_hs, a.do_rs, a.M);
      char* lq_t = smem + r * 2 * TILE_BYTES;
      char* lo_t = lq_t + TILE_BYTES;
      char* aux = smem + AUX_OFF + r * AUX_BYTES;
#pragma unroll
      for (int i = 0; i < Loader::PER; ++i) {
        if (Loader::NI % NW == 0 || i * NW + wave < Loader::NI) {
          const int rit = ((i * NW + wave) * Loader::RPI + lane / Loader::CPR) % BQ;
          const int gc = (lane % Loader::CPR) ^ swz<DL, SWZ_ROW>(rit);
          const int coff = gc < D / 8 ? gc * 16 : kOobOffset;
          const int ri = pmp[rit];
          const int rr = ri >= 0 ? ri : 0;
          buf_load_lds16(ldQ.rsrc, lq_t + (i * NW + wave) * 1024, rr * ldQ.row_bytes + coff, 0);
          buf_load_lds16(ldO.rsrc, lo_t + (i * NW + wave) * 1024, rr * ldO.row_bytes + coff, 0);
        }
      }
      const int ri = pmp[lane];
      const int rr = ri >= 0 ? ri : 0;
      if (wave == 0) glb_load_lds4(a.lse + (int64_t(b) * a.H + h) * a.M + rr, aux);
      if (wave == 1) glb_load_lds4(a.delta + (int64_t(b) * a.H + h) * a.M + rr, aux + 256);
      if (wave == 2) glb_load_lds4(ppp + lane, aux + 512);
    }
  }

  const T* kbase = reinterpret_cast<const T*>(a.k) + b * a.k_bs + hk * a.k_hs;
  const T* vbase = reinterpret_cast<const T*>(a.v) + b * a.v_bs + hk * a.v_hs;
  vec8 kf[KS], vf[KS];
  // (a slice spans less than 2 GiB: 32-bit byte offsets on top of the wave-uniform base)
  const unsigned k_rb = (unsigned)a.k_rs * 2u, v_rb = (unsigned)a.v_rs * 2u;
  auto load_kv = [&](int j) __attribute__((always_inline)) {
    const int key = key0 + 32 * j + lq;
    const unsigned keyc = (unsigned)(key < a.N ? key : a.N - 1);
    const char* kp = reinterpret_cast<const char*>(kbase) + (keyc * k_rb + (unsigned)g * 16u);
    const char* vp = reinterpret_cast<const char*>(vbase) + (keyc * v_rb + (unsigned)g * 16u);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = *reinterpret_cast<const vec8*>(kp + ks * 32);
      vf[ks] = *reinterpret_cast<const vec8*>(vp + ks * 32);
    }
  };
  int j = wave;
  if (j < nblk && nres > 0) load_kv(j);
  // the K / V rows are complete before the barrier below: its wait (every outstanding load) then covers the
  // resident tiles as well, and nothing asynchronous is in flight once the loop reads LDS
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) { settle(kf[ks]); settle(vf[ks]); }
  wait_async_loads();
  __syncthreads();
  FA_STAMP(g_trace_dkdv, 3, FA_CLOCK());

  const float c = a.scale_log2e;
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  for (; j < nblk; j += NW) {
    FA_TRACE_ONLY(++tr_blocks;)
    const int nw = key0 + 32 * j;
    const int key = nw + lq;
    // rows (named by the key position of their diagonal) that may see this lane's key: [row_lo, row_lo + row_span)
    const int row_lo = CAUSAL ? (key <= a.pfx_m1 ? 0 : max(0, key)) : 0;
    const int row_hi = CAUSAL ? min(kPosMax, key + a.win - 1) : kPosMax;
    const unsigned row_span = (key < a.N && row_hi >= row_lo) ? (unsigned)(row_hi - row_lo + 1) : 0u;

    vec8 p16[TMAX][2][2], ds16[TMAX][2][2];   // per resident tile, 32-row block, 16-row half
    bool live[TMAX];
#pragma unroll
    for (int r = 0; r < TMAX; ++r) {
      // no row of the tile reaches these 32 keys (causal), or all are past them (window): nothing to do
      live[r] = r < nres && r_rmax[r] >= 0 &&
                !(CAUSAL && ((r_rmax[r] < nw && nw > a.pfx_m1) || r_rmin[r] - a.win + 1 > nw + 31));
      if (!live[r]) continue;
      const char* lqt = smem + r * 2 * TILE_BYTES;
      const char* ldo = lqt + TILE_BYTES;
      const char* aux = smem + AUX_OFF + r * AUX_BYTES;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        f32x16 x = zero, dp = zero;
        int rw = row0;
        asm volatile("" : "+v"(rw));
        auto row_off = [&](const int ks) __attribute__((always_inline)) { return rw ^ (ks << 5); };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const vec8 rq = lds_row8<E>(lqt + row_off(ks) + qb * 32 * DL * 2);
          x = E::mfma32(rq, kf[ks], x);
          const vec8 ro = lds_row8<E>(ldo + row_off(ks) + qb * 32 * DL * 2);
          dp = E::mfma32(ro, vf[ks], dp);
        }
        {
          constexpr int NM = 2 * KS, PRE = NM < 4 ? NM : 4;
          __builtin_amdgcn_sched_group_barrier(0x100, PRE, 0);
#pragma unroll
          for (int i = 0; i < NM - PRE; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, PRE, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // LSE, delta and diagonal position of this lane's 16 rows of the block (row 8*q4 + 4*g + t)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int i0 = (32 * qb + 8 * q4 + 4 * g) * 4;
          const f32x4 Lv = *reinterpret_cast<const f32x4*>(aux + i0);
          const f32x4 dl = *reinterpret_cast<const f32x4*>(aux + 256 + i0);
          const i32x4 rowv = *reinterpret_cast<const i32x4*>(aux + 512 + i0);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int e = 4 * q4 + t;
            float p = fast_exp2(__builtin_fmaf(x[e], c, -Lv[t]));
            p = (unsigned)(rowv[t] - row_lo) < row_span ? p : 0.f;   // padding rows carry position -1
            x[e] = p;
            dp[e] = p * (dp[e] - dl[t]);
          }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int t = 0; t < 8; t += 2) {
            const typename E::vec2 pr = E::cvt2(x[8 * half + t], x[8 * half + t + 1]);
            p16[r][qb][half][t] = pr[0]; p16[r][qb][half][t + 1] = pr[1];
            const typename E::vec2 dr = E::cvt2(dp[8 * half + t], dp[8 * half + t + 1]);
            ds16[r][qb][half][t] = dr[0]; ds16[r][qb][half][t + 1] = dr[1];
          }
      }
    }
    // the next 32 keys of this wave: K and V rows travel while this block's second products run
    const bool more = j + NW < nblk && nres > 0;
    __builtin_amdgcn_sched_barrier(0);
    if (more) load_kv(j + NW);
    __builtin_amdgcn_sched_barrier(0);

    // second products: acc^T (lane = key column, registers = d rows) += A^T (transposed LDS reads) x B (16-bit fragments)
    auto second = [&](const int which, const float sc, T* obase, const unsigned ors_b) __attribute__((always_inline)) {
      f32x16 acc[DBN];
#pragma unroll
      for (int db = 0; db < DBN; ++db) acc[db] = zero;
#pragma unroll
      for (int r = 0; r < TMAX; ++r) {
        if (!live[r]) continue;
        const char* tr = smem + r * 2 * TILE_BYTES + (which == 0 ? TILE_BYTES : 0);   // dO^T for dV, Q^T for dK
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          constexpr int NM = 2 * DBN, PRE = NM < 2 ? NM : 2;
          int t0 = tr0[0], t1 = tr0[1];
          asm volatile("" : "+v"(t0), "+v"(t1));
          auto tr_off = [&](const int db, const int hh) __attribute__((always_inline)) { return (hh ? t1 : t0) ^ (db << 6); };
          auto fetch = [&](const int i) __attribute__((always_inline)) {
            const int half = i / DBN, db = i % DBN;
            const int goff = (2 * qb + half) * 16 * DL * 2;
            return lds_tr8<E>(tr + tr_off(db, 0) + goff, tr + tr_off(db, 1) + goff);
          };
          __builtin_amdgcn_sched_barrier(0);
          vec8 tf[NM];
#pragma unroll
          for (int i = 0; i < PRE; ++i) tf[i] = fetch(i);
#pragma unroll
          for (int i = 0; i < NM; ++i) {
            if (i + PRE < NM) tf[i + PRE] = fetch(i + PRE);
            __builtin_amdgcn_sched_barrier(0);
            acc[i % DBN] = E::mfma32(tf[i], which == 0 ? p16[r][qb][i / DBN] : ds16[r][qb][i / DBN], acc[i % DBN]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // The accumulators hold a key per lane and 4 consecutive columns per register quad: stored from there,
      // a wave instruction would write 64 pieces of 8 bytes, 256 bytes apart, and the lines of the result would
      // fill up over sixteen instructions (lines that leave the L2 half written are fetched back to be merged:
      // measured as one byte read for every byte written).  This kernel lives on its stores, so every block of
      // 16 keys x 64 columns goes through the wave's own patch of LDS and leaves as 16 bytes per lane, eight
      // lanes to a key: whole 128-byte lines per instruction (LDS operations of a wave execute in order).
      char* xp = smem + XP_OFF + wave * XP_BYTES;
#pragma unroll
      for (int d0 = 0; d0 < DBN; d0 += XP_DB) {
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
          if ((lq >> 4) == kh) {
#pragma unroll
            for (int dd = 0; dd < XP_DB; ++dd)
#pragma unroll
              for (int q4 = 0; q4 < 4; ++q4) {
                const int db = d0 + dd;
                const typename E::vec2 k0 = E::cvt2(acc[db][4 * q4 + 0] * sc, acc[db][4 * q4 + 1] * sc);
                const typename E::vec2 k1 = E::cvt2(acc[db][4 * q4 + 2] * sc, acc[db][4 * q4 + 3] * sc);
                typename E::vec4 xk = {k0[0], k0[1], k1[0], k1[1]};
                *reinterpret_cast<typename E::vec4*>(xp + (lq & 15) * kXpPitch + (32 * dd + 8 * q4 + 4 * g) * 2) = xk;
              }
          }
          asm volatile("" ::: "memory");   // (order only: the LDS executes a wave's operations in issue order)
#pragma unroll
          for (int i = 0; i < XP_NI; ++i) {
            const int kr = XP_RPI * i + lane / XP_CPR, cc = lane % XP_CPR;   // key row of the half block, 16-byte chunk of its row
            const vec8 x = *reinterpret_cast<const vec8*>(xp + kr * kXpPitch + cc * 16);
            const int key_o = nw + 16 * kh + kr;
            if (key_o < a.N && 32 * d0 + 8 * cc < D)
              __builtin_nontemporal_store(x, reinterpret_cast<vec8*>(reinterpret_cast<char*>(obase) + ((unsigned)key_o * ors_b + (unsigned)(64 * d0 + 16 * cc))));   // streaming: nobody reads these lines soon
          }
          asm volatile("" ::: "memory");   // the next writes to the patch are issued, hence executed, after these reads
        }
      }
    };
    second(0, 1.0f, reinterpret_cast<T*>(a.dv) + b * a.dv_bs + hk * a.dv_hs, (unsigned)a.dv_rs * 2u);
    second(1, a.scale, reinterpret_cast<T*>(a.dk) + b * a.dk_bs + hk * a.dk_hs, (unsigned)a.dk_rs * 2u);
  }
  FA_STAMP(g_trace_dkdv, 4, FA_CLOCK()); FA_STAMP(g_trace_dkdv, 6, tr_blocks); FA_STAMP(g_trace_dkdv, 5, FA_CLOCK());
}

}  // namespace fa
