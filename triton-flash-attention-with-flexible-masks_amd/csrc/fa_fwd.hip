// Forward kernel: O = softmax(Q K^T * scale + mask) V and the log2-domain LSE.
// Replaces _fwd_kernel of the reference (flash_triton.py:25-141).
//
// Work decomposition (gfx950):
//   workgroup = 4 waves = 128 query rows; wave w owns rows 32w .. 32w+31.
//   K/V tiles of 64 keys are streamed global -> LDS with buffer loads that write
//   LDS directly, double buffered (2 x (K + V) x 64 x D x 2 bytes; 64 KB at D = 128).
//   S^T = K Q^T  : A = K rows from LDS, B = Q^T held in registers for the whole
//                  kernel; each lane then owns ONE query column and 16 keys of
//                  every 32-key block, so row max / row sum are in-lane plus one
//                  exchange with lane ^ 32.
//   O^T += V^T P^T : A = V^T via ds_read_b64_tr_b16, B = P^T taken straight from
//                  the S^T accumulators (the key order of the accumulator
//                  registers is absorbed into the V^T read pattern).
//   The softmax reference point of a row is only moved (and O, l rescaled) when a lane's
//   partial row sum of a tile, taken against the reference point as it stands, exceeds 2^12
//   (or the point is not set yet), so most tiles skip both the row maximum and the
//   rescale; the result is mathematically unchanged.
// Tiles of keys that cannot hold a kept element for the 128 rows (by the id
// summaries of the mask plan) are never loaded; per wave, tiles that are fully
// masked for its 32 rows are skipped and tiles that are fully kept take a path
// with no per-element mask work.

#include "fa_tile.h"

namespace fa {

// Operand fragments requested ahead of the MFMA that consumes them, in program order (measured
// optimum of a sweep over 2..8): K rows of the first product, transposed V reads of the second.
constexpr int kFwdPre = 4;
constexpr int kFwdPre2 = 4;

#ifdef FA_TRACE
// words: 0 start, 1 rows and ids known, 2 before the tile loop, 3 after it, 4 end, 5 key tiles computed, 6 (merging workgroup only) partial result stored and arrival counted, 7 tile | chunk << 16 | chunks << 24 (-1: left at once)
FA_TRACE_ARRAY(g_trace_fwd);
#endif

template <typename Tag, int D, bool CAUSAL, bool DOC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D <= 64 ? 3 : 2, D <= 64 ? 3 : 2)))
void fwd_kernel(const KArgs a) {
  using E = Elem<Tag>;
  using T = typename E::scalar;
  using vec8 = typename E::vec8;
  constexpr int BM = 128, BN = 64, KS = D / 16;
  constexpr int DL = D < 32 ? 32 : D;  // LDS row width: D = 16 is staged as 32 columns, the upper 16 zero
  constexpr int DBN = DL / 32;
  constexpr int TILE_BYTES = BN * DL * 2;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 5;
  FA_STAMP(g_trace_fwd, 0, FA_CLOCK()); FA_STAMP(g_trace_fwd, 4, 0); FA_STAMP(g_trace_fwd, 6, 0); FA_STAMP(g_trace_fwd, 7, -1);
  FA_TRACE_ONLY(int tr_tiles = 0;)

  // heaviest tiles first: with ids the global-row tiles sit at the end of the permuted
  // order and see the longest key ranges; without ids the last rows do
  const int nQt = DOC ? a.Pp / BM : (a.M + BM - 1) / BM;
  const int nSlots = nQt + (DOC ? split_extra(a) : 0);
  int slot, bh;
  if (!block_to_tile(nSlots, a.B * a.H, DOC && nQt >= 32, slot, bh)) return;
  const int b = bh / a.H, h = bh % a.H, hk = h / a.G;
  QWork wk;
  QHeader hd = {};
  if (DOC) hd = a.qhdr[b * a.qh_bs + h * a.qh_hs];
  if (!q_work<DOC>(a, hd, nQt, slot, wk)) return;
  QTileCtx<CAUSAL, DOC> qc;
  if (!qc.init(a, b, h, wk.tile, threadIdx.x >> 6)) return;
  q_work_finish(a, hd, wk);
  int kt_first = qc.first_tile(a), kt_last = qc.last_tile(a);
  const int nsplit = split_range(a, wk, kt_first, kt_last);
  if (wk.split >= nsplit) return;
  FA_STAMP(g_trace_fwd, 1, FA_CLOCK()); FA_STAMP(g_trace_fwd, 7, (long long)wk.tile | ((long long)wk.split << 16) | ((long long)nsplit << 24));
  const int row = qc.row, rowc = qc.rowc, eq_i = qc.eq_i;
  const int* ekp = qc.ekp;

  const T* qp = reinterpret_cast<const T*>(a.q) + b * a.q_bs + h * a.q_hs;
  const T* kp = reinterpret_cast<const T*>(a.k) + b * a.k_bs + hk * a.k_hs;
  const T* vp = reinterpret_cast<const T*>(a.v) + b * a.v_bs + hk * a.v_hs;
  T* op = reinterpret_cast<T*>(a.o) + b * a.o_bs + h * a.o_hs;
  float* lsep = a.lse + (int64_t(b) * a.H + h) * a.M;

  // Q^T fragments (B operand): lane holds d = 16*ks + 8*g .. +7 of its query row.
  vec8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = *reinterpret_cast<const vec8*>(qp + int64_t(rowc) * a.q_rs + ks * 16 + g * 8);

  // decisions of this wave for key tile t, evaluated by the lane that tests the tile
  QBlockMask bmq;
  bmq.init(a, b, h, wk.tile);
  const bool halved = qc.halved;
  const int sub = __builtin_amdgcn_readfirstlane(qc.sub);   // halved tiles: this wave computes keys 32 * sub .. of every key tile
  auto dec = [&](int t, const IdSummary& ks) {
    const int fl = halved ? qc.decide(a, t * BN + 32 * sub, 32, ks.lo, ks.hi) : qc.decide(a, t * BN, BN, ks.lo, ks.hi);
    return tile_value(fl | (DOC ? 0 : bmq.flags(t)), 0);
  };
  TileIter it;
  it.init_keys(kt_first, kt_last, qc.ksum, qc.g_lo, qc.g_hi, qc.g_glob, dec);   // its summaries travel together with Q

  // Q has arrived before anything asynchronous is issued (the compiler's in-order wait at its first
  // use would otherwise also wait for the tile loads issued in between)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) settle(qf[ks]);
  float c = a.scale_log2e;
  if (c < 0.f) {  // keep max(raw score) == max(scaled score): move the sign into Q
    c = -c;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = neg8<E>(qf[ks]);
  }

  TileLoader<DL, BN, D> ldK, ldV;
  ldK.init(kp, a.k_rs, a.N);
  ldV.init(vp, a.v_rs, a.N);
  LdsOffsets<DL> lo;
  lo.init();
  int id_off = g * 16, key_off = 0;
  if (halved) {   // this wave's half of every key tile
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) lo.row[ks] += sub * (32 * DL * 2);
#pragma unroll
    for (int db = 0; db < DBN; ++db) { lo.tr[db][0] += sub * (32 * DL * 2); lo.tr[db][1] += sub * (32 * DL * 2); }
    id_off += sub * (32 * 4);
    key_off = 32 * sub;
  }

  f32x16 o[DBN];
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;
  // scaled reference point of the exponentials (shared by lanes l, l^32); "not set yet" is a huge
  // negative finite number, so that exp2(s - m_ref) is 0 for a masked score and +inf for any other
  constexpr float kUnset = -1e30f;
  float m_ref = kUnset;
  float l_run = 0.f;        // this lane's partial row sum

  // One K/V tile; BUF is a compile-time constant so every LDS address is base + immediate.
  // nb_c: 32-key blocks of the tile this wave computes: both, or (halved tiles, see QTileCtx) one -- the lane
  // offsets `lo`, `id_off` and `key_off` then point into that block, so both forms use the same immediates.
  auto compute = [&](const int BUF, const int cur, const int flags, auto nb_c) __attribute__((always_inline)) {
    constexpr int NB = decltype(nb_c)::value;
    const char* lk = smem + BUF * TILE_BYTES;
    const char* lv = smem + (2 + BUF) * TILE_BYTES;
    const char* lid = smem + 4 * TILE_BYTES + BUF * (BN * 4) + id_off;  // the tile's key ids
    const int n0 = cur * BN + key_off;

    if (flags & TF_SKIP) return;
    const bool need_lim = (flags & TF_LIM) != 0, need_doc = (flags & TF_DOC) != 0;

    f32x16 s[2];
    __builtin_amdgcn_sched_barrier(0);
    // Two accumulator chains are fed alternately: an MFMA that accumulates onto the result of the MFMA
    // issued right before it waits a full extra MFMA time, two interleaved chains do not.  With both
    // blocks the chains are the blocks; with one block they are its even and odd k-steps, added up after.
    {
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      s[0] = zero;
      s[1] = zero;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if constexpr (NB == 2) {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) {
            const vec8 kf = lds_row8<E>(lk + lo.row[ks] + kb * 32 * DL * 2);
            s[kb] = E::mfma32(kf, qf[ks], s[kb]);
          }
        } else {
          const vec8 kf = lds_row8<E>(lk + lo.row[ks]);
          s[ks & 1] = E::mfma32(kf, qf[ks], s[ks & 1]);
        }
      }
    }
    // Instruction order of this region: keep several K fragments in flight ahead of the MFMA that
    // consumes them (an LDS read takes about as long as three MFMAs).
    {
      constexpr int NQK = NB * KS, PRE = NQK < kFwdPre ? NQK : kFwdPre;
      __builtin_amdgcn_sched_group_barrier(0x100, PRE, 0);
#pragma unroll
      for (int i = 0; i < NQK - PRE; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, PRE, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (NB == 1) {
      if (KS > 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[0][r] += s[1][r];
      }
    }
    if (need_lim) {
      asm volatile("" ::: "memory");  // keep this a real (wave-uniform) branch: never if-converted
      const int rel = qc.lim_i - n0 - 4 * g;
      const int rel_lo = qc.low_i - n0 - 4 * g;
      mask_lim(s[0], rel, rel_lo, -INFINITY);
      if constexpr (NB == 2) mask_lim(s[1], rel - 32, rel_lo - 32, -INFINITY);
    }
    if (DOC && need_doc) {
      asm volatile("" ::: "memory");
      mask_doc(s[0], lid, eq_i, qc.glob_i, -INFINITY);
      if constexpr (NB == 2) mask_doc(s[1], lid + 32 * 4, eq_i, qc.glob_i, -INFINITY);
    }
    // Online softmax in the exp2 domain with a lazily moved reference point.  Fast path: the
    // exponentials are taken against the reference point as it stands and only their sum is looked
    // at -- while every lane's partial row sum stays below a limit no element can be large, so the
    // row maximum (24 max operations, a lane exchange, the comparison) is not needed at all.  A
    // reference point that is not set yet (the sum comes out +inf) or too low sends the
    // whole wave through the full path: row maximum, new reference point, O and l rescaled.  A row
    // that has not met a kept key yet stays on the fast path (its exponentials are exact zeros).
    constexpr float kSumLimit = 4096.f;   // per lane over its 32 keys: every p <= 4096 (fits fp16 too)
    f32x16 p[NB];
    float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      p[0][r] = fast_exp2(__builtin_fmaf(s[0][r], c, -m_ref));
      ps0 += p[0][r];
      if constexpr (NB == 2) {
        p[1][r] = fast_exp2(__builtin_fmaf(s[1][r], c, -m_ref));
        ps1 += p[1][r];
      }
    }
    if (__builtin_amdgcn_ballot_w64(!(ps0 + ps1 <= kSumLimit)) != 0) {
      float mx;
      if constexpr (NB == 2) {
        float mx0 = fmaxf(fmaxf(s[0][0], s[0][1]), s[0][2]);
        float mx1 = fmaxf(fmaxf(s[1][0], s[1][1]), s[1][2]);
#pragma unroll
        for (int r = 3; r < 15; r += 2) {
          mx0 = fmaxf(fmaxf(mx0, s[0][r]), s[0][r + 1]);
          mx1 = fmaxf(fmaxf(mx1, s[1][r]), s[1][r + 1]);
        }
        mx = fmaxf(fmaxf(mx0, mx1), fmaxf(s[0][15], s[1][15]));
      } else {
        mx = fmaxf(fmaxf(s[0][0], s[0][1]), s[0][2]);
#pragma unroll
        for (int r = 3; r < 15; r += 2) mx = fmaxf(fmaxf(mx, s[0][r]), s[0][r + 1]);
        mx = fmaxf(mx, s[0][15]);
      }
      mx = xhalf_max(mx) * c;   // -inf stays -inf (c > 0)
      {
        // the reference point moves to the running maximum whenever this path is taken (after it
        // every p of the row is <= 1 again, so the next tiles are back on the fast path)
        const float m_new = fmaxf(m_ref, mx);
        const float alpha = fast_exp2(m_ref - m_new);   // 0 when the reference point is set for the first time
        m_ref = m_new;
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < DBN; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
      }
      const float msub = m_ref;   // still unset: every score of the row so far is -inf, exp2(-inf) = 0
      ps0 = 0.f; ps1 = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[0][r] = fast_exp2(__builtin_fmaf(s[0][r], c, -msub));
        ps0 += p[0][r];
        if constexpr (NB == 2) {
          p[1][r] = fast_exp2(__builtin_fmaf(s[1][r], c, -msub));
          ps1 += p[1][r];
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s[0][r] = p[0][r];
      if constexpr (NB == 2) s[1][r] = p[1][r];
    }
    l_run += ps0 + ps1;
    // O^T += V^T P^T, 16 keys per MFMA.  V^T fragments (two transposed reads each) are requested
    // PRE MFMAs ahead in program order, P is converted just in time; the scheduling barriers pin
    // that order (left to itself the scheduler puts every read right before its MFMA).
    {
      constexpr int NPV = 2 * NB * DBN, PRE = NPV < kFwdPre2 ? NPV : kFwdPre2;
      auto fetch = [&](const int i) __attribute__((always_inline)) {
        const int c16 = i / DBN, db = i % DBN;
        return lds_tr8<E>(lv + lo.tr[db][0] + c16 * 16 * DL * 2, lv + lo.tr[db][1] + c16 * 16 * DL * 2);
      };
      __builtin_amdgcn_sched_barrier(0);
      vec8 vf[NPV];
#pragma unroll
      for (int i = 0; i < PRE; ++i) vf[i] = fetch(i);
      vec8 pf;
#pragma unroll
      for (int i = 0; i < NPV; ++i) {
        if (i + PRE < NPV) vf[i + PRE] = fetch(i + PRE);
        if (i % DBN == 0) {
          const int c16 = i / DBN;
#pragma unroll
          for (int t = 0; t < 8; t += 2) {
            const typename E::vec2 pr = E::cvt2(s[c16 >> 1][8 * (c16 & 1) + t], s[c16 >> 1][8 * (c16 & 1) + t + 1]);
            pf[t] = pr[0];
            pf[t + 1] = pr[1];
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        o[i % DBN] = E::mfma32(vf[i], pf, o[i % DBN]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // tile streams: K, V and (with ids) the 64 key ids of the tile, all straight into LDS
  auto issue = [&](const int BUF, const int t) __attribute__((always_inline)) {
    ldK.issue(t * BN, smem + BUF * TILE_BYTES);
    ldV.issue(t * BN, smem + (2 + BUF) * TILE_BYTES);
    if (DOC && wave == 0) glb_load_lds4(ekp + t * BN + lane, smem + 4 * TILE_BYTES + BUF * (BN * 4));
  };
  int cur = it.next(dec);
  int cur_fl = it.flags;
  FA_STAMP(g_trace_fwd, 2, FA_CLOCK());
  if (cur >= 0) issue(0, cur);
  // the tile stream; one loop per form (halved tiles or not), so that neither pays for the other's registers
  auto stream = [&](auto nb_c) __attribute__((always_inline)) {
    while (cur >= 0) {
      int nxt = it.next(dec);
      wait_async_loads();
      __syncthreads();
      if (nxt >= 0) issue(1, nxt);
      compute(0, cur, cur_fl, nb_c);
      FA_TRACE_ONLY(tr_tiles = __builtin_amdgcn_readfirstlane(tr_tiles + 1);)   // (kept scalar: as a plain counter it cost 19 spilled registers)
      cur = nxt; cur_fl = it.flags;
      if (cur < 0) break;
      nxt = it.next(dec);
      wait_async_loads();
      __syncthreads();
      if (nxt >= 0) issue(0, nxt);
      compute(1, cur, cur_fl, nb_c);
      FA_TRACE_ONLY(tr_tiles = __builtin_amdgcn_readfirstlane(tr_tiles + 1);)   // (kept scalar: as a plain counter it cost 19 spilled registers)
      cur = nxt; cur_fl = it.flags;
    }
  };
  if (halved) stream(IntC<1>{}); else stream(IntC<2>{});
  FA_STAMP(g_trace_fwd, 3, FA_CLOCK()); FA_STAMP(g_trace_fwd, 5, tr_tiles);

  if (halved) {
    // The wave that took the second half of every key tile hands its softmax state (reference point, partial
    // row sum, unnormalised O) to the wave that took the first half of the same rows, lane for lane, through
    // the LDS the tile stream no longer needs; that wave merges the two and goes on alone.
    constexpr int NV = 2 + 16 * DBN;
    __syncthreads();   // every wave is done with the last tile
    float* mb = reinterpret_cast<float*>(smem) + qc.rb * (NV * 64) + lane;
    if (sub == 1) {
      mb[0] = m_ref; mb[64] = l_run;
#pragma unroll
      for (int db = 0; db < DBN; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) mb[(2 + 16 * db + r) * 64] = o[db][r];
    }
    __syncthreads();
    if (sub == 0) {
      const float m_b = mb[0], l_b = mb[64];
      const float m_new = fmaxf(m_ref, m_b);
      const float ca = fast_exp2(m_ref - m_new), cb = fast_exp2(m_b - m_new);   // both unset: 1 and 1 on zeros
      m_ref = m_new;
      l_run = l_run * ca + l_b * cb;
#pragma unroll
      for (int db = 0; db < DBN; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] = o[db][r] * ca + mb[(2 + 16 * db + r) * 64] * cb;
    }
  }
  const bool writer = !halved || sub == 0;   // the wave that holds the rows' result
  const float l_tot = xhalf_sum(l_run);
  if (DOC && nsplit > 1) {
    // This workgroup saw one chunk of the keys: store the unnormalised partial result; the last
    // chunk to arrive combines them (log-sum-exp merge) and writes O and LSE.
    const int64_t tbase = (int64_t(b) * a.H + h) * a.split_tiles + wk.gt;
    float* po = a.sk_o + (tbase * a.split_k + wk.split) * (128 * D);
    float* pml = a.sk_ml + (tbase * a.split_k + wk.split) * (128 * 2);
    const int rt = qc.rb * 32 + (lane & 31);   // row inside the tile
    if (g == 0 && writer) store_dev(pml + rt * 2, m_ref, l_tot);
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        if (32 * db + 8 * q4 >= D || !writer) continue;
        f32x4 x = {o[db][4 * q4 + 0], o[db][4 * q4 + 1], o[db][4 * q4 + 2], o[db][4 * q4 + 3]};
        store_dev(po + part_index<D>(qc.rb, 4 * db + q4, lane) * 4, x);
      }
    if (!split_arrive(a.sk_cnt + tbase, nsplit)) { FA_STAMP(g_trace_fwd, 4, FA_CLOCK()); return; }
    FA_STAMP(g_trace_fwd, 6, FA_CLOCK());
    // merge: the whole workgroup walks the tile, one float4 of one row per thread and step.  The
    // partial results come through device-scope loads, each a round trip of its own: up to eight chunks are
    // requested together, four or two steps of them (16 + 16 loads in flight per thread), instead of one by one.
    constexpr int C4 = D / 4;
    const float* bo = a.sk_o + tbase * a.split_k * (128 * D);
    const float* bml = a.sk_ml + tbase * a.split_k * (128 * 2);
    const int* prm = a.perm + b * a.pm_bs + h * a.pm_hs + wk.tile * 128;
    auto finish_row = [&](int mrow, int c, float mmax, float lsum, f32x4 acc) __attribute__((always_inline)) {
      const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
      if (c == 0) lsep[mrow] = lsum > 0.f ? mmax + fast_log2(lsum) : -INFINITY;
      const typename E::vec2 x0 = E::cvt2(acc[0] * inv, acc[1] * inv);
      const typename E::vec2 x1 = E::cvt2(acc[2] * inv, acc[3] * inv);
      typename E::vec4 x = {x0[0], x0[1], x1[0], x1[1]};
      *reinterpret_cast<typename E::vec4*>(op + int64_t(mrow) * a.o_rs + 4 * c) = x;
    };
    // NS chunk slots of IT steps each: 16 + 16 loads in flight per thread whatever the number of chunks
    auto merge_batched = [&](auto it_c, auto ns_c) __attribute__((always_inline)) {
      constexpr int IT = decltype(it_c)::value, NS = decltype(ns_c)::value;
      for (int i0 = threadIdx.x; i0 < 128 * C4; i0 += 256 * IT) {
        float m_[IT][NS], l_[IT][NS];
        f32x4 x[IT][NS];
        int mrow[IT], cc[IT];
#pragma unroll
        for (int u = 0; u < IT; ++u) {
          const int i = i0 + 256 * u;
          int r, c;
          part_coords<D>(min(i, 128 * C4 - 1), r, c);
          cc[u] = c;
          mrow[u] = i < 128 * C4 ? prm[r] : -1;
          if (mrow[u] < 0) continue;   // no such row (a tile of a few dozen rows has mostly these): nothing to fetch
#pragma unroll
          for (int sp = 0; sp < NS; ++sp) {
            const int spc = min(sp, nsplit - 1);   // chunks past the last one repeat it (weight 0 below)
            load_dev(bml + spc * 256 + r * 2, m_[u][sp], l_[u][sp]);
            x[u][sp] = load_dev4(bo + spc * (128 * D) + i * 4);
          }
        }
#pragma unroll
        for (int u = 0; u < IT; ++u) {
          if (mrow[u] < 0) continue;
          float mmax = -INFINITY;
#pragma unroll
          for (int sp = 0; sp < NS; ++sp) mmax = fmaxf(mmax, m_[u][sp]);
          float lsum = 0.f;
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int sp = 0; sp < NS; ++sp) {
            const float w = (sp >= nsplit || m_[u][sp] == -INFINITY) ? 0.f : fast_exp2(m_[u][sp] - mmax);
            lsum += w * l_[u][sp];
            acc[0] += w * x[u][sp][0]; acc[1] += w * x[u][sp][1]; acc[2] += w * x[u][sp][2]; acc[3] += w * x[u][sp][3];
          }
          finish_row(mrow[u], cc[u], mmax, lsum, acc);
        }
      }
    };
    if (nsplit <= 8) {   // (with 9 .. 16 chunks the plain loop below measured the same or better)
      if (nsplit <= 4) merge_batched(IntC<4>{}, IntC<4>{});
      else merge_batched(IntC<2>{}, IntC<8>{});
      FA_STAMP(g_trace_fwd, 4, FA_CLOCK());
      return;
    }
    for (int i = threadIdx.x; i < 128 * C4; i += 256) {
      int r, c;
      part_coords<D>(i, r, c);
      const int mrow = prm[r];
      if (mrow < 0) continue;
      float mmax = -INFINITY;
      for (int sp = 0; sp < nsplit; ++sp) {
        float m_, l_;
        load_dev(bml + sp * 256 + r * 2, m_, l_);
        mmax = fmaxf(mmax, m_);
      }
      float lsum = 0.f;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < nsplit; ++sp) {
        float m_, l_;
        load_dev(bml + sp * 256 + r * 2, m_, l_);
        const float w = m_ == -INFINITY ? 0.f : fast_exp2(m_ - mmax);
        lsum += w * l_;
        const f32x4 x = load_dev4(bo + sp * (128 * D) + i * 4);
        acc[0] += w * x[0]; acc[1] += w * x[1]; acc[2] += w * x[2]; acc[3] += w * x[3];
      }
      finish_row(mrow, c, mmax, lsum, acc);
    }
    FA_STAMP(g_trace_fwd, 4, FA_CLOCK());
    return;
  }

  // epilogue: normalise, write O and LSE (the rows leave through LDS, see store_rows_through_lds: every wave is
  // done with the last tile first; a halved tile's writers use the part of LDS they have just read their partner's state from)
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (!halved) __syncthreads();
  if (row >= 0 && writer && g == 0) lsep[row] = l_tot > 0.f ? m_ref + fast_log2(l_tot) : -INFINITY;
  if (writer) {
    char* patch = smem + (halved ? qc.rb * ((2 + 16 * DBN) * 64 * 4) : wave * row_patch_bytes<D>());
    store_rows_through_lds<E, D, DBN>(patch, o, inv, [&](const int r) -> T* {
      const int rr = __shfl(row, r);
      return rr >= 0 ? op + int64_t(rr) * a.o_rs : nullptr;
    });
  }
  FA_STAMP(g_trace_fwd, 4, FA_CLOCK());
}

template <typename Tag, int D, bool CAUSAL, bool DOC>
static int launch_one(const KArgs& a, hipStream_t s) {
  constexpr int BM = 128, BN = 64;
  const int nQt = (DOC ? a.Pp / BM : (a.M + BM - 1) / BM) + (DOC ? split_extra(a) : 0);
  const size_t lds = 4 * BN * (D < 32 ? 32 : D) * 2 + 2 * BN * 4;  // K, V double buffered + key ids
  auto kern = fwd_kernel<Tag, D, CAUSAL, DOC>;
  static bool lds_allowed[64] = {};   // per kernel instantiation and device
  if (int e = allow_lds(kern, lds, lds_allowed)) return e;
  hipLaunchKernelGGL(kern, dim3(grid_blocks(nQt, a.B * a.H)), dim3(256), lds, s, a);
  return (int)hipGetLastError();
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
int trace_read_fwd(long long* host, int n) { return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_trace_fwd), size_t(n) * 8); }
#endif

int launch_fwd(const KArgs& a, int dtype, int D, bool causal, bool doc, hipStream_t s) {
  return dtype == FA_DTYPE_BF16 ? launch_d<bf16_t>(a, D, causal, doc, s) : launch_d<fp16_t>(a, D, causal, doc, s);
}

}  // namespace fa
