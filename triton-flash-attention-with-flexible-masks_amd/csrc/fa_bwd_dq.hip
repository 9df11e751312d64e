// dQ kernel of the split backward: one 128-row query tile resident, key/value
// tiles streamed.  Replaces _bwd_q_kernel of the reference (flash_triton.py:323-431).
//
//   S^T  = K Q^T          A = K rows (LDS),   B = Q^T (registers)
//   dP^T = V dO^T         A = V rows (LDS),   B = dO^T (registers)
//   P    = exp2(S*c - L)  masked elements -> 0            (flash_triton.py:396,402-414)
//   dS   = P * (dP - delta)                               (flash_triton.py:400)
//   dQ^T += K^T dS^T      A = K^T via ds_read_b64_tr_b16, B = dS^T from the accumulators
//   dQ   = dQ * sm_scale                                  (flash_triton.py:425)
// Same workgroup shape, LDS staging and tile skipping as the forward kernel.

#include "fa_tile.h"

namespace fa {

// Operand fragments requested ahead of the MFMA that consumes them, in program order (measured
// optimum of a sweep over 2..6): row-wise K / V reads, transposed K reads of the dQ product.
constexpr int kDqPre = 4;
constexpr int kDqPre2 = 3;

#ifdef FA_TRACE
// words: 0 start, 1 rows and ids known, 2 before the tile loop, 3 after it, 4 end, 5 key tiles computed, 6 (merging workgroup only) partial result stored and arrival counted, 7 tile | chunk << 16 | chunks << 24 (-1: left at once)
FA_TRACE_ARRAY(g_trace_dq);
#endif

template <typename Tag, int D, bool CAUSAL, bool DOC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D <= 64 ? 3 : 2, D <= 64 ? 3 : 2)))
void bwd_dq_kernel(const KArgs a) {
  using E = Elem<Tag>;
  using T = typename E::scalar;
  using vec8 = typename E::vec8;
  constexpr int BM = 128, BN = 64, KS = D / 16;
  constexpr int DL = D < 32 ? 32 : D;  // LDS row width: D = 16 is staged as 32 columns, the upper 16 zero
  constexpr int DBN = DL / 32;
  constexpr int TILE_BYTES = BN * DL * 2;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int lane = threadIdx.x & 63;
  const int g = lane >> 5;
  FA_STAMP(g_trace_dq, 0, FA_CLOCK()); FA_STAMP(g_trace_dq, 4, 0); FA_STAMP(g_trace_dq, 6, 0); FA_STAMP(g_trace_dq, 7, -1);
  FA_TRACE_ONLY(int tr_tiles = 0;)

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
  FA_STAMP(g_trace_dq, 1, FA_CLOCK()); FA_STAMP(g_trace_dq, 7, (long long)wk.tile | ((long long)wk.split << 16) | ((long long)nsplit << 24));
  const int row = qc.row, rowc = qc.rowc, eq_i = qc.eq_i;
  const int* ekp = qc.ekp;

  const T* qp = reinterpret_cast<const T*>(a.q) + b * a.q_bs + h * a.q_hs;
  const T* kp = reinterpret_cast<const T*>(a.k) + b * a.k_bs + hk * a.k_hs;
  const T* vp = reinterpret_cast<const T*>(a.v) + b * a.v_bs + hk * a.v_hs;
  const T* dop = reinterpret_cast<const T*>(a.dout) + b * a.do_bs + h * a.do_hs;
  T* dqp = reinterpret_cast<T*>(a.dq) + b * a.dq_bs + h * a.dq_hs;
  const float* lsep = a.lse + (int64_t(b) * a.H + h) * a.M;
  float* delp = a.delta + (int64_t(b) * a.H + h) * a.M;
  const T* op = reinterpret_cast<const T*>(a.o) + b * a.o_bs + h * a.o_hs;
  const bool own_delta = a.dq_delta != 0;   // delta = rowsum(O * dO) is computed here instead of being read

  vec8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks] = *reinterpret_cast<const vec8*>(qp + int64_t(rowc) * a.q_rs + ks * 16 + g * 8);
    dof[ks] = *reinterpret_cast<const vec8*>(dop + int64_t(rowc) * a.do_rs + ks * 16 + g * 8);
  }
  vec8 of[KS] = {};
  if (own_delta) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) of[ks] = *reinterpret_cast<const vec8*>(op + int64_t(rowc) * a.o_rs + ks * 16 + g * 8);
  }
  const float c = a.scale_log2e;
  float L_i = lsep[rowc];
  float delta_i = own_delta ? 0.f : delp[rowc];

  // decisions of this wave for key tile t, evaluated by the lane that tests the tile
  QBlockMask bmq;
  bmq.init(a, b, h, wk.tile);
  const bool halved = qc.halved;
  const int sub = __builtin_amdgcn_readfirstlane(qc.sub);   // halved tiles (QTileCtx): this wave computes keys 32 * sub .. of every key tile
  auto dec = [&](int t, const IdSummary& ks) {
    const int fl = halved ? qc.decide(a, t * BN + 32 * sub, 32, ks.lo, ks.hi) : qc.decide(a, t * BN, BN, ks.lo, ks.hi);
    return tile_value(fl | (DOC ? 0 : bmq.flags(t)), 0);
  };
  TileIter it;
  it.init_keys(kt_first, kt_last, qc.ksum, qc.g_lo, qc.g_hi, qc.g_glob, dec);   // its summaries travel together with Q, dO

  // the row operands have arrived before anything asynchronous is issued
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) { settle(qf[ks]); settle(dof[ks]); }
  settle(L_i);
  settle(delta_i);
  if (own_delta) {
    // the lane and its partner (lane ^ 32) hold the two halves of every 16 columns of the row
    float part = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < 8; ++t) part += float(of[ks][t]) * float(dof[ks][t]);
    delta_i = xhalf_sum(part);
    if (row >= 0 && g == 0 && wk.split == 0 && sub == 0) delp[row] = delta_i;   // for the dk/dv kernel
  }
  if (L_i == -INFINITY) L_i = INFINITY;  // row without any kept key: P = exp2(-inf) = 0

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

  f32x16 dq[DBN];
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[db][r] = 0.f;

  auto compute = [&](const int BUF, const int cur, const int flags) __attribute__((always_inline)) {
    const char* lk = smem + BUF * TILE_BYTES;
    const char* lv = smem + (2 + BUF) * TILE_BYTES;
    const char* lid = smem + 4 * TILE_BYTES + BUF * (BN * 4) + id_off;  // the tile's key ids
    const int n0 = cur * BN + key_off;
    if (flags & TF_SKIP) return;
    const bool need_lim = (flags & TF_LIM) != 0, need_doc = (flags & TF_DOC) != 0;
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // one 32-key block of the tile (kb a literal on the usual path: every offset an immediate)
    auto block = [&](const int kb) __attribute__((always_inline)) {
      f32x16 s = zero, dp = zero;
      __builtin_amdgcn_sched_barrier(0);
      // S and dP are accumulated alternately (an MFMA that accumulates onto the result of the MFMA
      // issued right before it waits a full extra MFMA time), operands a few LDS reads ahead.
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const vec8 kf = lds_row8<E>(lk + lo.row[ks] + kb * 32 * DL * 2);
        s = E::mfma32(kf, qf[ks], s);
        const vec8 vf = lds_row8<E>(lv + lo.row[ks] + kb * 32 * DL * 2);
        dp = E::mfma32(vf, dof[ks], dp);
      }
      {
        constexpr int NM = 2 * KS, PRE = NM < kDqPre ? NM : kDqPre;
        __builtin_amdgcn_sched_group_barrier(0x100, PRE, 0);
#pragma unroll
        for (int i = 0; i < NM - PRE; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, PRE, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // P and dS for this lane's 16 keys of the block
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = fast_exp2(__builtin_fmaf(s[r], c, -L_i));
        s[r] = p * (dp[r] - delta_i);
      }
      if (need_lim) {
        asm volatile("" ::: "memory");  // keep this a real (wave-uniform) branch: never if-converted
        mask_lim(s, qc.lim_i - n0 - 32 * kb - 4 * g, qc.low_i - n0 - 32 * kb - 4 * g, 0.f);
      }
      if (DOC && need_doc) {
        asm volatile("" ::: "memory");
        mask_doc(s, lid + kb * 32 * 4, eq_i, qc.glob_i, 0.f);
      }
      // dQ^T += K^T dS^T: K^T fragments (two transposed reads each) are requested PRE MFMAs ahead in
      // program order, dS is converted just in time; the scheduling barriers pin that order (left
      // to itself the scheduler puts every read right before its MFMA).
      {
        constexpr int NM = 2 * DBN, PRE = NM < kDqPre2 ? NM : kDqPre2;
        auto fetch = [&](const int i) __attribute__((always_inline)) {
          const int half = i / DBN, db = i % DBN;
          const int goff = (2 * kb + half) * 16 * DL * 2;
          return lds_tr8<E>(lk + lo.tr[db][0] + goff, lk + lo.tr[db][1] + goff);
        };
        __builtin_amdgcn_sched_barrier(0);
        vec8 ktf[NM];
#pragma unroll
        for (int i = 0; i < PRE; ++i) ktf[i] = fetch(i);
        vec8 dsf;
#pragma unroll
        for (int i = 0; i < NM; ++i) {
          if (i + PRE < NM) ktf[i + PRE] = fetch(i + PRE);
          if (i % DBN == 0) {
            const int half = i / DBN;
#pragma unroll
            for (int t = 0; t < 8; t += 2) {
              const typename E::vec2 pr = E::cvt2(s[8 * half + t], s[8 * half + t + 1]);
              dsf[t] = pr[0];
              dsf[t + 1] = pr[1];
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          dq[i % DBN] = E::mfma32(ktf[i], dsf, dq[i % DBN]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    block(0);
    if (!halved) block(1);   // (halved tiles: the lane offsets point into this wave's half, which is its whole tile)
  };

  // tile streams: K, V and (with ids) the 64 key ids of the tile, all straight into LDS
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  auto issue = [&](const int BUF, const int t) __attribute__((always_inline)) {
    ldK.issue(t * BN, smem + BUF * TILE_BYTES);
    ldV.issue(t * BN, smem + (2 + BUF) * TILE_BYTES);
    if (DOC && wave == 0) glb_load_lds4(ekp + t * BN + lane, smem + 4 * TILE_BYTES + BUF * (BN * 4));
  };
  int cur = it.next(dec);
  int cur_fl = it.flags;
  FA_STAMP(g_trace_dq, 2, FA_CLOCK());
  if (cur >= 0) issue(0, cur);
  while (cur >= 0) {
    int nxt = it.next(dec);
    wait_async_loads();
    __syncthreads();
    if (nxt >= 0) issue(1, nxt);
    compute(0, cur, cur_fl);
    FA_TRACE_ONLY(++tr_tiles;)
    cur = nxt; cur_fl = it.flags;
    if (cur < 0) break;
    nxt = it.next(dec);
    wait_async_loads();
    __syncthreads();
    if (nxt >= 0) issue(0, nxt);
    compute(1, cur, cur_fl);
    FA_TRACE_ONLY(++tr_tiles;)
    cur = nxt; cur_fl = it.flags;
  }
  FA_STAMP(g_trace_dq, 3, FA_CLOCK()); FA_STAMP(g_trace_dq, 5, tr_tiles);

  if (halved) {
    // the wave that took the second half of every key tile hands its partial dQ to the wave that took the
    // first half of the same rows, lane for lane, through the LDS the tile stream no longer needs
    __syncthreads();   // every wave is done with the last tile
    float* mb = reinterpret_cast<float*>(smem) + qc.rb * (16 * DBN * 64) + lane;
    if (sub == 1) {
#pragma unroll
      for (int db = 0; db < DBN; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) mb[(16 * db + r) * 64] = dq[db][r];
    }
    __syncthreads();
    if (sub == 0) {
#pragma unroll
      for (int db = 0; db < DBN; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq[db][r] += mb[(16 * db + r) * 64];
    }
  }
  const bool writer = !halved || sub == 0;   // the wave that holds the rows' result
  if (DOC && nsplit > 1) {
    // This workgroup saw one chunk of the keys: store the partial sum; the last chunk to arrive
    // adds them up in a fixed order and writes dQ.
    const int64_t tbase = (int64_t(b) * a.H + h) * a.split_tiles + wk.gt;
    float* po = a.sk_o + (tbase * a.split_k + wk.split) * (128 * D);
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        if (32 * db + 8 * q4 >= D || !writer) continue;
        f32x4 x = {dq[db][4 * q4 + 0], dq[db][4 * q4 + 1], dq[db][4 * q4 + 2], dq[db][4 * q4 + 3]};
        store_dev(po + part_index<D>(qc.rb, 4 * db + q4, lane) * 4, x);
      }
    if (!split_arrive(a.sk_cnt + tbase, nsplit)) { FA_STAMP(g_trace_dq, 4, FA_CLOCK()); return; }
    FA_STAMP(g_trace_dq, 6, FA_CLOCK());
    // (up to eight chunks are requested together, four or two steps of them: every device-scope load is a
    // round trip of its own, so they are put in flight side by side instead of one after the other)
    constexpr int C4 = D / 4;
    const float* bo = a.sk_o + tbase * a.split_k * (128 * D);
    const int* prm = a.perm + b * a.pm_bs + h * a.pm_hs + wk.tile * 128;
    auto finish_row = [&](int mrow, int c, f32x4 acc) __attribute__((always_inline)) {
      const typename E::vec2 x0 = E::cvt2(acc[0] * a.scale, acc[1] * a.scale);
      const typename E::vec2 x1 = E::cvt2(acc[2] * a.scale, acc[3] * a.scale);
      typename E::vec4 x = {x0[0], x0[1], x1[0], x1[1]};
      *reinterpret_cast<typename E::vec4*>(dqp + int64_t(mrow) * a.dq_rs + 4 * c) = x;
    };
    // NS chunk slots of IT steps each: 16 loads in flight per thread whatever the number of chunks
    auto merge_batched = [&](auto it_c, auto ns_c) __attribute__((always_inline)) {
      constexpr int IT = decltype(it_c)::value, NS = decltype(ns_c)::value;
      for (int i0 = threadIdx.x; i0 < 128 * C4; i0 += 256 * IT) {
        f32x4 x[IT][NS];
        int mrow[IT], cc[IT];
#pragma unroll
        for (int u = 0; u < IT; ++u) {
          const int i = i0 + 256 * u;
          int r, c;
          part_coords<D>(min(i, 128 * C4 - 1), r, c);
          cc[u] = c;
          mrow[u] = i < 128 * C4 ? prm[r] : -1;
          if (mrow[u] < 0) continue;   // no such row: nothing to fetch
#pragma unroll
          for (int sp = 0; sp < NS; ++sp) x[u][sp] = load_dev4(bo + min(sp, nsplit - 1) * (128 * D) + i * 4);
        }
#pragma unroll
        for (int u = 0; u < IT; ++u) {
          if (mrow[u] < 0) continue;
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int sp = 0; sp < NS; ++sp) {   // fixed order: chunk 0 first, as the one-by-one form below
            const float w = sp < nsplit ? 1.f : 0.f;
            acc[0] += w * x[u][sp][0]; acc[1] += w * x[u][sp][1]; acc[2] += w * x[u][sp][2]; acc[3] += w * x[u][sp][3];
          }
          finish_row(mrow[u], cc[u], acc);
        }
      }
    };
    if (nsplit <= 8) {   // (with 9 .. 16 chunks the plain loop below measured the same or better)
      if (nsplit <= 4) merge_batched(IntC<4>{}, IntC<4>{});
      else merge_batched(IntC<2>{}, IntC<8>{});
      FA_STAMP(g_trace_dq, 4, FA_CLOCK());
      return;
    }
    for (int i = threadIdx.x; i < 128 * C4; i += 256) {
      int r, c;
      part_coords<D>(i, r, c);
      const int mrow = prm[r];
      if (mrow < 0) continue;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < nsplit; ++sp) {
        const f32x4 x = load_dev4(bo + sp * (128 * D) + i * 4);
        acc[0] += x[0]; acc[1] += x[1]; acc[2] += x[2]; acc[3] += x[3];
      }
      finish_row(mrow, c, acc);
    }
    FA_STAMP(g_trace_dq, 4, FA_CLOCK());
    return;
  }

  // the rows leave through LDS (store_rows_through_lds): every wave is done with the last tile first; a halved
  // tile's writers use the part of LDS they have just read their partner's sums from
  if (!halved) __syncthreads();
  if (writer) {
    char* patch = smem + (halved ? qc.rb * (16 * DBN * 64 * 4) : wave * row_patch_bytes<D>());
    store_rows_through_lds<E, D, DBN>(patch, dq, a.scale, [&](const int r) -> T* {
      const int rr = __shfl(row, r);
      return rr >= 0 ? dqp + int64_t(rr) * a.dq_rs : nullptr;
    });
  }
  FA_STAMP(g_trace_dq, 4, FA_CLOCK());
}


template <typename Tag, int D, bool CAUSAL, bool DOC>
static int launch_one(const KArgs& a, hipStream_t s) {
  constexpr int BM = 128, BN = 64;
  const int nQt = (DOC ? a.Pp / BM : (a.M + BM - 1) / BM) + (DOC ? split_extra(a) : 0);
  const size_t lds = 4 * BN * (D < 32 ? 32 : D) * 2 + 2 * BN * 4;  // K, V double buffered + key ids
  auto kern = bwd_dq_kernel<Tag, D, CAUSAL, DOC>;
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
int trace_read_dq(long long* host, int n) { return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_trace_dq), size_t(n) * 8); }
#endif

int launch_bwd_dq(const KArgs& a, int dtype, int D, bool causal, bool doc, hipStream_t s) {
  return dtype == FA_DTYPE_BF16 ? launch_d<bf16_t>(a, D, causal, doc, s) : launch_d<fp16_t>(a, D, causal, doc, s);
}

}  // namespace fa
