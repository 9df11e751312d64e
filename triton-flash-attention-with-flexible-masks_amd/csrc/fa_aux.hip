// Small kernels around the attention kernels proper:
//   * mask plan : normalise eq/ek to int32 and write per-64-row id summaries
//                 (no counterpart in the reference, which tests every tile)
//   * mask dump : keep(i, j) as bytes, through the same keep_elem() the compute
//                 kernels use (mask expression of flash_triton.py:103-116)
//   * delta     : delta = rowsum(O * dO), replaces _bwd_preprocess
//                 (flash_triton.py:143-173)
#include "fa_common.h"

namespace fa {

FA_DEV int sat32(long long v) {
  return v > 2147483647LL ? 2147483647 : (v < -2147483648LL ? (int)-2147483648LL : (int)v);
}

template <bool I64>
FA_DEV int load_id(const void* ids, int64_t off) {
  return I64 ? sat32(reinterpret_cast<const long long*>(ids)[off]) : reinterpret_cast<const int*>(ids)[off];
}

FA_DEV int wave_min(int v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = min(v, __shfl_xor(v, off));
  return v;
}
FA_DEV int wave_max(int v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = max(v, __shfl_xor(v, off));
  return v;
}

// Key side: one wave per summary tile of 64 keys; 4 tiles per workgroup.
template <bool I64>
FA_DEV void plan_k_body(const int bx, const void* __restrict__ ids, int64_t s_b, int64_t s_h, int64_t s_r,
                        int L, int Lp, int nS, int H1, int* __restrict__ out32, IdSummary* __restrict__ sum) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = bx * 4 + wave;
  const int h = blockIdx.y, b = blockIdx.z;
  if (tile >= nS || h >= H1) return;
  const int r = tile * kSumRows + lane;
  const bool valid = r < L;
  const int v = valid ? load_id<I64>(ids, b * s_b + h * s_h + int64_t(r) * s_r) : 0;
  out32[(int64_t(b) * H1 + h) * Lp + r] = v;
  const int lo = wave_min(valid ? v : 0x7fffffff);
  const int hi = wave_max(valid ? v : (int)0x80000000);
  if (lane == 0) {
    IdSummary s;
    s.lo = lo; s.hi = hi; s.glob = 0; s.rmin = tile * kSumRows; s.rmax = min(L, (tile + 1) * kSumRows) - 1;
    s.nvalid = s.rmax - s.rmin + 1; s.kfirst = 0; s.klast = 0;
    sum[(int64_t(b) * H1 + h) * nS + tile] = s;
  }
}

// Query side, step 1: one workgroup per chunk of kPlanChunk rows.  Writes the int32 copy of the
// ids, the number of local rows (eq < 0) of the chunk, and pre-fills the chunk's share of the
// permuted order with -1.
constexpr int kPlanChunk = 1024;

template <bool I64>
FA_DEV void plan_count_body(const int ch, const void* __restrict__ ids, int64_t s_b, int64_t s_h, int64_t s_r,
                            int M, int Mp, int Pp, int nCh, int H1, int* __restrict__ eq32,
                            int* __restrict__ perm, int* __restrict__ peq,
                            int* __restrict__ ppos, int* __restrict__ cnt) {
  __shared__ int sh[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = blockIdx.y, b = blockIdx.z;
  if (h >= H1) return;   // (uniform over the workgroup)
  const int64_t bh = int64_t(b) * H1 + h;
  const int64_t base = b * s_b + h * s_h;
  int c = 0;
#pragma unroll
  for (int k = 0; k < kPlanChunk / 256; ++k) {
    const int r = ch * kPlanChunk + k * 256 + tid;
    if (r < Mp) {
      const int v = r < M ? load_id<I64>(ids, base + int64_t(r) * s_r) : 0;
      eq32[bh * Mp + r] = v;
      c += (r < M && v < 0) ? 1 : 0;
    }
  }
  // the last chunk also covers the tail of the permuted order (Pp > M)
  const int p_end = ch == nCh - 1 ? Pp : min(Pp, (ch + 1) * kPlanChunk);
  for (int i = ch * kPlanChunk + tid; i < p_end; i += 256) {
    perm[bh * Pp + i] = -1;
    peq[bh * Pp + i] = 0;
    ppos[bh * Pp + i] = -1;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) c += __shfl_xor(c, off);
  if (lane == 0) sh[wave] = c;
  __syncthreads();
  if (tid == 0) cnt[bh * nCh + ch] = sh[0] + sh[1] + sh[2] + sh[3];
}

// The two kernels above in one launch (they do not depend on each other, and every launch of a kernel this
// small costs more in the gap to the next one than in its run time): workgroups [0, nKb) take the key side,
// the rest the query side; grid.y covers the larger of the two head counts.
struct PlanSide { const void* ids; int64_t s_b, s_h, s_r; int L, Lp, H1; };
template <bool I64>
__global__ __launch_bounds__(256) void plan_kc_kernel(PlanSide k, int nS, int nKb, int* __restrict__ ek32, IdSummary* __restrict__ ksum,
                                                      PlanSide q, int Pp, int nCh, int* __restrict__ eq32, int* __restrict__ perm,
                                                      int* __restrict__ peq, int* __restrict__ ppos, int* __restrict__ cnt) {
  if ((int)blockIdx.x < nKb) plan_k_body<I64>(blockIdx.x, k.ids, k.s_b, k.s_h, k.s_r, k.L, k.Lp, nS, k.H1, ek32, ksum);
  else plan_count_body<I64>(blockIdx.x - nKb, q.ids, q.s_b, q.s_h, q.s_r, q.L, q.Lp, Pp, nCh, q.H1, eq32, perm, peq, ppos, cnt);
}

// Step 2: stable two-way partition.  Every chunk derives its output offsets from the counts of
// the chunks before it, then places its rows with ballot / popcount prefix sums: local rows go to
// perm[0 .. nL), global rows to perm[nLp .. nLp + nG), both in ascending row order.
__global__ __launch_bounds__(256) void plan_scatter_kernel(int M, int Mp, int Pp, int nCh, int H1,
                                                           const int* __restrict__ eq32, const int* __restrict__ cnt,
                                                           int* __restrict__ perm, int* __restrict__ peq,
                                                           int* __restrict__ ppos, const int* __restrict__ qpos, int64_t qp_bs,
                                                           int gap, QHeader* __restrict__ hdr) {
  __shared__ int sh_l[4], sh_g[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ch = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int64_t bh = int64_t(b) * H1 + h;
  const int* eqp = eq32 + bh * Mp;
  int* pmp = perm + bh * Pp;
  int* pqp = peq + bh * Pp;
  int* ppp = ppos + bh * Pp;
  int before = 0, nL = 0;
  for (int k = 0; k < nCh; ++k) {
    const int c = cnt[bh * nCh + k];
    before += k < ch ? c : 0;
    nL += c;
  }
  const int nG = M - nL;
  const int nLp = (nL + kPermAlign - 1) / kPermAlign * kPermAlign;
  int baseL = before;
  int baseG = nLp + (min(M, ch * kPlanChunk) - before);  // global rows before this chunk
  const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
  for (int k = 0; k < kPlanChunk / 256; ++k) {
    const int r = ch * kPlanChunk + k * 256 + tid;
    const bool valid = r < M;
    const int v = valid ? eqp[r] : 0;
    // key position of the row's diagonal: the caller's, or the one offset of flash_triton.py:521
    const int ps = !valid ? -1 : (qpos != nullptr ? clamp_pos(qpos[b * qp_bs + r]) : gap + r);
    const bool isL = valid && v < 0, isG = valid && v >= 0;
    const unsigned long long bl = __builtin_amdgcn_ballot_w64(isL), bg = __builtin_amdgcn_ballot_w64(isG);
    if (lane == 0) { sh_l[wave] = __builtin_popcountll(bl); sh_g[wave] = __builtin_popcountll(bg); }
    __syncthreads();
    int offL = 0, offG = 0, totL = 0, totG = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int cl = sh_l[w], cg = sh_g[w];
      if (w < wave) { offL += cl; offG += cg; }
      totL += cl; totG += cg;
    }
    if (isL) { const int pos = baseL + offL + __builtin_popcountll(bl & lt); pmp[pos] = r; pqp[pos] = v; ppp[pos] = ps; }
    if (isG) { const int pos = baseG + offG + __builtin_popcountll(bg & lt); pmp[pos] = r; pqp[pos] = v; ppp[pos] = ps; }
    baseL += totL; baseG += totG;
    __syncthreads();
  }
  if (ch == 0 && tid == 0) {
    QHeader q;
    q.nL = nL; q.nG = nG; q.nLp = nLp; q.nT128 = (nLp + (nG + 127) / 128 * 128) / 128;
    q.k0 = 0x7fffffff; q.pad[0] = q.pad[1] = q.pad[2] = 0;   // k0: lowered by plan_qsum_kernel
    hdr[bh] = q;
  }
}

// Step 3: one wave per 64 entries of the permuted order: id / row-index summary, and the range
// [kfirst, klast] of key tiles the entry's rows can need (by the key summaries and the causal
// bound), so that the compute kernels start their tile search in the right place.
__global__ __launch_bounds__(256) void plan_qsum_kernel(int Pp, int nQs, int nKs, int H1, int HK1, int causal, int kend_min,
                                                        const int* __restrict__ perm, const int* __restrict__ peq,
                                                        const int* __restrict__ ppos,
                                                        const IdSummary* __restrict__ ksum, IdSummary* __restrict__ qsum,
                                                        int* __restrict__ sk_cnt, int n_sk, QHeader* __restrict__ hdr) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // the arrival counters of the split-key merge start every forward at zero
  if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0)
    for (int i = threadIdx.x; i < n_sk; i += 256) sk_cnt[i] = 0;
  const int t = blockIdx.x * 4 + wave;
  if (t >= nQs) return;
  const int h = blockIdx.y, b = blockIdx.z;
  const int64_t bh = int64_t(b) * H1 + h;
  const int row = perm[bh * Pp + t * kSumRows + lane];
  const int v = peq[bh * Pp + t * kSumRows + lane];
  const int ps = ppos[bh * Pp + t * kSumRows + lane];
  const bool valid = row >= 0;
  const bool local = valid && v < 0;
  IdSummary s;
  s.lo = wave_min(local ? v : 0x7fffffff);
  s.hi = wave_max(local ? v : (int)0x80000000);
  s.rmin = wave_min(valid ? ps : 0x7fffffff);
  s.rmax = wave_max(valid ? ps : -1);
  s.glob = __builtin_amdgcn_ballot_w64(valid && v >= 0) != 0 ? 1 : 0;
  s.nvalid = __builtin_popcountll(__builtin_amdgcn_ballot_w64(valid));
  int kfirst = 0x7fffffff, klast = -1;
  if (H1 == HK1) {  // ids of both sides stored per the same heads: narrow the key range
    const IdSummary* ks = ksum + bh * nKs;
    // kend_min: key tiles of a prefix that every row sees whatever its causal bound
    const int kend = causal ? min(nKs, max(s.rmax / kSumRows + 1, kend_min)) : nKs;
    for (int k0 = 0; k0 < kend; k0 += 64) {
      const int k = k0 + lane;
      bool cand = false;
      if (k < kend) {
        const IdSummary kk = ks[k];
        cand = doc_may_keep(s.lo, s.hi, s.glob, kk.lo, kk.hi);
      }
      kfirst = min(kfirst, cand ? k : 0x7fffffff);
      klast = max(klast, cand ? k : -1);
    }
    kfirst = wave_min(kfirst);
    klast = wave_max(klast);
  } else {
    kfirst = 0; klast = nKs - 1;
  }
  s.kfirst = s.nvalid > 0 ? kfirst : 0x7fffffff;
  s.klast = s.nvalid > 0 ? klast : -1;
  if (lane == 0) {
    qsum[bh * nQs + t] = s;
    // first key tile any local row can need (the header starts at "none", set by plan_scatter_kernel)
    if (s.nvalid > 0 && s.glob == 0) atomicMin(&hdr[bh].k0, s.klast >= s.kfirst ? s.kfirst : 0x7fffffff);
  }
}

int launch_mask_plan(const fa_params* p, const WsLayout& w, hipStream_t s) {
  char* ws = reinterpret_cast<char*>(p->workspace);
  const bool i64 = p->id_dtype == FA_IDTYPE_I64;
  int* eq32 = reinterpret_cast<int*>(ws + w.off_eq32);
  int* ek32 = reinterpret_cast<int*>(ws + w.off_ek32);
  int* perm = reinterpret_cast<int*>(ws + w.off_perm);
  int* peq = reinterpret_cast<int*>(ws + w.off_peq);
  int* ppos = reinterpret_cast<int*>(ws + w.off_ppos);
  int* cnt = reinterpret_cast<int*>(ws + w.off_cnt);
  QHeader* hdr = reinterpret_cast<QHeader*>(ws + w.off_qhdr);
  IdSummary* qsum = reinterpret_cast<IdSummary*>(ws + w.off_qsum);
  IdSummary* ksum = reinterpret_cast<IdSummary*>(ws + w.off_ksum);
  hipError_t e;
  {
    const int64_t* sk = p->ek_stride;
    const int64_t* sq = p->eq_stride;
    const PlanSide ks = {p->ek, sk[0], sk[1], sk[2], p->N, w.Np, w.Hk1};
    const PlanSide qs = {p->eq, sq[0], sq[1], sq[2], p->M, w.Mp, w.Hq1};
    const int nKb = (w.nKs + 3) / 4;
    dim3 grid_kc(nKb + w.nCh, w.Hk1 > w.Hq1 ? w.Hk1 : w.Hq1, p->B);
    if (i64)
      hipLaunchKernelGGL(plan_kc_kernel<true>, grid_kc, dim3(256), 0, s, ks, w.nKs, nKb, ek32, ksum, qs, w.Pp, w.nCh, eq32, perm, peq, ppos, cnt);
    else
      hipLaunchKernelGGL(plan_kc_kernel<false>, grid_kc, dim3(256), 0, s, ks, w.nKs, nKb, ek32, ksum, qs, w.Pp, w.nCh, eq32, perm, peq, ppos, cnt);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
    dim3 grid(w.nCh, w.Hq1, p->B);
    const int gap = p->N > p->M ? p->N - p->M : 0;
    hipLaunchKernelGGL(plan_scatter_kernel, grid, dim3(256), 0, s, p->M, w.Mp, w.Pp, w.nCh, w.Hq1, eq32, cnt, perm, peq, ppos,
                       p->causal ? p->qpos : nullptr, p->qpos_stride, gap, hdr);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
    hipLaunchKernelGGL(plan_qsum_kernel, dim3((w.nQs + 3) / 4, w.Hq1, p->B), dim3(256), 0, s, w.Pp, w.nQs, w.nKs, w.Hq1, w.Hk1,
                       p->causal ? 1 : 0, p->prefix > 0 ? ((p->prefix < p->N ? p->prefix : p->N) - 1) / kSumRows + 1 : 0, perm, peq, ppos, ksum, qsum, reinterpret_cast<int*>(ws + w.off_sk_cnt),
                       p->B * p->H * w.split.tiles, hdr);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  return 0;
}

template <bool CAUSAL, bool DOC>
__global__ __launch_bounds__(256) void mask_dump_kernel(const KArgs a, uint8_t* __restrict__ out) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= a.N) return;
  // rows and (batch, head) pairs are walked with the grid's stride: grid dimensions y and z stop at 65535
  for (int bh = blockIdx.z; bh < a.B * a.H; bh += gridDim.z) {
    const int b = bh / a.H, h = bh % a.H;
    const int ek_j = DOC ? a.ek32[b * a.ek_bs + h * a.ek_hs + j] : 0;
    for (int i = blockIdx.y; i < a.M; i += gridDim.y) {
      const int eq_i = DOC ? a.eq32[b * a.eq_bs + h * a.eq_hs + i] : 0;
      const int pos_i = (DOC && CAUSAL && a.qpos != nullptr) ? clamp_pos(a.qpos[b * a.qp_bs + i]) : a.gap + i;
      bool keep = keep_elem<CAUSAL, DOC>(pos_i, j, a.N, eq_i, ek_j, a.win, a.pfx_m1);
      if (!DOC && a.bmask != nullptr)
        keep = keep && a.bmask[b * a.bm_bs + h * a.bm_hs + int64_t(i / FA_MASK_BLOCK) * a.bm_rs + j / FA_MASK_BLOCK] != 0;
      out[(int64_t(bh) * a.M + i) * a.N + j] = keep ? 1 : 0;
    }
  }
}

int launch_mask_dump(const KArgs& a, bool causal, bool doc, uint8_t* out, hipStream_t s) {
  dim3 grid((a.N + 255) / 256, a.M < 65535 ? a.M : 65535, a.B * a.H < 65535 ? a.B * a.H : 65535);
  if (causal && doc) hipLaunchKernelGGL((mask_dump_kernel<true, true>), grid, dim3(256), 0, s, a, out);
  else if (causal) hipLaunchKernelGGL((mask_dump_kernel<true, false>), grid, dim3(256), 0, s, a, out);
  else if (doc) hipLaunchKernelGGL((mask_dump_kernel<false, true>), grid, dim3(256), 0, s, a, out);
  else hipLaunchKernelGGL((mask_dump_kernel<false, false>), grid, dim3(256), 0, s, a, out);
  return (int)hipGetLastError();
}

// delta[b,h,m] = sum_d O[b,h,m,d] * dO[b,h,m,d]; D/8 lanes per row, 16-byte loads.
template <typename Tag, int D>
__global__ __launch_bounds__(256) void delta_kernel(const KArgs a) {
  using E = Elem<Tag>;
  using T = typename E::scalar;
  using vec8 = typename E::vec8;
  constexpr int LPR = D / 8;         // lanes per row
  constexpr int RPB = 256 / LPR;     // rows per block
  const int row = blockIdx.x * RPB + threadIdx.x / LPR;
  const int c = threadIdx.x % LPR;
  // (batch, head) pairs are walked with the grid's stride: grid dimension y stops at 65535
  for (int bh = blockIdx.y; bh < a.B * a.H; bh += gridDim.y) {
    const int b = bh / a.H, h = bh % a.H;
    float acc = 0.f;
    if (row < a.M) {
      const T* op = reinterpret_cast<const T*>(a.o) + b * a.o_bs + h * a.o_hs + int64_t(row) * a.o_rs + c * 8;
      const T* dp = reinterpret_cast<const T*>(a.dout) + b * a.do_bs + h * a.do_hs + int64_t(row) * a.do_rs + c * 8;
      const vec8 x = *reinterpret_cast<const vec8*>(op);
      const vec8 y = *reinterpret_cast<const vec8*>(dp);
#pragma unroll
      for (int t = 0; t < 8; ++t) acc += float(x[t]) * float(y[t]);
    }
#pragma unroll
    for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off);
    if (c == 0 && row < a.M) a.delta[(int64_t(b) * a.H + h) * a.M + row] = acc;
  }
}

template <typename Tag>
static int launch_delta_d(const KArgs& a, int D, hipStream_t s) {
  const int BH = a.B * a.H < 65535 ? a.B * a.H : 65535;
  switch (D) {
    case 128: hipLaunchKernelGGL((delta_kernel<Tag, 128>), dim3((a.M + 15) / 16, BH), dim3(256), 0, s, a); break;
    case 64: hipLaunchKernelGGL((delta_kernel<Tag, 64>), dim3((a.M + 31) / 32, BH), dim3(256), 0, s, a); break;
    case 32: hipLaunchKernelGGL((delta_kernel<Tag, 32>), dim3((a.M + 63) / 64, BH), dim3(256), 0, s, a); break;
    case 16: hipLaunchKernelGGL((delta_kernel<Tag, 16>), dim3((a.M + 127) / 128, BH), dim3(256), 0, s, a); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}

int launch_bwd_delta(const KArgs& a, int dtype, int D, hipStream_t s) {
  return dtype == FA_DTYPE_BF16 ? launch_delta_d<bf16_t>(a, D, s) : launch_delta_d<fp16_t>(a, D, s);
}

}  // namespace fa
