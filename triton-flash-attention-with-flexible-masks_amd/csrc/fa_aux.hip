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
__global__ __launch_bounds__(256) void plan_k_kernel(const void* __restrict__ ids, int64_t s_b, int64_t s_h, int64_t s_r,
                                                     int L, int Lp, int nS, int H1, int* __restrict__ out32,
                                                     IdSummary* __restrict__ sum) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x * 4 + wave;
  if (tile >= nS) return;
  const int h = blockIdx.y, b = blockIdx.z;
  const int r = tile * kSumRows + lane;
  const bool valid = r < L;
  const int v = valid ? load_id<I64>(ids, b * s_b + h * s_h + int64_t(r) * s_r) : 0;
  out32[(int64_t(b) * H1 + h) * Lp + r] = v;
  const int lo = wave_min(valid ? v : 0x7fffffff);
  const int hi = wave_max(valid ? v : (int)0x80000000);
  if (lane == 0) {
    IdSummary s;
    s.lo = lo; s.hi = hi; s.glob = 0; s.rmin = tile * kSumRows; s.rmax = min(L, (tile + 1) * kSumRows) - 1;
    s.nvalid = s.rmax - s.rmin + 1; s.pad0 = s.pad1 = 0;
    sum[(int64_t(b) * H1 + h) * nS + tile] = s;
  }
}

// Query side: one workgroup per (batch, stored head).  Normalises the ids to int32,
// builds the local-rows-first permutation with a stable two-way partition
// (ballot + popcount prefix sums), then summarises every 64 entries of it.
template <bool I64>
__global__ __launch_bounds__(256) void plan_q_kernel(const void* __restrict__ ids, int64_t s_b, int64_t s_h, int64_t s_r,
                                                     int M, int Mp, int Pp, int H1, int* __restrict__ eq32,
                                                     int* __restrict__ perm, QHeader* __restrict__ hdr,
                                                     IdSummary* __restrict__ qsum) {
  __shared__ int sh_l[4], sh_g[4], sh_tot;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = blockIdx.x, b = blockIdx.y;
  const int64_t bh = int64_t(b) * H1 + h;
  int* eqp = eq32 + bh * Mp;
  int* pmp = perm + bh * Pp;
  const int64_t base = b * s_b + h * s_h;

  // pass 1: int32 copy of the ids and the number of local rows
  int cnt = 0;
  for (int r = tid; r < Mp; r += 256) {
    const int v = r < M ? load_id<I64>(ids, base + int64_t(r) * s_r) : 0;
    eqp[r] = v;
    cnt += (r < M && v < 0) ? 1 : 0;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) cnt += __shfl_xor(cnt, off);
  if (lane == 0) sh_l[wave] = cnt;
  __syncthreads();
  const int nL = sh_l[0] + sh_l[1] + sh_l[2] + sh_l[3];
  const int nG = M - nL;
  const int nLp = (nL + 127) / 128 * 128;
  __syncthreads();

  // pass 2: stable partition, 256 rows per step
  int baseL = 0, baseG = nLp;
  const unsigned long long lt = (1ull << lane) - 1ull;
  for (int r0 = 0; r0 < M; r0 += 256) {
    const int r = r0 + tid;
    const bool valid = r < M;
    const int v = valid ? eqp[r] : 0;  // written by this same thread in pass 1
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
    if (isL) pmp[baseL + offL + __builtin_popcountll(bl & lt)] = r;
    if (isG) pmp[baseG + offG + __builtin_popcountll(bg & lt)] = r;
    baseL += totL; baseG += totG;
    __syncthreads();
  }
  for (int i = nL + tid; i < nLp; i += 256) pmp[i] = -1;
  for (int i = nLp + nG + tid; i < Pp; i += 256) pmp[i] = -1;
  __threadfence_block();
  __syncthreads();

  // pass 3: summaries of the permuted order, one wave per 64 entries
  const int nT = Pp / kSumRows;
  for (int t = wave; t < nT; t += 4) {
    const int row = pmp[t * kSumRows + lane];
    const bool valid = row >= 0;
    const int v = valid ? eqp[row] : 0;
    const bool local = valid && v < 0;
    IdSummary s;
    s.lo = wave_min(local ? v : 0x7fffffff);
    s.hi = wave_max(local ? v : (int)0x80000000);
    s.rmin = wave_min(valid ? row : 0x7fffffff);
    s.rmax = wave_max(valid ? row : -1);
    s.glob = __builtin_amdgcn_ballot_w64(valid && v >= 0) != 0 ? 1 : 0;
    s.nvalid = __builtin_popcountll(__builtin_amdgcn_ballot_w64(valid));
    s.pad0 = s.pad1 = 0;
    if (lane == 0) qsum[bh * nT + t] = s;
  }
  if (tid == 0) {
    QHeader q;
    q.nL = nL; q.nG = nG; q.nLp = nLp; q.nT128 = (nLp + (nG + 127) / 128 * 128) / 128;
    hdr[bh] = q;
  }
}

int launch_mask_plan(const fa_params* p, const WsLayout& w, hipStream_t s) {
  char* ws = reinterpret_cast<char*>(p->workspace);
  const bool i64 = p->id_dtype == FA_IDTYPE_I64;
  {
    int* out32 = reinterpret_cast<int*>(ws + w.off_ek32);
    IdSummary* sum = reinterpret_cast<IdSummary*>(ws + w.off_ksum);
    const int64_t* st = p->ek_stride;
    dim3 grid((w.nKs + 3) / 4, w.Hk1, p->B);
    if (i64)
      hipLaunchKernelGGL(plan_k_kernel<true>, grid, dim3(256), 0, s, p->ek, st[0], st[1], st[2], p->N, w.Np, w.nKs, w.Hk1, out32, sum);
    else
      hipLaunchKernelGGL(plan_k_kernel<false>, grid, dim3(256), 0, s, p->ek, st[0], st[1], st[2], p->N, w.Np, w.nKs, w.Hk1, out32, sum);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  {
    int* eq32 = reinterpret_cast<int*>(ws + w.off_eq32);
    int* perm = reinterpret_cast<int*>(ws + w.off_perm);
    QHeader* hdr = reinterpret_cast<QHeader*>(ws + w.off_qhdr);
    IdSummary* sum = reinterpret_cast<IdSummary*>(ws + w.off_qsum);
    const int64_t* st = p->eq_stride;
    dim3 grid(w.Hq1, p->B);
    if (i64)
      hipLaunchKernelGGL(plan_q_kernel<true>, grid, dim3(256), 0, s, p->eq, st[0], st[1], st[2], p->M, w.Mp, w.Pp, w.Hq1, eq32, perm, hdr, sum);
    else
      hipLaunchKernelGGL(plan_q_kernel<false>, grid, dim3(256), 0, s, p->eq, st[0], st[1], st[2], p->M, w.Mp, w.Pp, w.Hq1, eq32, perm, hdr, sum);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  return 0;
}

template <bool CAUSAL, bool DOC>
__global__ __launch_bounds__(256) void mask_dump_kernel(const KArgs a, uint8_t* __restrict__ out) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  const int i = blockIdx.y;
  const int bh = blockIdx.z, b = bh / a.H, h = bh % a.H;
  if (j >= a.N) return;
  int eq_i = 0, ek_j = 0;
  if (DOC) {
    eq_i = a.eq32[b * a.eq_bs + h * a.eq_hs + i];
    ek_j = a.ek32[b * a.ek_bs + h * a.ek_hs + j];
  }
  out[(int64_t(bh) * a.M + i) * a.N + j] = keep_elem<CAUSAL, DOC>(i, j, a.gap, a.N, eq_i, ek_j) ? 1 : 0;
}

int launch_mask_dump(const KArgs& a, bool causal, bool doc, uint8_t* out, hipStream_t s) {
  dim3 grid((a.N + 255) / 256, a.M, a.B * a.H);
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
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int row = blockIdx.x * RPB + threadIdx.x / LPR;
  const int c = threadIdx.x % LPR;
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

template <typename Tag>
static int launch_delta_d(const KArgs& a, int D, hipStream_t s) {
  const int BH = a.B * a.H;
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
