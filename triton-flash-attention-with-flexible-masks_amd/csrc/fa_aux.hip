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

// One wave per summary tile of kSumRows (= 64) rows; 4 tiles per workgroup.
template <bool I64>
__global__ __launch_bounds__(256) void plan_kernel(const void* __restrict__ ids, int64_t s_b, int64_t s_h, int64_t s_r,
                                                   int L, int Lp, int nS, int H1, int* __restrict__ out32,
                                                   IdSummary* __restrict__ sum, int query_side) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x * 4 + wave;
  if (tile >= nS) return;
  const int h = blockIdx.y, b = blockIdx.z;
  const int r = tile * kSumRows + lane;
  const bool valid = r < L;
  int v = 0;
  if (valid) {
    const int64_t off = b * s_b + h * s_h + int64_t(r) * s_r;
    v = I64 ? sat32(reinterpret_cast<const long long*>(ids)[off]) : reinterpret_cast<const int*>(ids)[off];
  }
  out32[(int64_t(b) * H1 + h) * Lp + r] = v;
  const bool use = valid && (query_side ? v < 0 : true);
  int lo = use ? v : 0x7fffffff;
  int hi = use ? v : (int)0x80000000;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    lo = min(lo, __shfl_xor(lo, off));
    hi = max(hi, __shfl_xor(hi, off));
  }
  const int glob = query_side ? (__builtin_amdgcn_ballot_w64(valid && v >= 0) != 0) : 0;
  if (lane == 0) {
    IdSummary s;
    s.lo = lo; s.hi = hi; s.glob = glob; s.pad = 0;
    sum[(int64_t(b) * H1 + h) * nS + tile] = s;
  }
}

int launch_mask_plan(const fa_params* p, const WsLayout& w, hipStream_t s) {
  char* ws = reinterpret_cast<char*>(p->workspace);
  const bool i64 = p->id_dtype == FA_IDTYPE_I64;
  for (int side = 0; side < 2; ++side) {
    const bool qs = side == 0;
    const void* ids = qs ? p->eq : p->ek;
    const int64_t* st = qs ? p->eq_stride : p->ek_stride;
    const int L = qs ? p->M : p->N, Lp = qs ? w.Mp : w.Np, nS = qs ? w.nQs : w.nKs, H1 = qs ? w.Hq1 : w.Hk1;
    int* out32 = reinterpret_cast<int*>(ws + (qs ? w.off_eq32 : w.off_ek32));
    IdSummary* sum = reinterpret_cast<IdSummary*>(ws + (qs ? w.off_qsum : w.off_ksum));
    dim3 grid((nS + 3) / 4, H1, p->B);
    if (i64)
      hipLaunchKernelGGL(plan_kernel<true>, grid, dim3(256), 0, s, ids, st[0], st[1], st[2], L, Lp, nS, H1, out32, sum, qs ? 1 : 0);
    else
      hipLaunchKernelGGL(plan_kernel<false>, grid, dim3(256), 0, s, ids, st[0], st[1], st[2], L, Lp, nS, H1, out32, sum, qs ? 1 : 0);
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
