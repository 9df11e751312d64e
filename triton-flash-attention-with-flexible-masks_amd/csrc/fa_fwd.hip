// Forward kernel: O = softmax(Q K^T * scale + mask) V and the log2-domain LSE.
// Replaces _fwd_kernel of the reference (flash_triton.py:25-141).
//
// Work decomposition (gfx950):
//   workgroup = 4 waves = 128 query rows; wave w owns rows 32w .. 32w+31.
//   K/V tiles of 64 keys are streamed global -> LDS with direct-to-LDS loads,
//   double buffered (2 x (K + V) x 64 x D x 2 bytes; 64 KB at D = 128).
//   S^T = K Q^T  : A = K rows from LDS, B = Q^T held in registers for the whole
//                  kernel; each lane then owns ONE query column and 16 keys of
//                  every 32-key block, so row max / row sum are in-lane plus one
//                  exchange with lane ^ 32.
//   O^T += V^T P^T : A = V^T via ds_read_b64_tr_b16, B = P^T taken straight from
//                  the S^T accumulators (the key order of the accumulator
//                  registers is absorbed into the V^T read pattern).
// Tiles of keys that cannot hold a kept element for the 128 rows (by the id
// summaries of the mask plan) are never loaded; per wave, tiles that are fully
// masked for its 32 rows are skipped and tiles that are fully kept take a path
// with no per-element mask work.
#include "fa_tile.h"

namespace fa {

template <typename Tag, int D, bool CAUSAL, bool DOC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void fwd_kernel(const KArgs a) {
  using E = Elem<Tag>;
  using T = typename E::scalar;
  using vec8 = typename E::vec8;
  constexpr int BM = 128, BN = 64, KS = D / 16, DBN = D / 32;
  constexpr int TILE_BYTES = BN * D * 2;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lq = lane & 31, g = lane >> 5;

  // blockIdx -> (q tile, batch*head): consecutive workgroup ids land on
  // different XCDs, so give each XCD whole heads (its L2 then holds that
  // head's K/V) and walk the q tiles from the causally heaviest down.
  const int nQt = (a.M + BM - 1) / BM;
  const int BH = a.B * a.H;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int bh = (idx / nQt) * 8 + xcd;
  if (bh >= BH) return;
  const int qt = nQt - 1 - (idx % nQt);
  const int b = bh / a.H, h = bh % a.H, hk = h / a.G;

  const T* qp = reinterpret_cast<const T*>(a.q) + b * a.q_bs + h * a.q_hs;
  const T* kp = reinterpret_cast<const T*>(a.k) + b * a.k_bs + hk * a.k_hs;
  const T* vp = reinterpret_cast<const T*>(a.v) + b * a.v_bs + hk * a.v_hs;
  T* op = reinterpret_cast<T*>(a.o) + b * a.o_bs + h * a.o_hs;
  float* lsep = a.lse + (int64_t(b) * a.H + h) * a.M;

  const int m0 = qt * BM;
  const int mw = m0 + wave * 32;
  const int row = mw + lq;
  const int rowc = row < a.M ? row : a.M - 1;

  // Q^T fragments (B operand): lane holds d = 16*ks + 8*g .. +7 of its query row.
  vec8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = *reinterpret_cast<const vec8*>(qp + int64_t(rowc) * a.q_rs + ks * 16 + g * 8);
  float c = a.scale_log2e;
  if (c < 0.f) {  // keep max(raw score) == max(scaled score): move the sign into Q
    c = -c;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = neg8<E>(qf[ks]);
  }

  // ids and summaries
  int eq_i = 0;
  int wq_lo = 0, wq_hi = -1, wq_glob = 1;  // this wave's 32 rows
  int gq_lo = 0, gq_hi = -1, gq_glob = 1;  // the workgroup's 128 rows
  const int* ekp = nullptr;
  const IdSummary* ksum = nullptr;
  if (DOC) {
    eq_i = a.eq32[b * a.eq_bs + h * a.eq_hs + rowc];
    ekp = a.ek32 + b * a.ek_bs + h * a.ek_hs;
    ksum = a.ksum + b * a.ks_bs + h * a.ks_hs;
    const IdSummary* qs = a.qsum + b * a.qs_bs + h * a.qs_hs;
    const IdSummary s0 = qs[m0 / kSumRows];
    gq_lo = s0.lo; gq_hi = s0.hi; gq_glob = s0.glob;
    if (m0 / kSumRows + 1 < a.nQs) {
      const IdSummary s1 = qs[m0 / kSumRows + 1];
      gq_lo = min(gq_lo, s1.lo); gq_hi = max(gq_hi, s1.hi); gq_glob |= s1.glob;
    }
    // wave-level summary from the lanes' own ids (both half waves hold the same 32 rows)
    const bool local = (eq_i < 0) && (row < a.M);
    int lo = local ? eq_i : 0x7fffffff, hi = local ? eq_i : (int)0x80000000;
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) {
      lo = min(lo, __shfl_xor(lo, off));
      hi = max(hi, __shfl_xor(hi, off));
    }
    wq_lo = lo; wq_hi = hi;
    wq_glob = __builtin_amdgcn_ballot_w64(eq_i >= 0 && row < a.M) != 0;
  }

  const int hi_key = CAUSAL ? min(a.N, a.gap + m0 + BM) : a.N;
  TileIter it;
  it.init(0, (hi_key + BN - 1) / BN, ksum, gq_lo, gq_hi, gq_glob, true);

  f32x16 o[DBN];
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;
  float m_run = -INFINITY;  // running max of raw scores (shared by lanes l, l^32)
  float l_run = 0.f;        // this lane's partial row sum

  int cur = it.next();
  int buf = 0;
  if (cur >= 0) {
    tile_load_async<T, D, BN, SWZ_ROW>(kp, a.k_rs, cur * BN, a.N, smem + 0 * TILE_BYTES);
    tile_load_async<T, D, BN, SWZ_TR>(vp, a.v_rs, cur * BN, a.N, smem + 2 * TILE_BYTES);
  }
  while (cur >= 0) {
    const int nxt = it.next();
    wait_async_loads();
    __syncthreads();
    if (nxt >= 0) {
      tile_load_async<T, D, BN, SWZ_ROW>(kp, a.k_rs, nxt * BN, a.N, smem + (buf ^ 1) * TILE_BYTES);
      tile_load_async<T, D, BN, SWZ_TR>(vp, a.v_rs, nxt * BN, a.N, smem + (2 + (buf ^ 1)) * TILE_BYTES);
    }
    const char* lk = smem + buf * TILE_BYTES;
    const char* lv = smem + (2 + buf) * TILE_BYTES;
    const int n0 = cur * BN;

    // wave-level decisions for this tile
    bool skip = CAUSAL && (n0 > a.gap + mw + 31);
    bool need_mask = (n0 + BN > a.N) || (CAUSAL && (n0 + BN - 1 > a.gap + mw));
    if (DOC) {
      const IdSummary ks = ksum[cur];
      skip = skip || !doc_may_keep(wq_lo, wq_hi, wq_glob, ks.lo, ks.hi);
      need_mask = need_mask || !doc_all_keep(wq_lo, wq_hi, ks.lo, ks.hi);
    }
    if (!skip) {
      f32x16 s[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const vec8 kf = frag_row<E, D, SWZ_ROW>(lk, kb * 32 + lq, 2 * ks + g);
          s[kb] = E::mfma32(kf, qf[ks], s[kb]);
        }
      }
      if (need_mask) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            const int j0 = n0 + 32 * kb + 8 * q4 + 4 * g;
            i32x4 ekv = {0, 0, 0, 0};
            if (DOC) ekv = *reinterpret_cast<const i32x4*>(ekp + j0);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const bool keep = keep_elem<CAUSAL, DOC>(row, j0 + t, a.gap, a.N, eq_i, ekv[t]);
              s[kb][4 * q4 + t] = keep ? s[kb][4 * q4 + t] : -INFINITY;
            }
          }
        }
      }
      // online softmax in the exp2 domain
      float mx = s[0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kb][r]);
      mx = xhalf_max(mx);
      const float m_new = fmaxf(m_run, mx);
      const float msc = (m_new == -INFINITY) ? 0.f : m_new * c;
      const float alpha = fast_exp2(m_run * c - msc);
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fast_exp2(__builtin_fmaf(s[kb][r], c, -msc));
          s[kb][r] = p;
          psum += p;
        }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int db = 0; db < DBN; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
      // O^T += V^T P^T, 16 keys per MFMA
#pragma unroll
      for (int c16 = 0; c16 < 4; ++c16) {
        vec8 pf;
#pragma unroll
        for (int t = 0; t < 8; t += 2) {
          const typename E::vec2 pr = E::cvt2(s[c16 >> 1][8 * (c16 & 1) + t], s[c16 >> 1][8 * (c16 & 1) + t + 1]);
          pf[t] = pr[0];
          pf[t + 1] = pr[1];
        }
#pragma unroll
        for (int db = 0; db < DBN; ++db) {
          const vec8 vf = frag_tr<E, D, SWZ_TR>(lv, 16 * c16, db);
          o[db] = E::mfma32(vf, pf, o[db]);
        }
      }
    }
    cur = nxt;
    buf ^= 1;
  }

  // epilogue: normalise, write O and LSE
  const float l_tot = xhalf_sum(l_run);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (row < a.M) {
    if (g == 0) lsep[row] = l_tot > 0.f ? m_run * c + fast_log2(l_tot) : -INFINITY;
    T* orow = op + int64_t(row) * a.o_rs;
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const typename E::vec2 x0 = E::cvt2(o[db][4 * q4 + 0] * inv, o[db][4 * q4 + 1] * inv);
        const typename E::vec2 x1 = E::cvt2(o[db][4 * q4 + 2] * inv, o[db][4 * q4 + 3] * inv);
        typename E::vec4 x = {x0[0], x0[1], x1[0], x1[1]};
        *reinterpret_cast<typename E::vec4*>(orow + 32 * db + 8 * q4 + 4 * g) = x;
      }
  }
}

template <typename Tag, int D, bool CAUSAL, bool DOC>
static int launch_one(const KArgs& a, hipStream_t s) {
  constexpr int BM = 128, BN = 64;
  const int nQt = (a.M + BM - 1) / BM;
  const int slots = (a.B * a.H + 7) / 8;
  const size_t lds = 4 * BN * D * 2;
  auto kern = fwd_kernel<Tag, D, CAUSAL, DOC>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(8 * slots * nQt), dim3(256), lds, s, a);
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
    default: return -1;
  }
}

int launch_fwd(const KArgs& a, int dtype, int D, bool causal, bool doc, hipStream_t s) {
  return dtype == FA_DTYPE_BF16 ? launch_d<bf16_t>(a, D, causal, doc, s) : launch_d<fp16_t>(a, D, causal, doc, s);
}

}  // namespace fa
