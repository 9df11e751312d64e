// The operator for fp32 tensors: forward, delta, dk/dv and dq with `v_mfma_f32_32x32x2_f32`
// (products and accumulation in fp32 throughout).  The reference accepts fp32 tensors like any
// other float type (flash_triton.py:508-564 has no dtype check; its score and probability
// matrices then stay fp32, :88,126) -- this is that case, at full fp32 precision.
//
// Shape of all three kernels: 4 waves per workgroup, ONE wave per SIMD, so that a wave may use the
// whole 512-entry register file: the operands of the side a wave owns (32 query rows, or 32 keys)
// and its accumulators stay in registers for the whole kernel; the other side is streamed through
// LDS in tiles of 32 rows (the next tile travels global -> registers while the current one is
// used).  A 32x32x2 MFMA takes ONE operand element per lane, so every operand read from LDS is a
// single `ds_read_b32` per lane and a transposed operand costs the same as a plain one: rows are
// padded to D + 1 floats, which makes both access patterns conflict-free.
//   forward  S^T = K Q^T | online softmax (exp2 domain) | O^T += V^T P^T          flash_triton.py:26-172
//   dq       S^T = K Q^T, dP^T = V dO^T | dS = P (dP - delta) | dQ^T += K^T dS^T  flash_triton.py:325-433
//   dk/dv    S = Q K^T, dP = dO V^T | P, dS | dV^T += dO^T P, dK^T += Q^T dS      flash_triton.py:175-321
// In the accumulator layout of a 32x32 MFMA a lane owns one column (its query row, or its key) and
// rows 8*q4 + 4*(lane/32) + t; P^T / dS^T / P / dS are consumed as the B operand of the next
// product straight from those registers (the contraction index is walked in that same order on
// the A side), so nothing is exchanged or transposed.
// Masks: the element masks are the routines of the 16-bit kernels (same accumulator layout); a wave
// skips a 32x32 block when the causal bound or the id intervals of its rows and of the block's keys
// (reduced from the ids staged with the tile) exclude every pair.  Without ids rows are walked in
// natural order.  With ids the query side is walked in the permuted order of the mask plan (local
// rows first, then global rows: a tile of local rows meets the keys of its own documents only),
// rows are gathered through the permutation, causal terms use the diagonal positions the plan
// stored, and tiles that the plan's summaries rule out for the whole workgroup are not loaded.
#include "fa_tile.h"

namespace fa {
namespace {

FA_DEV f32x16 mfma_f32(float a, float b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }

constexpr int kRows = 32;       // rows of a streamed tile
constexpr int kThreads = 256;

// A [32 x D] tile on its way from global memory to LDS, held in registers in between.
template <int D>
struct TileRegs {
  static constexpr int C4 = D / 4, N4 = kRows * C4, PER = (N4 + kThreads - 1) / kThreads;
  f32x4 v[PER];
  // rows row0 .. row0+31 of a matrix with `nrows` rows; rows past the end read as zero
  FA_DEV void load(const float* base, int64_t rs, int row0, int nrows) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = threadIdx.x + kThreads * i;
      const int r = idx / C4, c4 = idx % C4;
      const bool ok = idx < N4 && row0 + r < nrows;
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      v[i] = ok ? *reinterpret_cast<const f32x4*>(base + int64_t(row0 + r) * rs + 4 * c4) : z;
    }
  }
  // the same for a tile whose rows are rows[0..31] of the matrix (-1: no row, reads as zero)
  FA_DEV void load_rows(const float* base, int64_t rs, const int* rows) {
    int ri[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = threadIdx.x + kThreads * i;
      ri[i] = idx < N4 ? rows[idx / C4] : -1;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int c4 = (threadIdx.x + kThreads * i) % C4;
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      v[i] = ri[i] >= 0 ? *reinterpret_cast<const f32x4*>(base + int64_t(ri[i]) * rs + 4 * c4) : z;
    }
  }
  FA_DEV void store(float* lds) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = threadIdx.x + kThreads * i;
      const int r = idx / C4, c4 = idx % C4;
      if (idx < N4) {
        float* d = lds + r * (D + 1) + 4 * c4;
        d[0] = v[i][0]; d[1] = v[i][1]; d[2] = v[i][2]; d[3] = v[i][3];
      }
    }
  }
};

// min / max over the 32 lanes of a half wave (both halves hold the same 32 rows)
FA_DEV int half_min(int x) {
#pragma unroll
  for (int off = 16; off >= 1; off >>= 1) x = min(x, __shfl_xor(x, off));
  return x;
}
FA_DEV int half_max(int x) {
#pragma unroll
  for (int off = 16; off >= 1; off >>= 1) x = max(x, __shfl_xor(x, off));
  return x;
}

// A run of N MFMAs whose A operands come from LDS: the operands are requested a chunk of CH ahead
// of the MFMAs that consume them, in program order (left to itself the compiler puts a read, a
// full wait and its MFMAs back to back).  rd(i) reads operand i, mm(i, a) issues MFMA i.
template <int N, int CH, typename RD, typename MM>
FA_DEV void pipelined(RD&& rd, MM&& mm) {
  static_assert(N % CH == 0, "chunking");
  float buf[2][CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) buf[0][i] = rd(i);
#pragma unroll
  for (int c = 0; c < N / CH; ++c) {
    if (c + 1 < N / CH) {
#pragma unroll
      for (int i = 0; i < CH; ++i) buf[(c + 1) & 1][i] = rd((c + 1) * CH + i);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < CH; ++i) mm(c * CH + i, buf[c & 1][i]);
    __builtin_amdgcn_sched_barrier(0);
  }
}
constexpr int kChunk = 8;

// (min, max, or) of one value triple per wave over the 4 waves of the workgroup
FA_DEV void wg_reduce3(int& lo, int& hi, int& glob) {
  __shared__ int red[12];
  const int wave = threadIdx.x >> 6;
  __syncthreads();   // a previous use of the buffer is over
  if ((threadIdx.x & 63) == 0) { red[wave * 3] = lo; red[wave * 3 + 1] = hi; red[wave * 3 + 2] = glob; }
  __syncthreads();
  lo = min(min(red[0], red[3]), min(red[6], red[9]));
  hi = max(max(red[1], red[4]), max(red[7], red[10]));
  glob = red[2] | red[5] | red[8] | red[11];
}

template <int D>
constexpr size_t lds_bytes() { return size_t(2 * kRows * (D + 1) + 4 * kRows + 64) * 4; }

// Query side of the forward and dq kernels: which row a lane owns, its id, its causal limits, what
// its wave and its workgroup can see.  Without ids: natural order.  With ids: tile `tile` of the
// permuted order of the mask plan; the diagonal of a row sits at the position the plan stored.
template <bool CAUSAL, bool DOC>
struct QSideF32 {
  int row, rowc;        // the lane's row (-1: none), clamped for loads
  bool live;
  int eq_i;
  bool glob_i;
  int lim_i, low_i;     // last / first key the row may see
  int w_lim, w_low;     // largest last key / smallest first key among the wave's rows
  bool w_any;           // the wave holds a row
  int w_lo, w_hi, w_glob;
  int g_lo, g_hi, g_glob;
  int kt0, nkt;         // key tiles (of kRows) the workgroup walks: [kt0, nkt)
  // returns false when the tile holds no row at all (uniform over the workgroup)
  FA_DEV bool init(const KArgs& a, int b, int h, int tile, int wave, int lq) {
    int posc, g_pmin, g_pmax, kfirst = 0, klast = 0x3fffffff;
    if (!DOC) {
      const int m0 = tile * 128, mw = m0 + wave * 32;
      row = mw + lq < a.M ? mw + lq : -1;
      posc = a.gap + min(mw + lq, a.M - 1);
      eq_i = 0;
      g_pmin = a.gap + m0; g_pmax = a.gap + min(m0 + 127, a.M - 1);
    } else {
      const IdSummary* qs = a.qsum + b * a.qs_bs + h * a.qs_hs + 2 * tile;
      const IdSummary s0 = qs[0], s1 = qs[1];
      const int64_t pi = b * a.pm_bs + h * a.pm_hs + tile * 128 + wave * 32 + lq;
      row = a.perm[pi];
      eq_i = a.peq[pi];
      posc = a.ppos[pi];
      if (s0.nvalid + s1.nvalid == 0) return false;
      g_pmin = min(s0.rmin, s1.rmin); g_pmax = max(s0.rmax, s1.rmax);
      kfirst = min(s0.kfirst, s1.kfirst); klast = max(s0.klast, s1.klast);
    }
    live = row >= 0;
    rowc = live ? row : 0;
    if (!live) posc = -1;
    glob_i = eq_i >= 0;
    lim_i = CAUSAL ? min(max(posc, a.pfx_m1), a.N - 1) : a.N - 1;
    low_i = CAUSAL ? posc - a.win + 1 : -0x3fffffff;
    w_any = __builtin_amdgcn_ballot_w64(live) != 0;
    w_lim = half_max(live ? lim_i : -1);
    w_low = half_min(live ? low_i : 0x7fffffff);
    w_lo = 0x7fffffff; w_hi = (int)0x80000000; w_glob = 0;
    if (DOC) {
      w_lo = half_min(live && !glob_i ? eq_i : 0x7fffffff);
      w_hi = half_max(live && !glob_i ? eq_i : (int)0x80000000);
      w_glob = __builtin_amdgcn_ballot_w64(live && glob_i) != 0;
    }
    g_lo = w_lo; g_hi = w_hi; g_glob = w_glob;
    if (DOC) wg_reduce3(g_lo, g_hi, g_glob);
    const int n_end = CAUSAL ? min(a.N, max(g_pmax, a.pfx_m1) + 1) : a.N;
    kt0 = CAUSAL ? max(0, g_pmin - a.win + 1) / kRows : 0;   // sliding window: first tile any row sees
    nkt = (n_end + kRows - 1) / kRows;                       // the same for all waves: the tile stream has barriers
    if (DOC) {                                               // the plan's key range of these rows (tiles of kSumRows keys)
      if (klast < kfirst) nkt = 0;
      else {
        kt0 = max(kt0, kfirst * (kSumRows / kRows));
        nkt = min(nkt, (klast + 1) * (kSumRows / kRows));
      }
    }
    return true;
  }
  FA_DEV bool skips(int n0) const { return !w_any || n0 > w_lim || n0 + kRows - 1 < w_low; }
};

// ---------------------------------------------------------------------------------------------
template <int D, bool CAUSAL, bool DOC>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
void fwd_f32_kernel(const KArgs a) {
  constexpr int RS = D + 1, KS2 = D / 2, DBN = (D + 31) / 32;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* lk = reinterpret_cast<float*>(smem);
  float* lv = lk + kRows * RS;
  int* lid = reinterpret_cast<int*>(lv + kRows * RS);

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lq = lane & 31, g = lane >> 5;
  const int BH = a.B * a.H;
  const int nQt = DOC ? a.Pp / 128 : (a.M + 127) / 128;
  const int tile = nQt - 1 - blockIdx.x / BH;   // the last rows see the most keys (with ids: the global rows): first
  const int bh = blockIdx.x % BH, b = bh / a.H, h = bh % a.H, hk = h / a.G;
  QSideF32<CAUSAL, DOC> qc;
  if (!qc.init(a, b, h, tile, wave, lq)) return;
  const int row = qc.row, rowc = qc.rowc;

  const float* qp = reinterpret_cast<const float*>(a.q) + b * a.q_bs + h * a.q_hs + int64_t(rowc) * a.q_rs;
  const float* kp = reinterpret_cast<const float*>(a.k) + b * a.k_bs + hk * a.k_hs;
  const float* vp = reinterpret_cast<const float*>(a.v) + b * a.v_bs + hk * a.v_hs;
  const int* ekp = DOC ? a.ek32 + b * a.ek_bs + h * a.ek_hs : nullptr;

  float c = a.scale_log2e;
  float qreg[KS2];   // B operand of S^T = K Q^T: Q[row][2*s + g]
#pragma unroll
  for (int s = 0; s < KS2; ++s) qreg[s] = qp[2 * s + g];
  if (c < 0.f) {     // keep max(raw score) == max(scaled score): move the sign into Q
    c = -c;
#pragma unroll
    for (int s = 0; s < KS2; ++s) qreg[s] = -qreg[s];
  }
  const int eq_i = qc.eq_i;
  const bool glob_i = qc.glob_i;
  const int lim_i = qc.lim_i, low_i = qc.low_i;
  const int w_lo = qc.w_lo, w_hi = qc.w_hi, w_glob = qc.w_glob;
  const int kt0 = qc.kt0, nkt = qc.nkt;

  f32x16 o[DBN];
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;   // running reference point (scaled) and this lane's partial row sum

  TileRegs<D> rk, rv;
  int rid = 0;
  // With ids, key tiles that no row of the workgroup can see (by the 64-key summaries of the mask
  // plan) are not even loaded: a packed batch costs its block diagonal, not the whole triangle.
  const int g_lo = qc.g_lo, g_hi = qc.g_hi, g_glob = qc.g_glob;
  const IdSummary* ksum = DOC ? a.ksum + b * a.ks_bs + h * a.ks_hs : nullptr;
  // block mask: the byte rows of the workgroup's two 64-row halves (the second one may lie past the last row)
  const unsigned char* bm0 = nullptr;
  const unsigned char* bm1 = nullptr;
  if (!DOC && a.bmask != nullptr) {
    const unsigned char* base = a.bmask + b * a.bm_bs + h * a.bm_hs;
    bm0 = base + int64_t(2 * tile) * a.bm_rs;
    if (2 * tile + 1 < a.nBr) bm1 = base + int64_t(2 * tile + 1) * a.bm_rs;
  }
  auto next_kt = [&](int kt) {
    if (DOC)
      while (kt < nkt) {
        const IdSummary ks = ksum[(kt * kRows) / kSumRows];
        if (doc_may_keep(g_lo, g_hi, g_glob, ks.lo, ks.hi)) break;
        ++kt;
      }
    if (!DOC && bm0 != nullptr)
      while (kt < nkt) {   // tiles whose block is off for both halves are not even loaded
        const int col = (kt * kRows) / FA_MASK_BLOCK;
        if ((bm0[col] | (bm1 != nullptr ? bm1[col] : 0)) != 0) break;
        ++kt;
      }
    return kt;
  };
  int kt = next_kt(kt0);
  if (kt < nkt) {
    rk.load(kp, a.k_rs, kt * kRows, a.N);
    rv.load(vp, a.v_rs, kt * kRows, a.N);
    if (DOC && threadIdx.x < kRows) rid = ekp[min(kt * kRows + (int)threadIdx.x, a.N - 1)];
  }

  while (kt < nkt) {
    const int n0 = kt * kRows;
    const int kt_next = next_kt(kt + 1);
    __syncthreads();   // the previous tile is no longer read
    rk.store(lk);
    rv.store(lv);
    if (DOC && threadIdx.x < kRows) lid[threadIdx.x] = rid;
    __syncthreads();
    if (kt_next < nkt) {   // the next tile travels while this one is used
      rk.load(kp, a.k_rs, kt_next * kRows, a.N);
      rv.load(vp, a.v_rs, kt_next * kRows, a.N);
      if (DOC && threadIdx.x < kRows) rid = ekp[min(kt_next * kRows + (int)threadIdx.x, a.N - 1)];
    }
    kt = kt_next;
    bool skip = qc.skips(n0);
    if (!DOC && bm0 != nullptr && !skip) {   // the wave's 32 rows and the tile's 32 keys lie inside one block
      const unsigned char* r = wave >= 2 ? bm1 : bm0;
      skip = r == nullptr || r[n0 / FA_MASK_BLOCK] == 0;
    }
    if (DOC && !skip) {
      const bool kv = n0 + lq < a.N;
      const int id = lid[lq];
      const int k_lo = half_min(kv ? id : 0x7fffffff), k_hi = half_max(kv ? id : (int)0x80000000);
      skip = !doc_may_keep(w_lo, w_hi, w_glob, k_lo, k_hi);
    }
    if (skip) continue;

    f32x16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
    pipelined<KS2, kChunk>([&](int i) __attribute__((always_inline)) { return lk[lq * RS + 2 * i + g]; },
                           [&](int i, float x) __attribute__((always_inline)) { s = mfma_f32(x, qreg[i], s); });
    mask_lim(s, lim_i - n0 - 4 * g, low_i - n0 - 4 * g, -INFINITY);
    if (DOC) mask_doc(s, reinterpret_cast<const char*>(lid) + g * 16, eq_i, glob_i, -INFINITY);

    float mx = s[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[r]);
    mx = xhalf_max(mx) * c;                 // -inf stays -inf (c > 0)
    const float m_new = fmaxf(m_run, mx);
    const float alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(m_run - m_new);
    const float msub = (m_new == -INFINITY) ? 0.f : m_new;   // nothing kept so far: exp2(-inf - 0) = 0
    m_run = m_new;
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s[r] = fast_exp2(__builtin_fmaf(s[r], c, -msub));
      ps += s[r];
    }
    l_run = l_run * alpha + ps;
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
    // O^T += V^T P^T: the lane's half supplies key 8*q4 + 4*g + t on both operand sides
    pipelined<16 * DBN, kChunk>(
        [&](int i) __attribute__((always_inline)) {
          const int r = i % 16, key = 8 * (r >> 2) + 4 * g + (r & 3);
          return lv[key * RS + 32 * (i / 16) + lq];
        },
        [&](int i, float x) __attribute__((always_inline)) { o[i / 16] = mfma_f32(x, s[i % 16], o[i / 16]); });
  }

  const float l_tot = xhalf_sum(l_run);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (row >= 0) {
    float* op = reinterpret_cast<float*>(a.o) + b * a.o_bs + h * a.o_hs + int64_t(row) * a.o_rs;
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d0 = 32 * db + 8 * q4 + 4 * g;
        if (d0 >= D) continue;
        const f32x4 x = {o[db][4 * q4] * inv, o[db][4 * q4 + 1] * inv, o[db][4 * q4 + 2] * inv, o[db][4 * q4 + 3] * inv};
        *reinterpret_cast<f32x4*>(op + d0) = x;
      }
    if (g == 0) a.lse[(int64_t(b) * a.H + h) * a.M + row] = l_tot > 0.f ? m_run + fast_log2(l_tot) : -INFINITY;
  }
}

// ---------------------------------------------------------------------------------------------
template <int D, bool CAUSAL, bool DOC>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
void dq_f32_kernel(const KArgs a) {
  constexpr int RS = D + 1, KS2 = D / 2, DBN = (D + 31) / 32;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* lk = reinterpret_cast<float*>(smem);
  float* lv = lk + kRows * RS;
  int* lid = reinterpret_cast<int*>(lv + kRows * RS);

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lq = lane & 31, g = lane >> 5;
  const int BH = a.B * a.H;
  const int nQt = DOC ? a.Pp / 128 : (a.M + 127) / 128;
  const int tile = nQt - 1 - blockIdx.x / BH;
  const int bh = blockIdx.x % BH, b = bh / a.H, h = bh % a.H, hk = h / a.G;
  QSideF32<CAUSAL, DOC> qc;
  if (!qc.init(a, b, h, tile, wave, lq)) return;
  const int row = qc.row, rowc = qc.rowc;

  const float* qp = reinterpret_cast<const float*>(a.q) + b * a.q_bs + h * a.q_hs + int64_t(rowc) * a.q_rs;
  const float* dop = reinterpret_cast<const float*>(a.dout) + b * a.do_bs + h * a.do_hs + int64_t(rowc) * a.do_rs;
  const float* kp = reinterpret_cast<const float*>(a.k) + b * a.k_bs + hk * a.k_hs;
  const float* vp = reinterpret_cast<const float*>(a.v) + b * a.v_bs + hk * a.v_hs;
  const int* ekp = DOC ? a.ek32 + b * a.ek_bs + h * a.ek_hs : nullptr;

  const float c = a.scale_log2e;
  float qreg[KS2], doreg[KS2];
#pragma unroll
  for (int s = 0; s < KS2; ++s) { qreg[s] = qp[2 * s + g]; doreg[s] = dop[2 * s + g]; }
  float L_i = a.lse[(int64_t(b) * a.H + h) * a.M + rowc];
  if (L_i == -INFINITY) L_i = INFINITY;   // row without any kept key: P = exp2(-inf) = 0
  float delta_i;
  if (a.dq_delta) {   // delta = rowsum(O * dO) formed here (the lane and its partner hold the two halves of the row) and left for dk/dv
    const float* op = reinterpret_cast<const float*>(a.o) + b * a.o_bs + h * a.o_hs + int64_t(rowc) * a.o_rs;
    float part = 0.f;
#pragma unroll
    for (int s = 0; s < KS2; ++s) part += op[2 * s + g] * doreg[s];
    delta_i = xhalf_sum(part);
    if (row >= 0 && g == 0) a.delta[(int64_t(b) * a.H + h) * a.M + row] = delta_i;
  } else {
    delta_i = a.delta[(int64_t(b) * a.H + h) * a.M + rowc];
  }
  const int eq_i = qc.eq_i;
  const bool glob_i = qc.glob_i;
  const int lim_i = qc.lim_i, low_i = qc.low_i;
  const int w_lo = qc.w_lo, w_hi = qc.w_hi, w_glob = qc.w_glob;
  const int kt0 = qc.kt0, nkt = qc.nkt;

  f32x16 acc[DBN];
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  TileRegs<D> rk, rv;
  int rid = 0;
  // With ids, key tiles that no row of the workgroup can see (by the 64-key summaries of the mask
  // plan) are not even loaded: a packed batch costs its block diagonal, not the whole triangle.
  const int g_lo = qc.g_lo, g_hi = qc.g_hi, g_glob = qc.g_glob;
  const IdSummary* ksum = DOC ? a.ksum + b * a.ks_bs + h * a.ks_hs : nullptr;
  // block mask: the byte rows of the workgroup's two 64-row halves (the second one may lie past the last row)
  const unsigned char* bm0 = nullptr;
  const unsigned char* bm1 = nullptr;
  if (!DOC && a.bmask != nullptr) {
    const unsigned char* base = a.bmask + b * a.bm_bs + h * a.bm_hs;
    bm0 = base + int64_t(2 * tile) * a.bm_rs;
    if (2 * tile + 1 < a.nBr) bm1 = base + int64_t(2 * tile + 1) * a.bm_rs;
  }
  auto next_kt = [&](int kt) {
    if (DOC)
      while (kt < nkt) {
        const IdSummary ks = ksum[(kt * kRows) / kSumRows];
        if (doc_may_keep(g_lo, g_hi, g_glob, ks.lo, ks.hi)) break;
        ++kt;
      }
    if (!DOC && bm0 != nullptr)
      while (kt < nkt) {   // tiles whose block is off for both halves are not even loaded
        const int col = (kt * kRows) / FA_MASK_BLOCK;
        if ((bm0[col] | (bm1 != nullptr ? bm1[col] : 0)) != 0) break;
        ++kt;
      }
    return kt;
  };
  int kt = next_kt(kt0);
  if (kt < nkt) {
    rk.load(kp, a.k_rs, kt * kRows, a.N);
    rv.load(vp, a.v_rs, kt * kRows, a.N);
    if (DOC && threadIdx.x < kRows) rid = ekp[min(kt * kRows + (int)threadIdx.x, a.N - 1)];
  }

  while (kt < nkt) {
    const int n0 = kt * kRows;
    const int kt_next = next_kt(kt + 1);
    __syncthreads();
    rk.store(lk);
    rv.store(lv);
    if (DOC && threadIdx.x < kRows) lid[threadIdx.x] = rid;
    __syncthreads();
    if (kt_next < nkt) {
      rk.load(kp, a.k_rs, kt_next * kRows, a.N);
      rv.load(vp, a.v_rs, kt_next * kRows, a.N);
      if (DOC && threadIdx.x < kRows) rid = ekp[min(kt_next * kRows + (int)threadIdx.x, a.N - 1)];
    }
    kt = kt_next;
    bool skip = qc.skips(n0);
    if (!DOC && bm0 != nullptr && !skip) {   // the wave's 32 rows and the tile's 32 keys lie inside one block
      const unsigned char* r = wave >= 2 ? bm1 : bm0;
      skip = r == nullptr || r[n0 / FA_MASK_BLOCK] == 0;
    }
    if (DOC && !skip) {
      const bool kv = n0 + lq < a.N;
      const int id = lid[lq];
      const int k_lo = half_min(kv ? id : 0x7fffffff), k_hi = half_max(kv ? id : (int)0x80000000);
      skip = !doc_may_keep(w_lo, w_hi, w_glob, k_lo, k_hi);
    }
    if (skip) continue;

    f32x16 s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
    pipelined<2 * KS2, kChunk>(
        [&](int i) __attribute__((always_inline)) { return ((i & 1) ? lv : lk)[lq * RS + 2 * (i / 2) + g]; },
        [&](int i, float x) __attribute__((always_inline)) {
          if (i & 1) dp = mfma_f32(x, doreg[i / 2], dp);
          else s = mfma_f32(x, qreg[i / 2], s);
        });
    // dS = P (dP - delta); masked pairs -> 0 (a select, so an overflowed exponential of a masked pair is harmless)
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = fast_exp2(__builtin_fmaf(s[r], c, -L_i)) * (dp[r] - delta_i);
    mask_lim(s, lim_i - n0 - 4 * g, low_i - n0 - 4 * g, 0.f);
    if (DOC) mask_doc(s, reinterpret_cast<const char*>(lid) + g * 16, eq_i, glob_i, 0.f);
    // dQ^T += K^T dS^T
    pipelined<16 * DBN, kChunk>(
        [&](int i) __attribute__((always_inline)) {
          const int r = i % 16, key = 8 * (r >> 2) + 4 * g + (r & 3);
          return lk[key * RS + 32 * (i / 16) + lq];
        },
        [&](int i, float x) __attribute__((always_inline)) { acc[i / 16] = mfma_f32(x, s[i % 16], acc[i / 16]); });
  }

  if (row >= 0) {
    float* dqp = reinterpret_cast<float*>(a.dq) + b * a.dq_bs + h * a.dq_hs + int64_t(row) * a.dq_rs;
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d0 = 32 * db + 8 * q4 + 4 * g;
        if (d0 >= D) continue;
        const f32x4 x = {acc[db][4 * q4] * a.scale, acc[db][4 * q4 + 1] * a.scale, acc[db][4 * q4 + 2] * a.scale,
                         acc[db][4 * q4 + 3] * a.scale};
        *reinterpret_cast<f32x4*>(dqp + d0) = x;
      }
  }
}

// ---------------------------------------------------------------------------------------------
template <int D, bool CAUSAL, bool DOC>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
void dkdv_f32_kernel(const KArgs a) {
  constexpr int RS = D + 1, KS2 = D / 2, DBN = (D + 31) / 32;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* lqt = reinterpret_cast<float*>(smem);
  float* ldo = lqt + kRows * RS;
  float* laux = ldo + kRows * RS;               // [LSE | delta | eq | row name] x 32
  const int* leq = reinterpret_cast<const int*>(laux + 2 * kRows);
  const int* lnm = reinterpret_cast<const int*>(laux + 3 * kRows);

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lq = lane & 31, g = lane >> 5;
  const int BHk = a.B * a.Hk;
  const int kt = blockIdx.x / BHk;               // causal: the first keys are seen by the most rows: first
  const int bhk = blockIdx.x % BHk, b = bhk / a.Hk, hk = bhk % a.Hk;
  const int n0 = kt * 128, nw = n0 + wave * 32;
  const int key = nw + lq, keyc = min(key, a.N - 1);

  const float* kp = reinterpret_cast<const float*>(a.k) + b * a.k_bs + hk * a.k_hs + int64_t(keyc) * a.k_rs;
  const float* vp = reinterpret_cast<const float*>(a.v) + b * a.v_bs + hk * a.v_hs + int64_t(keyc) * a.v_rs;
  float kreg[KS2], vreg[KS2];   // B operands of S = Q K^T and dP = dO V^T: K[key][2*s + g], V[key][2*s + g]
#pragma unroll
  for (int s = 0; s < KS2; ++s) { kreg[s] = kp[2 * s + g]; vreg[s] = vp[2 * s + g]; }
  const float c = a.scale_log2e;
  // A row is named by its index (its diagonal sits at key gap + index) or, with ids, by the diagonal
  // position the mask plan stored for it (offset 0, names up to kPosMax; -1: no row).
  // Rows that may see this lane's key: names [row_lo, row_lo + row_span)
  // (causal: from the diagonal on, or from 0 for a key of the prefix; sliding window: `win` names)
  const int gk = DOC ? 0 : a.gap;
  const int rcap = DOC ? kPosMax : a.M - 1;
  const int row_lo = CAUSAL ? (key <= a.pfx_m1 ? 0 : max(0, key - gk)) : 0;
  const int row_hi = CAUSAL ? min(rcap, key - gk + a.win - 1) : rcap;
  const unsigned row_span = (key < a.N && row_hi >= row_lo) ? (unsigned)(row_hi - row_lo + 1) : 0u;
  const int wg_rhi = CAUSAL ? min(rcap, n0 + 127 - gk + a.win - 1) : rcap;   // last name that sees a key of the workgroup
  // query tiles of 32 rows: natural order from the diagonal on, or every tile of the permuted order
  const int mt0 = DOC ? 0 : (CAUSAL ? (n0 <= a.pfx_m1 ? 0 : max(0, n0 - gk) / kRows) : 0);
  const int nMt = DOC ? a.Pp / kRows : max(0, wg_rhi + kRows) / kRows;

  f32x16 dv[DBN], dk[DBN];
#pragma unroll
  for (int db = 0; db < DBN; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dv[db][r] = 0.f; dk[db][r] = 0.f; }

  for (int gi = 0; gi < a.G; ++gi) {
    const int h = hk * a.G + gi;
    const float* qp = reinterpret_cast<const float*>(a.q) + b * a.q_bs + h * a.q_hs;
    const float* dop = reinterpret_cast<const float*>(a.dout) + b * a.do_bs + h * a.do_hs;
    const float* lsep = a.lse + (int64_t(b) * a.H + h) * a.M;
    const float* delp = a.delta + (int64_t(b) * a.H + h) * a.M;
    const int* pmp = DOC ? a.perm + b * a.pm_bs + h * a.pm_hs : nullptr;
    const int* pqp = DOC ? a.peq + b * a.pm_bs + h * a.pm_hs : nullptr;
    const int* ppp = DOC ? a.ppos + b * a.pm_bs + h * a.pm_hs : nullptr;
    int ek_j = 0, wk_lo = 0, wk_hi = 0;
    if (DOC) {
      ek_j = a.ek32[b * a.ek_bs + h * a.ek_hs + keyc];
      wk_lo = half_min(key < a.N ? ek_j : 0x7fffffff);
      wk_hi = half_max(key < a.N ? ek_j : (int)0x80000000);
    }
    // one auxiliary value per thread of the first four groups of 32: LSE, delta, id, name of a tile row
    auto aux_load = [&](int mt) -> float {
      const int t = threadIdx.x & 31, which = threadIdx.x >> 5;
      if (!DOC) {
        const int r = mt * kRows + t, rc = min(r, a.M - 1);
        if (which == 0) return lsep[rc];
        if (which == 1) return delp[rc];
        return 0.f;
      }
      if (which == 2) return __int_as_float(pqp[mt * kRows + t]);
      if (which == 3) return __int_as_float(ppp[mt * kRows + t]);
      const int r = max(pmp[mt * kRows + t], 0);
      return which == 0 ? lsep[r] : delp[r];
    };
    // With ids: query tiles whose 64-entry summary of the plan excludes every key of the workgroup
    // (no row, ids that cannot meet, diagonals before the first key or beyond the window) are not loaded.
    int gk_lo = wk_lo, gk_hi = wk_hi, gk_unused = 0;
    const IdSummary* qsum = nullptr;
    if (DOC) {
      wg_reduce3(gk_lo, gk_hi, gk_unused);
      qsum = a.qsum + b * a.qs_bs + h * a.qs_hs;
    }
    // block mask: the one or two byte columns of the workgroup's 128 keys
    const unsigned char* bmc = (!DOC && a.bmask != nullptr) ? a.bmask + b * a.bm_bs + h * a.bm_hs + n0 / FA_MASK_BLOCK : nullptr;
    const bool bm_two = n0 / FA_MASK_BLOCK + 1 < a.nBc;
    auto next_mt = [&](int mt) {
      if (DOC)
        while (mt < nMt) {
          const IdSummary qs = qsum[(mt * kRows) / kSumRows];
          const bool out = qs.nvalid == 0 || !doc_may_keep(qs.lo, qs.hi, qs.glob, gk_lo, gk_hi) ||
                           (CAUSAL && ((qs.rmax < n0 && n0 > a.pfx_m1) || qs.rmin > wg_rhi));
          if (!out) break;
          ++mt;
        }
      if (bmc != nullptr)
        while (mt < nMt) {   // tiles whose block is off for both key columns are not even loaded
          const unsigned char* r = bmc + int64_t((mt * kRows) / FA_MASK_BLOCK) * a.bm_rs;
          if ((r[0] | (bm_two ? r[1] : 0)) != 0) break;
          ++mt;
        }
      return mt;
    };
    TileRegs<D> rq, rdo;
    float raux = 0.f;
    auto load_tile = [&](int mt) {
      if (DOC) {
        rq.load_rows(qp, a.q_rs, pmp + mt * kRows);
        rdo.load_rows(dop, a.do_rs, pmp + mt * kRows);
      } else {
        rq.load(qp, a.q_rs, mt * kRows, a.M);
        rdo.load(dop, a.do_rs, mt * kRows, a.M);
      }
      if (threadIdx.x < 4 * kRows) raux = aux_load(mt);
    };
    int mt = next_mt(mt0);
    if (mt < nMt) load_tile(mt);
    while (mt < nMt) {
      const int mt_next = next_mt(mt + 1);
      __syncthreads();
      rq.store(lqt);
      rdo.store(ldo);
      if (threadIdx.x < 4 * kRows) laux[threadIdx.x] = raux;
      __syncthreads();
      if (mt_next < nMt) load_tile(mt_next);
      const int m0 = mt * kRows;   // natural order only
      mt = mt_next;
      // names of the tile's rows (-1: none): smallest / largest among the 32
      const int nm = DOC ? lnm[lq] : (m0 + lq < a.M ? m0 + lq : -1);
      const int t_min = DOC ? half_min(nm >= 0 ? nm : 0x7fffffff) : m0;
      const int t_max = DOC ? half_max(nm) : min(m0 + kRows - 1, a.M - 1);
      bool skip = nw >= a.N || t_max < 0 ||
                  (CAUSAL && ((gk + t_max < nw && nw > a.pfx_m1) || gk + t_min - a.win + 1 > nw + 31));
      if (bmc != nullptr && !skip)   // the wave's 32 keys and the tile's 32 rows lie inside one block
        skip = bmc[int64_t((t_min / FA_MASK_BLOCK)) * a.bm_rs + (wave >= 2 ? 1 : 0)] == 0;
      if (DOC && !skip) {
        const bool rv_ = nm >= 0;
        const int id = leq[lq];
        const bool loc = rv_ && id < 0;
        const int q_lo = half_min(loc ? id : 0x7fffffff), q_hi = half_max(loc ? id : (int)0x80000000);
        const int q_glob = __builtin_amdgcn_ballot_w64(rv_ && id >= 0) != 0;
        skip = !doc_may_keep(q_lo, q_hi, q_glob, wk_lo, wk_hi);
      }
      if (skip) continue;

      f32x16 x, dp;
#pragma unroll
      for (int r = 0; r < 16; ++r) { x[r] = 0.f; dp[r] = 0.f; }
      pipelined<2 * KS2, kChunk>(
          [&](int i) __attribute__((always_inline)) { return ((i & 1) ? ldo : lqt)[lq * RS + 2 * (i / 2) + g]; },
          [&](int i, float v_) __attribute__((always_inline)) {
            if (i & 1) dp = mfma_f32(v_, vreg[i / 2], dp);
            else x = mfma_f32(v_, kreg[i / 2], x);
          });
      // lane = key, register 4*q4 + t = row 8*q4 + 4*g + t of the tile
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int i0 = 8 * q4 + 4 * g;
        const f32x4 Lv = *reinterpret_cast<const f32x4*>(laux + i0);
        const f32x4 dl = *reinterpret_cast<const f32x4*>(laux + kRows + i0);
        const i32x4 eqv = *reinterpret_cast<const i32x4*>(leq + i0);
        i32x4 nmv = {m0 + i0, m0 + i0 + 1, m0 + i0 + 2, m0 + i0 + 3};   // rows past the end lie beyond every span
        if (DOC) nmv = *reinterpret_cast<const i32x4*>(lnm + i0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          bool keep = (unsigned)(nmv[t] - row_lo) < row_span;
          if (DOC) keep = keep && (eqv[t] >= 0 || eqv[t] == ek_j);
          const float p = fast_exp2(__builtin_fmaf(x[4 * q4 + t], c, -Lv[t]));
          x[4 * q4 + t] = keep ? p : 0.f;
          dp[4 * q4 + t] = keep ? p * (dp[4 * q4 + t] - dl[t]) : 0.f;
        }
      }
      // dV^T += dO^T P, dK^T += Q^T dS
      pipelined<32 * DBN, kChunk>(
          [&](int i) __attribute__((always_inline)) {
            const int r = (i / 2) % 16, qr = 8 * (r >> 2) + 4 * g + (r & 3);
            return ((i & 1) ? lqt : ldo)[qr * RS + 32 * (i / 32) + lq];
          },
          [&](int i, float v_) __attribute__((always_inline)) {
            const int r = (i / 2) % 16, db = i / 32;
            if (i & 1) dk[db] = mfma_f32(v_, dp[r], dk[db]);
            else dv[db] = mfma_f32(v_, x[r], dv[db]);
          });
    }
  }

  if (key < a.N) {
    float* dvp = reinterpret_cast<float*>(a.dv) + b * a.dv_bs + hk * a.dv_hs + int64_t(key) * a.dv_rs;
    float* dkp = reinterpret_cast<float*>(a.dk) + b * a.dk_bs + hk * a.dk_hs + int64_t(key) * a.dk_rs;
#pragma unroll
    for (int db = 0; db < DBN; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d0 = 32 * db + 8 * q4 + 4 * g;
        if (d0 >= D) continue;
        const f32x4 xv = {dv[db][4 * q4], dv[db][4 * q4 + 1], dv[db][4 * q4 + 2], dv[db][4 * q4 + 3]};
        const f32x4 xk = {dk[db][4 * q4] * a.scale, dk[db][4 * q4 + 1] * a.scale, dk[db][4 * q4 + 2] * a.scale,
                          dk[db][4 * q4 + 3] * a.scale};
        *reinterpret_cast<f32x4*>(dvp + d0) = xv;
        *reinterpret_cast<f32x4*>(dkp + d0) = xk;
      }
  }
}

// delta[b,h,m] = sum_d O[b,h,m,d] * dO[b,h,m,d]; D/4 lanes per row, 16-byte loads.
template <int D>
__global__ __launch_bounds__(kThreads) void delta_f32_kernel(const KArgs a) {
  constexpr int LPR = D / 4, RPB = kThreads / LPR;
  const int row = blockIdx.x * RPB + threadIdx.x / LPR;
  const int cc = threadIdx.x % LPR;
  // (batch, head) pairs are walked with the grid's stride: grid dimension y stops at 65535
  for (int bh = blockIdx.y; bh < a.B * a.H; bh += gridDim.y) {
    const int b = bh / a.H, h = bh % a.H;
    float acc = 0.f;
    if (row < a.M) {
      const f32x4 x = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(a.o) + b * a.o_bs + h * a.o_hs +
                                                      int64_t(row) * a.o_rs + cc * 4);
      const f32x4 y = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(a.dout) + b * a.do_bs + h * a.do_hs +
                                                      int64_t(row) * a.do_rs + cc * 4);
      acc = x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
    }
#pragma unroll
    for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off);
    if (cc == 0 && row < a.M) a.delta[(int64_t(b) * a.H + h) * a.M + row] = acc;
  }
}

enum { kFwd, kDq, kDkdv };

template <int WHICH, int D, bool CAUSAL, bool DOC>
int launch_one(const KArgs& a, hipStream_t s) {
  auto kern = WHICH == kFwd ? fwd_f32_kernel<D, CAUSAL, DOC> : WHICH == kDq ? dq_f32_kernel<D, CAUSAL, DOC>
                                                                            : dkdv_f32_kernel<D, CAUSAL, DOC>;
  // query tiles: of the natural order, or of the mask plan's permuted order with ids
  const int blocks = WHICH == kDkdv ? ((a.N + 127) / 128) * a.B * a.Hk : (DOC ? a.Pp / 128 : (a.M + 127) / 128) * a.B * a.H;
  static bool lds_allowed[64] = {};   // per kernel instantiation and device
  if (int e = allow_lds(kern, lds_bytes<D>(), lds_allowed)) return e;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(kThreads), lds_bytes<D>(), s, a);
  return (int)hipGetLastError();
}

template <int WHICH, int D>
int launch_cd(const KArgs& a, bool causal, bool doc, hipStream_t s) {
  if (causal) return doc ? launch_one<WHICH, D, true, true>(a, s) : launch_one<WHICH, D, true, false>(a, s);
  return doc ? launch_one<WHICH, D, false, true>(a, s) : launch_one<WHICH, D, false, false>(a, s);
}

template <int WHICH>
int launch_d(const KArgs& a, int D, bool causal, bool doc, hipStream_t s) {
  switch (D) {
    case 128: return launch_cd<WHICH, 128>(a, causal, doc, s);
    case 64: return launch_cd<WHICH, 64>(a, causal, doc, s);
    case 32: return launch_cd<WHICH, 32>(a, causal, doc, s);
    case 16: return launch_cd<WHICH, 16>(a, causal, doc, s);
    default: return -1;
  }
}

}  // namespace

int launch_fwd_f32(const KArgs& a, int D, bool causal, bool doc, hipStream_t s) { return launch_d<kFwd>(a, D, causal, doc, s); }
int launch_bwd_dq_f32(const KArgs& a, int D, bool causal, bool doc, hipStream_t s) { return launch_d<kDq>(a, D, causal, doc, s); }
int launch_bwd_dkdv_f32(const KArgs& a, int D, bool causal, bool doc, hipStream_t s) { return launch_d<kDkdv>(a, D, causal, doc, s); }

int launch_bwd_delta_f32(const KArgs& a, int D, hipStream_t s) {
  const int BH = a.B * a.H < 65535 ? a.B * a.H : 65535;
  switch (D) {
    case 128: hipLaunchKernelGGL((delta_f32_kernel<128>), dim3((a.M + 7) / 8, BH), dim3(kThreads), 0, s, a); break;
    case 64: hipLaunchKernelGGL((delta_f32_kernel<64>), dim3((a.M + 15) / 16, BH), dim3(kThreads), 0, s, a); break;
    case 32: hipLaunchKernelGGL((delta_f32_kernel<32>), dim3((a.M + 31) / 32, BH), dim3(kThreads), 0, s, a); break;
    case 16: hipLaunchKernelGGL((delta_f32_kernel<16>), dim3((a.M + 63) / 64, BH), dim3(kThreads), 0, s, a); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}

}  // namespace fa
