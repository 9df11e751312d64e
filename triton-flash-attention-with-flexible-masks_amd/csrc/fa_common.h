// Shared device/host definitions for the gfx950 flash-attention kernels.
//
// Register-level conventions used by every compute kernel in this directory
// (CDNA4 v_mfma_f32_32x32x16_{bf16,f16}, wave64):
//   A operand (32 x 16): lane l holds row  (l & 31), k = 8*(l >> 5) .. +7
//   B operand (16 x 32): lane l holds col  (l & 31), k = 8*(l >> 5) .. +7
//   C/D       (32 x 32): lane l holds col  (l & 31), register r (0..15) is
//                        row 8*(r >> 2) + 4*(l >> 5) + (r & 3)
// ds_read_b64_tr_b16: inside each group of 16 lanes, result lane i, element e is
// taken from source lane 4*e + (i >> 2), element (i & 3) of its 8-byte read.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/flash_mi355.h"

namespace fa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

#define FA_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define FA_GLB(p) ((const __attribute__((address_space(1))) void*)(p))
#define FA_DEV __device__ __forceinline__
#define FA_HD __host__ __device__ inline

constexpr float kLog2e = 1.4426950408889634f;

// Rows covered by one entry of the id summaries written by the mask plan.
constexpr int kSumRows = 64;
// The local-row part of the permuted order is padded to this many entries, so that a
// workgroup of up to 256 query rows never mixes local and global rows.
constexpr int kPermAlign = 256;
// Tiles of global rows (eq >= 0) see every key up to their own position, i.e. up to the whole
// sequence: a single workgroup walking 16K keys is the critical path of the kernel.  The key range
// of the first `tiles` such tiles of a (batch, head) is therefore cut into up to `k` chunks handled
// by different workgroups; each writes an fp32 partial result and the last one to arrive (an atomic
// counter per tile) merges them.  The merge order is fixed, results stay reproducible.
constexpr int kSplitMinTiles = 16;   // key tiles (of 64) per chunk below which splitting does not pay
constexpr int kSplitKMax = 4;        // more chunks did not pay on any shape with enough query tiles to fill the chip
constexpr int kSplitKMaxFew = 16;    // ... but they do when the whole launch is short of workgroups (few query rows)
constexpr int kSplitFewWgs = 1024;   // query tiles in the launch (all heads) below which it counts as short of workgroups
struct SplitCfg {
  int k;      // chunks per tile (1: nothing is ever split)
  int tiles;  // global-row tiles per (batch, head) that can be split
};
// Chunks of at least 32 key tiles (2 .. kSplitKMax of them), and as many splittable tiles as the
// scratch budget allows (at most 64): long sequences with few heads have many global-row tiles, each
// of them long.  The budget is a hard bound on the scratch part of the workspace: with many (batch,
// head) pairs it buys fewer tiles per pair, down to none (such launches have workgroups to spare and
// short key ranges per tile; with fewer than two tiles in the budget at 4 chunks, 2 chunks are tried).
// With fewer than kSplitFewWgs query tiles in the whole launch (decoding, the tail of a long prompt, a short
// query block against a long packed key sequence) the chunks go down to kSplitMinTiles key tiles, up to
// kSplitKMaxFew of them.  Never more splittable tiles than M rows can fill.
constexpr uint64_t kSplitScratchBudget = uint64_t(128) << 20;   // bytes of sk_ml + sk_o
inline SplitCfg split_config(int B, int H, int M, int N, int D, uint64_t budget = kSplitScratchBudget) {
  SplitCfg c = {1, 0};
  const int nKs = (N + kSumRows - 1) / kSumRows;
  if (nKs < 2 * kSplitMinTiles) return c;   // no key range can be long enough to be cut
  const int qtiles = (M + 127) / 128 + 1;   // 128-row tiles of global rows a (batch, head) can have
  const uint64_t wgs = uint64_t(B) * H * qtiles;
  if (wgs < kSplitFewWgs) {
    // Short of workgroups: the chunks of the global-row tiles are what fills the chip.  About 256 workgroups
    // that each stream their own K / V chunk keep the memory system busy (more of them only add merge work),
    // and every (batch, head) has at least one such tile.
    const uint64_t bh = uint64_t(B) * H;
    const int fill = int(256 / bh);
    const int kmax = fill < kSplitKMax ? kSplitKMax : (fill > kSplitKMaxFew ? kSplitKMaxFew : fill);
    const int want = nKs / kSplitMinTiles;
    c.k = want < 2 ? 2 : (want > kmax ? kmax : want);
  } else {
    c.k = nKs / 32 < 2 ? 2 : (nKs / 32 > kSplitKMax ? kSplitKMax : nKs / 32);
  }
  auto tiles_for = [&](int k) {
    const uint64_t per_tile = uint64_t(k) * 128 * (D + 2) * 4;
    const uint64_t t = budget / (uint64_t(B) * H * per_tile);
    return t > 64 ? 64 : int(t);
  };
  c.tiles = tiles_for(c.k);
  if (c.tiles < 2 && c.k > 2) { c.k = 2; c.tiles = tiles_for(2); }
  if (c.tiles > qtiles) c.tiles = qtiles;
  if (c.tiles <= 0) { c.tiles = 0; c.k = 1; }
  return c;
}

// Compile-time integer handed to a generic lambda.
template <int V> struct IntC { static constexpr int value = V; };

constexpr int kPairSpinDefault = 1 << 14;

// Clock stamps per workgroup, for the measurement build only (compiled with -DFA_TRACE into a library of its
// own, libflash_mi355_trace.so, read by `bench.py --wg-trace`).  A traced kernel keeps eight 64-bit words per
// workgroup in a device array (wall clock, 100 MHz) that fa_trace_read copies out.  In the product build the
// macros expand to nothing.
#ifdef FA_TRACE
constexpr int kTraceWgs = 65536;
#define FA_TRACE_ARRAY(name) __device__ long long name[8 * fa::kTraceWgs]
#define FA_STAMP(buf, i, v) do { if (threadIdx.x == 0 && blockIdx.x < fa::kTraceWgs) buf[blockIdx.x * 8 + (i)] = (long long)(v); } while (0)
#define FA_CLOCK() wall_clock64()
#define FA_TRACE_ONLY(...) __VA_ARGS__
#else
#define FA_STAMP(buf, i, v) do {} while (0)
#define FA_CLOCK() 0
#define FA_TRACE_ONLY(...)
#endif

// Key position of a row's diagonal as the kernels use it: at least -1 (the row sees nothing), and
// small enough that position + window never overflows.
constexpr int kPosMax = 0x3fffffff;
FA_HD int clamp_pos(int v) { return v < -1 ? -1 : (v > kPosMax ? kPosMax : v); }

struct bf16_t {};
struct fp16_t {};

template <typename Tag> struct Elem;

template <> struct Elem<bf16_t> {
  typedef __bf16 scalar;
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  typedef bf16x2 vec2;
  static FA_DEV f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static FA_DEV vec4 lds_tr(const void* p) {
    return __builtin_bit_cast(vec4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p)));
  }
  static FA_DEV vec2 cvt2(float x, float y) {
    f32x2 t = {x, y};
    return __builtin_convertvector(t, vec2);
  }
};

template <> struct Elem<fp16_t> {
  typedef _Float16 scalar;
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  typedef f16x2 vec2;
  static FA_DEV f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static FA_DEV vec4 lds_tr(const void* p) {
    return __builtin_bit_cast(vec4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p)));
  }
  static FA_DEV vec2 cvt2(float x, float y) {
    f32x2 t = {x, y};
    return __builtin_convertvector(t, vec2);
  }
};

// Sign flip of 8 packed 16-bit floats (exact for both bf16 and fp16).
template <typename E>
FA_DEV typename E::vec8 neg8(typename E::vec8 x) {
  i32x4 u = __builtin_bit_cast(i32x4, x);
  u ^= (int)0x80008000;
  return __builtin_bit_cast(typename E::vec8, u);
}

// Exchange between lane l and lane l ^ 32: returns the partner's value.
FA_DEV float xhalf(float x) {
  unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  // r[0] = {lo, lo}, r[1] = {hi, hi}: the partner of a low lane is r[1], of a high lane r[0]
  unsigned lo = r[0], hi = r[1];
  return __uint_as_float((threadIdx.x & 32) ? lo : hi);
}
FA_DEV float xhalf_max(float x) {
  unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
FA_DEV float xhalf_sum(float x) {
  unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Make a 16-byte value loaded from global memory "used" right here.  The compiler waits for a
// load at the first use of its result; for operands that are loaded once and first used inside
// the tile loop that wait (s_waitcnt vmcnt) would sit in the loop, where it also waits for the
// asynchronous tile loads issued just before it -- the loads it is meant to overlap with.
template <typename V>
FA_DEV void settle(V& x) {
  i32x4 u = __builtin_bit_cast(i32x4, x);
  asm volatile("" : "+v"(u));
  x = __builtin_bit_cast(V, u);
}
FA_DEV void settle(float& x) { asm volatile("" : "+v"(x)); }
FA_DEV void settle(int& x) { asm volatile("" : "+v"(x)); }

FA_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
FA_DEV float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---------------------------------------------------------------------------
// Mask engine, element level.  keep(i, j) of the reference:
//   tail   : j < N (and i < M at the store)             flash_triton.py:103-105
//   causal : gap + i >= j, gap = max(0, N - M)          flash_triton.py:107
//   doc    : eq_i >= 0 || eq_i == ek_j                  flash_triton.py:114
// ---------------------------------------------------------------------------
//   window : j > gap + i - win (win = 0x3fffffff: off)    sliding window, causal only
//   prefix : the causal term also holds for j <= pfx_m1   prefix-LM (pfx_m1 = -1: off)
//   pos_i  : key position of row i's diagonal: gap + i, or the caller's per-row position (fa_params.qpos)
template <bool CAUSAL, bool DOC>
FA_DEV bool keep_elem(int pos_i, int j, int N, int eq_i, int ek_j, int win, int pfx_m1) {
  bool keep = j < N;
  if (CAUSAL) keep = keep && ((pos_i >= j) || (j <= pfx_m1)) && (j > pos_i - win);
  if (DOC) keep = keep && ((eq_i >= 0) || (eq_i == ek_j));
  return keep;
}

// ---------------------------------------------------------------------------
// Mask plan.  With document ids the query rows of one (batch, head) are split
// into LOCAL rows (eq < 0: see only keys with the same id) and GLOBAL rows
// (eq >= 0: see every key), each group kept in ascending row order:
//   perm[0 .. nL)            local rows            (padded with -1 up to nLp,
//   perm[nLp .. nLp + nG)    global rows            nLp = nL rounded up to kPermAlign)
// Query-side tiles are tiles of this permuted order, so a tile is either all
// local (it only needs the key tiles whose id interval meets its own) or all
// global (no doc test at all, plain causal structure).  Keys stay in natural
// order.  One IdSummary describes 64 consecutive entries of either side.
// ---------------------------------------------------------------------------
struct IdSummary {
  int lo, hi;      // min / max id: query side over local rows (lo > hi if none), key side over all keys
  int glob;        // query side: 1 if the tile holds global rows
  int rmin, rmax;  // query side: smallest / largest diagonal position (ppos) of the tile's rows (rmax = -1 if empty);
                   // key side: first / last key of the tile
  int nvalid;      // query side: rows of the tile that exist
  int kfirst, klast;  // query side: first / last key tile (of 64 keys) the rows can need (klast < kfirst: none)
};

struct QHeader {
  int nL, nG, nLp, nT128;  // nT128: 128-row tiles of the permuted order that hold rows
  int k0;                  // first key tile (of 64) that a local row can need (0x7fffffff: none can need any):
                           // the keys before it are seen by global rows only
  int pad[3];
};

// A tile pair can hold a kept element only if a global query row exists or the
// local-id interval of the query rows meets the id interval of the keys.
FA_DEV bool doc_may_keep(int q_lo, int q_hi, int q_glob, int k_lo, int k_hi) {
  return q_glob || (q_lo <= k_hi && k_lo <= q_hi);
}
// Every (row, key) pair of the tile pair passes the doc test.
FA_DEV bool doc_all_keep(int q_lo, int q_hi, int k_lo, int k_hi) {
  // no local row at all, or one local id shared by every key
  return (q_lo > q_hi) || (q_lo == q_hi && k_lo == k_hi && q_lo == k_lo);
}

// Key columns that no local row can need (QHeader::k0) are seen by the global rows only.  When those rows
// are few -- at most kGcolTilesMax tiles of 64, over all query heads of a group -- a kernel of its own takes
// these columns: it keeps the rows' Q / dO tiles in LDS and streams the keys (fa_dkdv_cols.h), instead
// of one workgroup per 64 keys that sets up a tile stream for one or two tiles.
constexpr int kGcolTilesMax = 2;
constexpr int kGcolMinGap = 512;   // keys without a diagonal of their own from which the form is put into the launch

// Kernel-side view of the operands (built on the host from fa_params).
struct KArgs {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  const void* dout;
  void* dq;
  void* dk;
  void* dv;
  float* delta;
  const int* eq32;        // [B, Hq', Mp]   ids in natural row order
  const int* ek32;        // [B, Hk', Np]
  const int* perm;        // [B, Hq', Pp]   permuted order -> original row (or -1)
  const int* peq;         // [B, Hq', Pp]   id of that row
  const int* ppos;        // [B, Hq', Pp]   key position of that row's diagonal (gap + row, or the caller's qpos), -1 for padding
  const int* qpos;        // the caller's per-row positions [B, M] in natural order, or null (mask dump)
  int64_t qp_bs;
  const QHeader* qhdr;    // [B, Hq']
  const IdSummary* qsum;  // [B, Hq', nQs]  per 64 entries of the permuted order
  const IdSummary* ksum;  // [B, Hk', nKs]  per 64 keys
  // split-key scratch of the global-row tiles, see SplitCfg: per (b, h, global tile g)
  int split_k, split_tiles;
  int* sk_cnt;            // [B, H, split_tiles]                  arrival counters (zero between kernels)
  float* sk_ml;           // [B, H, split_tiles, split_k, 128, 2]  per row: reference point, row sum
  float* sk_o;            // [B, H, split_tiles, split_k, 128, D]  per row: unnormalised partial result
  int64_t q_bs, q_hs, q_rs;
  int64_t k_bs, k_hs, k_rs;
  int64_t v_bs, v_hs, v_rs;
  int64_t o_bs, o_hs, o_rs;
  int64_t do_bs, do_hs, do_rs;
  int64_t dq_bs, dq_hs, dq_rs;
  int64_t dk_bs, dk_hs, dk_rs;
  int64_t dv_bs, dv_hs, dv_rs;
  int64_t eq_bs, eq_hs;   // strides of eq32 (head stride 0 when shared)
  int64_t ek_bs, ek_hs;
  int64_t pm_bs, pm_hs;   // strides of perm
  int64_t qh_bs, qh_hs;   // strides of qhdr in entries
  int64_t qs_bs, qs_hs;   // strides of qsum in entries
  int64_t ks_bs, ks_hs;
  int B, H, Hk, G, M, N, gap;
  int win;      // sliding window: a row sees keys j > gap + i - win (0x3fffffff: no window)
  int pfx_m1;   // prefix-LM: keys j <= pfx_m1 are seen by every row (-1: no prefix)
  int Pp;                 // entries of the permuted order per (b, h)
  int nQs, nKs;           // summary entries per (b, h)
  int dq_delta;           // the dq kernel computes delta from O and dO itself and stores it
  int pair_spin;          // dk/dv, role-split form: polls of the pair flag before the gradient wave gives up
  // block mask (FA_SCORE_MODE2_BLOCK): bytes [B, H, nBr, nBc] per 64 x 64 block of (row, key) pairs, or null
  const unsigned char* bmask;
  int64_t bm_bs, bm_hs, bm_rs;
  int nBr, nBc;
  float scale;            // sm_scale
  float scale_log2e;      // sm_scale * log2(e)
};

// Workspace layout shared by host and device code.
struct WsLayout {
  int Hq1, Hk1;           // heads stored for eq / ek (1 when the head stride is 0)
  int Mp, Np;             // M, N rounded up to kSumRows
  int Pp;                 // length of the permuted order
  int nQs, nKs;
  int nCh;                // row chunks of the partition kernels
  uint64_t off_eq32, off_ek32, off_perm, off_peq, off_ppos, off_cnt, off_qhdr, off_qsum, off_ksum;  // bytes
  uint64_t off_sk_cnt, off_sk_ml, off_sk_o, total;
  uint64_t plan_bytes;   // leading part that carries state from the plan to the kernels; the rest is scratch
  SplitCfg split;        // split of long key ranges this layout has scratch for
};

// split_budget: bytes the scratch of the split key ranges (sk_ml, sk_o) may take
inline WsLayout ws_layout(const fa_params* p, uint64_t split_budget = kSplitScratchBudget) {
  WsLayout w;
  w.Hq1 = (p->eq_stride[1] == 0) ? 1 : p->H;
  w.Hk1 = (p->ek_stride[1] == 0) ? 1 : p->H;
  w.Mp = (p->M + kSumRows - 1) / kSumRows * kSumRows;
  w.nKs = (p->N + kSumRows - 1) / kSumRows;
  w.Np = w.nKs * kSumRows;
  w.Pp = (p->M + kPermAlign - 1) / kPermAlign * kPermAlign + kPermAlign;
  w.nQs = w.Pp / kSumRows;
  uint64_t o = 0;
  auto take = [&](uint64_t bytes) { uint64_t r = o; o += (bytes + 255) & ~uint64_t(255); return r; };
  w.off_eq32 = take(uint64_t(p->B) * w.Hq1 * w.Mp * 4);
  w.off_ek32 = take(uint64_t(p->B) * w.Hk1 * w.Np * 4);
  w.off_perm = take(uint64_t(p->B) * w.Hq1 * w.Pp * 4);
  w.off_peq = take(uint64_t(p->B) * w.Hq1 * w.Pp * 4);
  w.off_ppos = take(uint64_t(p->B) * w.Hq1 * w.Pp * 4);
  w.nCh = (w.Mp + 1023) / 1024;
  w.off_cnt = take(uint64_t(p->B) * w.Hq1 * w.nCh * 4);
  w.off_qhdr = take(uint64_t(p->B) * w.Hq1 * sizeof(QHeader));
  w.off_qsum = take(uint64_t(p->B) * w.Hq1 * w.nQs * sizeof(IdSummary));
  w.off_ksum = take(uint64_t(p->B) * w.Hk1 * w.nKs * sizeof(IdSummary));
  // scratch of the split tiles: only when a key range can be long enough to be cut
  const SplitCfg sc = split_config(p->B, p->H, p->M, p->N, p->D, split_budget);
  w.split = sc;
  const uint64_t nsk = uint64_t(p->B) * p->H * sc.tiles;
  w.off_sk_cnt = take(nsk * 4);
  w.plan_bytes = o;      // the counters (zeroed by the plan, left at zero by every kernel) are state
  w.off_sk_ml = take(nsk * sc.k * 128 * 2 * 4);
  w.off_sk_o = take(nsk * sc.k * 128 * uint64_t(p->D) * 4);
  w.total = o;
  return w;
}

// Raise the dynamic LDS limit of a kernel once per device (the attribute is per device and per
// kernel; a process may drive several GPUs).  `done` is the caller's per-kernel record.
template <typename K>
static int allow_lds(K kern, size_t lds, bool (&done)[64]) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= 64 || !done[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    if (dev >= 0 && dev < 64) done[dev] = true;
  }
  return 0;
}

// Launchers implemented one per translation unit; each returns a hipError_t as int.
int launch_fwd(const KArgs& a, int dtype, int D, bool causal, bool doc, hipStream_t s);
int launch_bwd_delta(const KArgs& a, int dtype, int D, hipStream_t s);
int launch_bwd_dq(const KArgs& a, int dtype, int D, bool causal, bool doc, hipStream_t s);
int launch_bwd_dkdv(const KArgs& a, int dtype, int D, bool causal, bool doc, hipStream_t s);
int read_pair_wait_expired(unsigned long long* n);   // expired pair waits of the dk/dv kernel on the current device (synchronises)
#ifdef FA_TRACE
int trace_read_fwd(long long* host, int n);
int trace_read_dq(long long* host, int n);
int trace_read_dkdv(long long* host, int n);
#endif
// the same four for fp32 tensors (fa_f32.hip)
int launch_fwd_f32(const KArgs& a, int D, bool causal, bool doc, hipStream_t s);
int launch_bwd_delta_f32(const KArgs& a, int D, hipStream_t s);
int launch_bwd_dq_f32(const KArgs& a, int D, bool causal, bool doc, hipStream_t s);
int launch_bwd_dkdv_f32(const KArgs& a, int D, bool causal, bool doc, hipStream_t s);
int launch_mask_plan(const fa_params* p, const WsLayout& w, hipStream_t s);
int launch_mask_dump(const KArgs& a, bool causal, bool doc, uint8_t* out, hipStream_t s);

}  // namespace fa
