// C ABI of the library (see include/flash_mi355.h): argument validation that
// mirrors the asserts of FlashAttention.forward (flash_triton.py:508-530),
// translation of fa_params into the kernel-side view, and dispatch.
#include <atomic>

#include "fa_common.h"

using namespace fa;

static thread_local int g_last_hip_error = 0;

static bool d_supported(int D) { return D == 16 || D == 32 || D == 64 || D == 128; }

// rows/D: extent of one (batch, head) slice; the kernels address a slice through a
// buffer resource whose byte range must stay below 2 GiB
static int check_tensor(const void* ptr, const int64_t* st, int rows, int D, int dtype) {
  const int esize = dtype == FA_DTYPE_FP32 ? 4 : 2, per16 = 16 / esize;
  if (ptr == nullptr) return FA_ERR_NULLPTR;
  if (st[2] < 0 || (int64_t(rows - 1) * st[2] + D) * esize >= (int64_t(1) << 31)) return FA_ERR_NOT_IMPLEMENTED;
  if ((reinterpret_cast<uintptr_t>(ptr) & 15) != 0) return FA_ERR_ALIGN;
  if (st[3] != 1) return FA_ERR_STRIDE;
  if ((st[0] % per16) != 0 || (st[1] % per16) != 0 || (st[2] % per16) != 0) return FA_ERR_ALIGN;
  return FA_OK;
}

extern "C" int fa_version(void) { return FA_ABI_VERSION; }
extern "C" uint64_t fa_params_size(void) { return sizeof(fa_params); }
extern "C" int fa_last_hip_error(void) { return g_last_hip_error; }

extern "C" const char* fa_error_string(int code) {
  switch (code) {
    case FA_OK: return "ok";
    case FA_ERR_NULLPTR: return "null pointer for a required operand";
    case FA_ERR_UNSUPPORTED_D: return "head dimension must be one of 16, 32, 64, 128";
    case FA_ERR_DTYPE: return "unsupported element or id type";
    case FA_ERR_SHAPE: return "inconsistent sizes (H % Hk != 0, causal with N < M and no qpos, or a size <= 0)";
    case FA_ERR_ALIGN: return "pointers must be 16-byte aligned and outer strides multiples of 16 bytes";
    case FA_ERR_STRIDE: return "innermost stride must be 1";
    case FA_ERR_MODE: return "unknown score mode, doc mode without eq/ek, window / prefix without causal (or both), or qpos without causal + ids (or with prefix)";
    case FA_ERR_WORKSPACE: return "workspace missing or too small";
    case FA_ERR_HIP: return "kernel launch failed";
    case FA_ERR_NOT_IMPLEMENTED: return "configuration not implemented";
    default: return "unknown error";
  }
}

extern "C" int fa_validate(const fa_params* p, int stage) {
  if (p == nullptr) return FA_ERR_NULLPTR;
  if (!d_supported(p->D)) return FA_ERR_UNSUPPORTED_D;
  if (p->dtype != FA_DTYPE_BF16 && p->dtype != FA_DTYPE_FP16 && p->dtype != FA_DTYPE_FP32) return FA_ERR_DTYPE;
  if (p->B <= 0 || p->H <= 0 || p->Hk <= 0 || p->M <= 0 || p->N <= 0) return FA_ERR_SHAPE;
  if (p->H % p->Hk != 0) return FA_ERR_SHAPE;
  if (p->causal && p->N < p->M && p->qpos == nullptr) return FA_ERR_SHAPE;
  if (p->score_mode != FA_SCORE_MODE0_NOPE && p->score_mode != FA_SCORE_MODE1_DOC && p->score_mode != FA_SCORE_MODE2_BLOCK)
    return FA_ERR_MODE;
  if (p->score_mode == FA_SCORE_MODE2_BLOCK) {
    if (p->eq == nullptr) return FA_ERR_MODE;
    if (p->eq_stride[0] < 0 || p->eq_stride[1] < 0 || p->eq_stride[2] < (p->N + FA_MASK_BLOCK - 1) / FA_MASK_BLOCK) return FA_ERR_STRIDE;
  }
  if ((p->flags & ~(FA_FLAG_DQ_DELTA | FA_FLAG_DEBUG_NO_PAIR_WAIT)) != 0) return FA_ERR_MODE;
  if ((p->flags & FA_FLAG_DEBUG_NO_PAIR_WAIT) != 0 && stage != 3) return FA_ERR_MODE;   // a diagnostic of fa_bwd_dkdv alone
  if (p->window < 0 || p->prefix < 0 || (p->window > 0 && p->prefix > 0)) return FA_ERR_MODE;
  if ((p->window > 0 || p->prefix > 0) && !p->causal) return FA_ERR_MODE;
  if (p->qpos != nullptr && (!p->causal || p->score_mode != FA_SCORE_MODE1_DOC || p->prefix > 0 || p->qpos_stride < 0)) return FA_ERR_MODE;
  if (p->score_mode == FA_SCORE_MODE1_DOC) {
    if (p->eq == nullptr || p->ek == nullptr) return FA_ERR_MODE;
    if (p->id_dtype != FA_IDTYPE_I32 && p->id_dtype != FA_IDTYPE_I64) return FA_ERR_DTYPE;
    if (p->workspace == nullptr) return FA_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(p->workspace) & 255) != 0) return FA_ERR_ALIGN;
    if (p->split_scratch == nullptr) {
      if (p->workspace_bytes < fa_workspace_bytes(p)) return FA_ERR_WORKSPACE;
    } else {
      if ((reinterpret_cast<uintptr_t>(p->split_scratch) & 255) != 0) return FA_ERR_ALIGN;
      if (p->workspace_bytes < fa_workspace_plan_bytes(p)) return FA_ERR_WORKSPACE;
      if (p->split_scratch_bytes < fa_workspace_scratch_bytes(p)) return FA_ERR_WORKSPACE;
    }
  }
  if (stage == 2) return FA_OK;
  int rc;
  if ((rc = check_tensor(p->q, p->q_stride, p->M, p->D, p->dtype)) != FA_OK) return rc;
  if ((rc = check_tensor(p->k, p->k_stride, p->N, p->D, p->dtype)) != FA_OK) return rc;
  if ((rc = check_tensor(p->v, p->v_stride, p->N, p->D, p->dtype)) != FA_OK) return rc;
  if ((rc = check_tensor(p->o, p->o_stride, p->M, p->D, p->dtype)) != FA_OK) return rc;
  if (p->lse == nullptr) return FA_ERR_NULLPTR;
  if (stage == 1 || stage == 3) {
    if ((rc = check_tensor(p->dout, p->do_stride, p->M, p->D, p->dtype)) != FA_OK) return rc;
    if ((rc = check_tensor(p->dq, p->dq_stride, p->M, p->D, p->dtype)) != FA_OK) return rc;
    if ((rc = check_tensor(p->dk, p->dk_stride, p->N, p->D, p->dtype)) != FA_OK) return rc;
    if ((rc = check_tensor(p->dv, p->dv_stride, p->N, p->D, p->dtype)) != FA_OK) return rc;
    if (p->delta == nullptr) return FA_ERR_NULLPTR;
  }
  return FA_OK;
}

extern "C" uint64_t fa_workspace_bytes(const fa_params* p) {
  if (p == nullptr || p->score_mode != FA_SCORE_MODE1_DOC) return 0;
  if (p->B <= 0 || p->H <= 0 || p->M <= 0 || p->N <= 0) return 0;
  return ws_layout(p).total;
}

extern "C" uint64_t fa_workspace_plan_bytes(const fa_params* p) {
  if (p == nullptr || p->score_mode != FA_SCORE_MODE1_DOC) return 0;
  if (p->B <= 0 || p->H <= 0 || p->M <= 0 || p->N <= 0) return 0;
  return ws_layout(p).plan_bytes;
}

extern "C" uint64_t fa_workspace_scratch_bytes(const fa_params* p) {
  if (p == nullptr || p->score_mode != FA_SCORE_MODE1_DOC) return 0;
  if (p->B <= 0 || p->H <= 0 || p->M <= 0 || p->N <= 0) return 0;
  const WsLayout w = ws_layout(p);
  return w.total - w.plan_bytes;
}

static KArgs make_args(const fa_params* p, uint64_t split_budget = kSplitScratchBudget) {
  KArgs a;
  a.q = p->q; a.k = p->k; a.v = p->v; a.o = p->o; a.lse = p->lse;
  a.dout = p->dout; a.dq = p->dq; a.dk = p->dk; a.dv = p->dv; a.delta = p->delta;
  a.q_bs = p->q_stride[0]; a.q_hs = p->q_stride[1]; a.q_rs = p->q_stride[2];
  a.k_bs = p->k_stride[0]; a.k_hs = p->k_stride[1]; a.k_rs = p->k_stride[2];
  a.v_bs = p->v_stride[0]; a.v_hs = p->v_stride[1]; a.v_rs = p->v_stride[2];
  a.o_bs = p->o_stride[0]; a.o_hs = p->o_stride[1]; a.o_rs = p->o_stride[2];
  a.do_bs = p->do_stride[0]; a.do_hs = p->do_stride[1]; a.do_rs = p->do_stride[2];
  a.dq_bs = p->dq_stride[0]; a.dq_hs = p->dq_stride[1]; a.dq_rs = p->dq_stride[2];
  a.dk_bs = p->dk_stride[0]; a.dk_hs = p->dk_stride[1]; a.dk_rs = p->dk_stride[2];
  a.dv_bs = p->dv_stride[0]; a.dv_hs = p->dv_stride[1]; a.dv_rs = p->dv_stride[2];
  a.B = p->B; a.H = p->H; a.Hk = p->Hk; a.G = p->H / p->Hk; a.M = p->M; a.N = p->N;
  a.gap = p->N > p->M ? p->N - p->M : 0;  // flash_triton.py:521
  a.win = p->window > 0 ? (p->window < 0x3fffffff ? p->window : 0x3fffffff) : 0x3fffffff;
  a.pfx_m1 = p->prefix > 0 ? (p->prefix < p->N ? p->prefix : p->N) - 1 : -1;
  a.scale = p->sm_scale;
  a.scale_log2e = p->sm_scale * kLog2e;
  a.ppos = nullptr; a.qpos = p->qpos; a.qp_bs = p->qpos_stride;
  a.eq32 = nullptr; a.ek32 = nullptr; a.perm = nullptr; a.peq = nullptr; a.qhdr = nullptr; a.qsum = nullptr; a.ksum = nullptr;
  a.sk_cnt = nullptr; a.sk_ml = nullptr; a.sk_o = nullptr;
  a.split_k = 1; a.split_tiles = 0;
  a.eq_bs = a.eq_hs = a.ek_bs = a.ek_hs = a.pm_bs = a.pm_hs = a.qh_bs = a.qh_hs = 0;
  a.qs_bs = a.qs_hs = a.ks_bs = a.ks_hs = 0;
  a.nQs = a.nKs = a.Pp = 0;
  a.dq_delta = (p->flags & FA_FLAG_DQ_DELTA) != 0;
  a.pair_spin = (p->flags & FA_FLAG_DEBUG_NO_PAIR_WAIT) ? 0 : kPairSpinDefault;
  a.bmask = nullptr; a.bm_bs = a.bm_hs = a.bm_rs = 0;
  a.nBr = (p->M + FA_MASK_BLOCK - 1) / FA_MASK_BLOCK; a.nBc = (p->N + FA_MASK_BLOCK - 1) / FA_MASK_BLOCK;
  if (p->score_mode == FA_SCORE_MODE2_BLOCK) {
    a.bmask = reinterpret_cast<const unsigned char*>(p->eq);
    a.bm_bs = p->eq_stride[0]; a.bm_hs = p->eq_stride[1]; a.bm_rs = p->eq_stride[2];
  }
  if (p->score_mode == FA_SCORE_MODE1_DOC) {
    const WsLayout w = ws_layout(p, split_budget);
    char* ws = reinterpret_cast<char*>(p->workspace);
    a.eq32 = reinterpret_cast<const int*>(ws + w.off_eq32);
    a.ek32 = reinterpret_cast<const int*>(ws + w.off_ek32);
    a.perm = reinterpret_cast<const int*>(ws + w.off_perm);
    a.peq = reinterpret_cast<const int*>(ws + w.off_peq);
    a.ppos = reinterpret_cast<const int*>(ws + w.off_ppos);
    a.qhdr = reinterpret_cast<const QHeader*>(ws + w.off_qhdr);
    a.qsum = reinterpret_cast<const IdSummary*>(ws + w.off_qsum);
    a.ksum = reinterpret_cast<const IdSummary*>(ws + w.off_ksum);
    a.eq_bs = int64_t(w.Hq1) * w.Mp; a.eq_hs = w.Hq1 == 1 ? 0 : w.Mp;
    a.ek_bs = int64_t(w.Hk1) * w.Np; a.ek_hs = w.Hk1 == 1 ? 0 : w.Np;
    a.pm_bs = int64_t(w.Hq1) * w.Pp; a.pm_hs = w.Hq1 == 1 ? 0 : w.Pp;
    a.qh_bs = w.Hq1; a.qh_hs = w.Hq1 == 1 ? 0 : 1;
    a.qs_bs = int64_t(w.Hq1) * w.nQs; a.qs_hs = w.Hq1 == 1 ? 0 : w.nQs;
    a.ks_bs = int64_t(w.Hk1) * w.nKs; a.ks_hs = w.Hk1 == 1 ? 0 : w.nKs;
    a.nQs = w.nQs; a.nKs = w.nKs; a.Pp = w.Pp;
    const SplitCfg sc = w.split;
    a.split_k = sc.k; a.split_tiles = sc.tiles;
    a.sk_cnt = reinterpret_cast<int*>(ws + w.off_sk_cnt);
    // the stateless part: behind the plan, or in the caller's separate scratch
    char* sc_base = p->split_scratch != nullptr ? reinterpret_cast<char*>(p->split_scratch) - w.plan_bytes : ws;
    a.sk_ml = reinterpret_cast<float*>(sc_base + w.off_sk_ml);
    a.sk_o = reinterpret_cast<float*>(sc_base + w.off_sk_o);
  }
  return a;
}

static int finish(int hip_rc) {
  if (hip_rc == 0) return FA_OK;
  if (hip_rc < 0) return FA_ERR_NOT_IMPLEMENTED;
  g_last_hip_error = hip_rc;
  return FA_ERR_HIP;
}

extern "C" int fa_mask_plan(const fa_params* p, void* stream) {
  int rc = fa_validate(p, 2);
  if (rc != FA_OK) return rc;
  if (p->score_mode != FA_SCORE_MODE1_DOC) return FA_OK;
  return finish(launch_mask_plan(p, ws_layout(p), reinterpret_cast<hipStream_t>(stream)));
}

extern "C" int fa_fwd(const fa_params* p, void* stream) {
  int rc = fa_validate(p, 0);
  if (rc != FA_OK) return rc;
  const bool causal = p->causal != 0, doc = p->score_mode == FA_SCORE_MODE1_DOC;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (p->dtype == FA_DTYPE_FP32) return finish(launch_fwd_f32(make_args(p), p->D, causal, doc, s));
  return finish(launch_fwd(make_args(p), p->dtype, p->D, causal, doc, s));
}

// ---------------------------------------------------------------------------
// Forward without any allocation anywhere: the mask plan and the scratch of the split key ranges
// live in a static device array instead of a caller's workspace.  Every GPU the library runs on
// holds its own copy of the array at its own address until the process ends; the address is looked
// up once per device (with that device current) and only that pointer is ever handed to kernels,
// memsets or copies -- the array's name is a host-side stand-in, not a device address.
// ---------------------------------------------------------------------------
constexpr uint64_t kStaticSplitBudget = uint64_t(24) << 20;   // of FA_STATIC_WS_BYTES; the rest is for the plan
static __device__ __align__(256) unsigned char scratch[FA_STATIC_WS_BYTES];
static std::atomic<void*> g_scratch_ptr[64];

static int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= 64) return (int)hipErrorInvalidDevice;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));   // this device's copy (the current device)
    if (e != hipSuccess) return (int)e;
    if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // racing first calls find the same address
  }
  *out = ptr;
  return 0;
}

extern "C" int fa_fwd_static(const fa_params* p, void* stream) {
  if (p == nullptr) return FA_ERR_NULLPTR;
  if (p->score_mode != FA_SCORE_MODE1_DOC) return fa_fwd(p, stream);   // no workspace in these modes
  fa_params q = *p;
  q.workspace = reinterpret_cast<void*>(uintptr_t(256));   // placeholder for the checks below; replaced before any launch
  q.workspace_bytes = ~uint64_t(0);
  int rc = fa_validate(&q, 0);
  if (rc != FA_OK) return rc;
  const WsLayout w = ws_layout(&q, kStaticSplitBudget);
  if (w.total > FA_STATIC_WS_BYTES) return FA_ERR_WORKSPACE;   // sizes beyond the static array
  void* ws = nullptr;
  if (int e = static_scratch(&ws)) return finish(e);
  q.workspace = ws;
  q.workspace_bytes = FA_STATIC_WS_BYTES;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // the plan rewrites everything the kernels read (ids, order, summaries) and zeroes the arrival
  // counters with a kernel, so nothing of an earlier call's contents is ever looked at
  if (int e = launch_mask_plan(&q, w, s)) return finish(e);
  const bool causal = q.causal != 0;
  if (q.dtype == FA_DTYPE_FP32) return finish(launch_fwd_f32(make_args(&q, kStaticSplitBudget), q.D, causal, true, s));
  return finish(launch_fwd(make_args(&q, kStaticSplitBudget), q.dtype, q.D, causal, true, s));
}

extern "C" int fa_bwd_delta(const fa_params* p, void* stream) {
  int rc = fa_validate(p, 1);
  if (rc != FA_OK) return rc;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (p->dtype == FA_DTYPE_FP32) return finish(launch_bwd_delta_f32(make_args(p), p->D, s));
  return finish(launch_bwd_delta(make_args(p), p->dtype, p->D, s));
}

extern "C" int fa_pair_wait_expired(uint64_t* count) {
  if (count == nullptr) return FA_ERR_NULLPTR;
  unsigned long long n = 0;
  if (int e = read_pair_wait_expired(&n)) return finish(e);
  *count = n;
  return FA_OK;
}

extern "C" int fa_bwd_dkdv(const fa_params* p, void* stream) {
  int rc = fa_validate(p, 3);
  if (rc != FA_OK) return rc;
  const bool causal = p->causal != 0, doc = p->score_mode == FA_SCORE_MODE1_DOC;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (p->dtype == FA_DTYPE_FP32) return finish(launch_bwd_dkdv_f32(make_args(p), p->D, causal, doc, s));
  return finish(launch_bwd_dkdv(make_args(p), p->dtype, p->D, causal, doc, s));
}

extern "C" int fa_bwd_dq(const fa_params* p, void* stream) {
  int rc = fa_validate(p, 1);
  if (rc != FA_OK) return rc;
  const bool causal = p->causal != 0, doc = p->score_mode == FA_SCORE_MODE1_DOC;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (p->dtype == FA_DTYPE_FP32) return finish(launch_bwd_dq_f32(make_args(p), p->D, causal, doc, s));
  return finish(launch_bwd_dq(make_args(p), p->dtype, p->D, causal, doc, s));
}

extern "C" int fa_mask_dump(const fa_params* p, uint8_t* out, void* stream) {
  int rc = fa_validate(p, 2);
  if (rc != FA_OK) return rc;
  if (out == nullptr) return FA_ERR_NULLPTR;
  return finish(launch_mask_dump(make_args(p), p->causal != 0, p->score_mode == FA_SCORE_MODE1_DOC, out,
                                 reinterpret_cast<hipStream_t>(stream)));
}

#ifdef FA_TRACE
// Measurement build only (not part of the product library or of its header): copies the clock
// stamps of the last launch of one kernel to the host, 8 words per workgroup.
// which: 0 forward, 1 dQ, 2 dK/dV.  n = number of 64-bit words (at most 8 * 65536).
extern "C" int fa_trace_read(int which, long long* host, int n) {
  if (host == nullptr) return FA_ERR_NULLPTR;
  if (n < 0 || n > 8 * fa::kTraceWgs) return FA_ERR_SHAPE;
  hipDeviceSynchronize();
  const int e = which == 0 ? fa::trace_read_fwd(host, n) : which == 1 ? fa::trace_read_dq(host, n) : fa::trace_read_dkdv(host, n);
  return e == 0 ? FA_OK : FA_ERR_HIP;
}
#endif
