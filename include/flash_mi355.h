/*
 * flash_mi355.h -- C ABI of the MI355X (gfx950) flexible-mask flash-attention library.
 *
 * One shared library, plain pointers and sizes, no torch or HIP types in any
 * signature (a HIP stream is passed as void*).  The library allocates nothing,
 * keeps no state between calls and never synchronises the host: every entry
 * point enqueues kernels on the caller's stream and returns.
 *
 * Each entry point replaces one launch site of the reference operator
 * (flash_triton.py of zzsfornlp/Triton-Flash-Attention-with-Flexible-Masks):
 *
 *   fa_fwd        <- _fwd_kernel[grid](...)          flash_triton.py:541-556
 *   fa_bwd_delta  <- _bwd_preprocess[grid](...)      flash_triton.py:585-592
 *   fa_bwd_dkdv   <- _bwd_kv_kernel[grid](...)       flash_triton.py:596-614
 *   fa_bwd_dq     <- _bwd_q_kernel[grid](...)        flash_triton.py:617-634
 *   fa_mask_plan  <- (no counterpart: the reference evaluates the doc mask on
 *                     every tile, README.md:18)  builds the per-tile id
 *                     summaries the kernels use to skip fully masked tiles
 *   fa_mask_dump  <- the mask expression of flash_triton.py:103-116 written out
 *                     as bytes, for bit-exact mask tests
 *   fa_validate   <- the asserts of FlashAttention.forward, flash_triton.py:508-530
 *
 * Tensor conventions (identical to the reference, flash_triton.py:27-36):
 *   q, o, dout, dq : [B, H,  M, D]      k, v : [B, Hk, N, D]   (H % Hk == 0)
 *   dk, dv         : [B, Hk, N, D]      already summed over the query heads of each
 *                                       group (the reference writes [B,H,N,D] and
 *                                       sums afterwards, flash_triton.py:594-595,635-637)
 *   lse, delta     : [B, H, M] float32, contiguous.  lse is in log2 units
 *                    (m + log2(l), flash_triton.py:133); -inf for a row with
 *                    no unmasked key
 *   eq : [B, H, M]   ek : [B, H, N]     integer ids, indexed by the *query* head
 *                                       (flash_triton.py:75-76), any strides
 *                                       including 0
 * Strides are in elements.  The innermost stride of every 4-D tensor must be 1
 * (the reference forces that with maybe_contiguous, flash_triton.py:435-437,525).
 * Base pointers must be 16-byte aligned and outer strides multiples of 16 bytes
 * (8 elements of a 16-bit type, 4 of fp32).
 */
#ifndef FLASH_MI355_H
#define FLASH_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_ABI_VERSION 7

/* score_func_mode, flash_triton.py:20-22 */
#define FA_SCORE_MODE0_NOPE 0
#define FA_SCORE_MODE1_DOC  1
/* Block mask (no counterpart in the reference, whose README.md:17-18 names block-sparse patterns as the
   extension point): `eq` points to bytes [B, H, ceil(M/64), ceil(N/64)], eq_stride = its batch, head
   and row strides in bytes (0 allowed for batch and head), the column stride is 1; `ek`, `id_dtype`
   and the workspace are not used and fa_mask_plan is not needed.  A pair (i, j) is kept iff the byte of
   block (i / 64, j / 64) is non-zero and the causal / window / prefix terms hold. */
#define FA_SCORE_MODE2_BLOCK 2
#define FA_MASK_BLOCK 64

/* element types */
#define FA_DTYPE_BF16 0
#define FA_DTYPE_FP16 1
#define FA_DTYPE_FP32 2   /* fp32 tensors: fp32 MFMA throughout (the reference takes fp32 like any float type) */
#define FA_IDTYPE_I32 0
#define FA_IDTYPE_I64 1   /* values must fit in int32: fa_mask_plan narrows them with saturation */

/* return codes */
#define FA_OK                    0
#define FA_ERR_NULLPTR          -1
#define FA_ERR_UNSUPPORTED_D    -2   /* D not in {16,32,64,128}: flash_triton.py:512 */
#define FA_ERR_DTYPE            -3
#define FA_ERR_SHAPE            -4   /* H % Hk != 0, causal with N < M (without qpos), sizes <= 0 */
#define FA_ERR_ALIGN            -5
#define FA_ERR_STRIDE           -6
#define FA_ERR_MODE             -7   /* unknown score mode, doc mode without ids, window / prefix / qpos misuse */
#define FA_ERR_WORKSPACE        -8   /* workspace missing or too small */
#define FA_ERR_HIP              -9   /* kernel launch failed; see fa_last_hip_error */
#define FA_ERR_NOT_IMPLEMENTED -10

/* fa_params.flags */
#define FA_FLAG_DQ_DELTA 1  /* fa_bwd_dq computes delta = rowsum(o * dout) of its own rows itself (o must be set)
                               and also stores it to p->delta: the fa_bwd_delta launch is then not needed, and
                               fa_bwd_dkdv, which reads delta, goes after fa_bwd_dq on the stream.
                               Ignored by every other call. */
#define FA_FLAG_DEBUG_NO_PAIR_WAIT 0x100
                            /* Diagnostic, for tests of the failure path below; never set it in production.
                               In fa_bwd_dkdv at D = 128 two waves share each block of 32 keys: one publishes P in
                               on-chip memory, the other polls a sequence number for it.  The poll is bounded (about
                               a millisecond) so that every wave ends whatever happens; a wave whose wait expired
                               has used a P it cannot trust and REPORTS it by writing NaN into its 32 rows of dk
                               (dv is not affected).  A NaN in dk after a backward with finite inputs therefore
                               means "a pair wait expired", not an arithmetic overflow.  With this flag the poll
                               budget is zero, so the report can be provoked without hanging or faulting anything.
                               Accepted by fa_bwd_dkdv only; every other entry point refuses it (FA_ERR_MODE).
                               Every expiry is also counted, see fa_pair_wait_expired. */

typedef struct fa_params {
  /* forward operands */
  const void* q;
  const void* k;
  const void* v;
  void*       o;
  float*      lse;        /* [B,H,M] log2-domain */
  /* backward operands */
  const void* dout;
  void*       dq;
  void*       dk;         /* [B,Hk,N,D] */
  void*       dv;         /* [B,Hk,N,D] */
  float*      delta;      /* [B,H,M] */
  /* flexible-mask ids */
  const void* eq;
  const void* ek;
  /* scratch written by fa_mask_plan and read by the compute kernels
     (required when score_mode != 0; size from fa_workspace_bytes) */
  void*       workspace;
  uint64_t    workspace_bytes;

  int64_t q_stride[4], k_stride[4], v_stride[4], o_stride[4];
  int64_t do_stride[4], dq_stride[4], dk_stride[4], dv_stride[4];
  int64_t eq_stride[3], ek_stride[3];

  int32_t B, H, Hk, M, N, D;
  int32_t causal;         /* bottom-right aligned: keep iff max(0,N-M)+i >= j */
  int32_t score_mode;     /* FA_SCORE_MODE* */
  int32_t dtype;          /* FA_DTYPE_*  (q,k,v,o,dout,dq,dk,dv share it) */
  int32_t id_dtype;       /* FA_IDTYPE_* (eq, ek) */
  float   sm_scale;
  int32_t flags;          /* FA_FLAG_* bits, 0 for the reference's launch sequence */
  /* Two more causal masks on the same machinery (no counterpart in the reference, whose README.md:17-18
     names such masks as the extension point); 0 = off; both need causal != 0 and exclude each other:
       window > 0 : sliding window -- row i sees only the last `window` keys up to its diagonal:
                    keep additionally needs j > max(0,N-M) + i - window
       prefix > 0 : prefix-LM -- the first `prefix` keys are seen by every row:
                    the causal term becomes (max(0,N-M) + i >= j) || (j < prefix)                     */
  int32_t window;
  int32_t prefix;
  /* Per-row causal positions (no counterpart in the reference, whose causal bound is the one offset
     max(0,N-M) of flash_triton.py:521): int32 [B, M], row stride 1, or NULL.  With causal != 0 and
     score_mode == FA_SCORE_MODE1_DOC, row i of batch b has its diagonal at key qpos[b][i] instead of
     max(0,N-M)+i: keep needs j <= qpos[b][i] (and j > qpos[b][i] - window).  Values are clamped to
     >= -1 (-1: the row sees no key).  This is what a packed batch needs whose query and key
     boundaries differ (every sequence bottom-right aligned on its own: the tail of a longer key
     sequence, chunked prefill, decoding): the ids confine a row to its sequence and qpos places its
     diagonal.  N >= M is not required then.  Excludes prefix.  Read by fa_mask_plan only (which
     stores the positions with the plan), and by fa_mask_dump. */
  const int32_t* qpos;
  int64_t qpos_stride;    /* batch stride of qpos in elements (0: one vector for every batch) */
  /* Optional home of the stateless part of the workspace (the partial results of key ranges that are
     split over several workgroups), so that a caller can keep the small plan between forward and
     backward -- as the reference keeps eq / ek in its ctx, flash_triton.py:557-562 -- without holding
     on to, copying or re-planning anything else.  NULL: that part follows the plan inside `workspace`
     (which then needs fa_workspace_bytes).  Non-NULL (256-byte aligned, at least
     fa_workspace_scratch_bytes): `workspace` needs fa_workspace_plan_bytes only.  Nothing is carried in
     it from one call to the next; two launches that share it must be ordered on one stream. */
  void*       split_scratch;
  uint64_t    split_scratch_bytes;
} fa_params;

/* ABI version of the loaded library (== FA_ABI_VERSION of the header it was built from). */
int fa_version(void);

/* sizeof(fa_params) as compiled, so a binding can check its own struct packing. */
uint64_t fa_params_size(void);

/* Static text for a return code. */
const char* fa_error_string(int code);

/* hipError_t of the last failed launch on this thread (0 if none). */
int fa_last_hip_error(void);

/* Shape / dtype / stride / alignment / null checks for the given stage.
   Touches no GPU API; callable on a machine without a GPU.
   stage: 0 = forward, 1 = backward (fa_bwd_delta, fa_bwd_dq), 2 = mask plan only,
          3 = fa_bwd_dkdv (stage 1, and FA_FLAG_DEBUG_NO_PAIR_WAIT is accepted). */
int fa_validate(const fa_params* p, int stage);

/* Bytes of workspace fa_mask_plan needs for these sizes (0 when score_mode == 0). */
uint64_t fa_workspace_bytes(const fa_params* p);

/* The first fa_workspace_plan_bytes() bytes of the workspace carry the plan from fa_mask_plan to
   the compute calls (and stay valid after them); the rest is scratch without state between calls.
   A caller that keeps a plan between forward and backward (as the reference keeps eq/ek,
   flash_triton.py:557) needs to keep this prefix only and may copy it into a fresh workspace. */
uint64_t fa_workspace_plan_bytes(const fa_params* p);

/* Bytes of the stateless rest (what p->split_scratch may carry instead of the tail of the workspace);
   fa_workspace_bytes = plan bytes + scratch bytes.  0 when no key range of these sizes is ever split. */
uint64_t fa_workspace_scratch_bytes(const fa_params* p);

/* Mask engine: normalise eq/ek to int32 and build per-tile id summaries
   into p->workspace.  Must be enqueued before fa_fwd / fa_bwd_* on the same
   stream whenever score_mode != 0.  The same workspace serves forward and backward.
   The plan depends on the ids, the sizes AND on `causal` and `prefix` (key ranges are narrowed with
   the causal bound): plan again when any of them changes.  The workspace also holds the scratch
   of the tiles whose key range is split over several workgroups, so two launches that share a
   workspace must be ordered on one stream. */
int fa_mask_plan(const fa_params* p, void* stream);

/* O = softmax(q k^T * sm_scale + mask) v ; lse = log2-sum-exp2 of the scaled scores. */
int fa_fwd(const fa_params* p, void* stream);

/* fa_fwd for callers that cannot allocate device memory and hold no workspace (code under HIP graph
   capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
   Same operands and results as fa_mask_plan + fa_fwd, but p->workspace / p->workspace_bytes are
   ignored: the mask plan and the scratch of the split key ranges live in a static device array of
   FA_STATIC_WS_BYTES inside the library (held by every GPU the library runs on until the process
   ends).  The call enqueues the plan kernels and the forward on `stream` and allocates nothing, on
   the host or the device.  Problems whose plan does not fit the array are refused with
   FA_ERR_WORKSPACE (the plan needs about 17 bytes per query row and 5 per key, times the batch, times
   the heads unless the ids' head stride is 0; the headline shape B=1 H=32 L=16384 takes 0.5 MB plus
   split scratch).  Every call on a GPU uses that GPU's one array, which keeps the last call's
   contents: calls that overlap on one GPU (different streams, different threads) race and must be
   ordered by the caller; a backward needs its own fa_mask_plan into a caller's workspace.
   With score_mode 0 or 2 there is no workspace and the call is fa_fwd. */
#define FA_STATIC_WS_BYTES (32u << 20)
int fa_fwd_static(const fa_params* p, void* stream);

/* delta = rowsum(o * dout). */
int fa_bwd_delta(const fa_params* p, void* stream);

/* dk, dv summed over each group's query heads (needs lse, delta). */
int fa_bwd_dkdv(const fa_params* p, void* stream);

/* dq (needs lse, and delta unless FA_FLAG_DQ_DELTA is set). */
int fa_bwd_dq(const fa_params* p, void* stream);

/* Number of wave-level pair waits of fa_bwd_dkdv that expired on the current device since the library
   was loaded (see FA_FLAG_DEBUG_NO_PAIR_WAIT: each one also shows as NaN in 32 rows of dk).  0 in any
   healthy run.  Waits for the device to be idle before it reads the count (a diagnostic, not for hot
   loops); returns FA_OK or FA_ERR_HIP.  No counterpart in the reference. */
int fa_pair_wait_expired(uint64_t* count);

/* Write keep(i,j) as one byte (0/1) per element into out[B,H,M,N] (contiguous),
   evaluated by the same device routine the compute kernels use. */
int fa_mask_dump(const fa_params* p, uint8_t* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_MI355_H */
