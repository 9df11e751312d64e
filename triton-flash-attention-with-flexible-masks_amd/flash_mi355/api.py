"""Drop-in operator: ``attention(q, k, v, causal, sm_scale, eq, ek, score_func_mode)``.

Same entry point, argument order, defaults, checks and return values as the
reference's ``flash_triton.attention`` / ``FlashAttention`` (flash_triton.py:506-641);
the kernels behind it are the hand-written gfx950 kernels of libflash_mi355.so.
torch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes
import math

import torch

from . import _cabi

SCORE_FUNC_MODE0_NOPE = 0  # flash_triton.py:20
SCORE_FUNC_MODE1_DOC = 1   # flash_triton.py:22
SCORE_FUNC_MODE2_BLOCK = 2  # block mask: set by the block_mask argument of attention(), no counterpart in the reference

_DTYPES = {torch.bfloat16: _cabi.FA_DTYPE_BF16, torch.float16: _cabi.FA_DTYPE_FP16, torch.float32: _cabi.FA_DTYPE_FP32}
_ID_DTYPES = {torch.int32: _cabi.FA_IDTYPE_I32, torch.int64: _cabi.FA_IDTYPE_I64}


def maybe_contiguous(x):
    """Innermost dimension must be contiguous (flash_triton.py:435-437)."""
    return x.contiguous() if x.stride(-1) != 1 else x


def _aligned(x):
    """16-byte aligned base and outer strides that are multiples of 16 bytes."""
    per16 = 16 // x.element_size()
    ok = x.data_ptr() % 16 == 0 and all(s % per16 == 0 for s in x.stride()[:-1])
    return x if ok else x.contiguous()


def _set4(dst, t):
    for i in range(4):
        dst[i] = t.stride(i)


def _set3(dst, t):
    for i in range(3):
        dst[i] = t.stride(i)


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class _Plan:
    """fa_params filled in for one problem, plus the tensors that keep its pointers alive."""

    def __init__(self, q, k, v, causal, sm_scale, eq, ek, score_func_mode, window=0, prefix=0, qpos=None):
        B, H, M, D = q.shape
        N, Hk = k.shape[2], k.shape[1]
        p = _cabi.FaParams()
        p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
        _set4(p.q_stride, q); _set4(p.k_stride, k); _set4(p.v_stride, v)
        p.B, p.H, p.Hk, p.M, p.N, p.D = B, H, Hk, M, N, D
        p.causal = 1 if causal else 0
        p.score_mode = int(score_func_mode)
        p.dtype = _DTYPES[q.dtype]
        p.sm_scale = float(sm_scale)
        p.flags = 0
        p.window, p.prefix = int(window), int(prefix)
        self.keep = [q, k, v]
        if score_func_mode == SCORE_FUNC_MODE2_BLOCK:   # eq is the block map [B, H, rows of blocks, columns of blocks], bytes
            p.eq = eq.data_ptr()
            _set3(p.eq_stride, eq)
            self.keep += [eq]
        elif score_func_mode != SCORE_FUNC_MODE0_NOPE:
            p.eq, p.ek = eq.data_ptr(), ek.data_ptr()
            _set3(p.eq_stride, eq); _set3(p.ek_stride, ek)
            p.id_dtype = _ID_DTYPES[eq.dtype]
            self.keep += [eq, ek]
        if qpos is not None:   # int32 [B | 1, M], row stride 1
            p.qpos = qpos.data_ptr()
            p.qpos_stride = qpos.stride(0) if qpos.shape[0] > 1 else 0
            self.keep += [qpos]
        self.p = p
        self.workspace = None
        self.scratch = None

    def ensure_workspace(self, device, plan_state=None):
        """Workspace of the call: the small part that carries the mask plan (a tensor of its own, which the
        forward hands to the backward as it is -- nothing is cloned, copied or planned twice) and the
        stateless scratch of the split key ranges (a fresh tensor per call from torch's caching allocator,
        released when the call's kernels are done).  plan_state: a plan written by an earlier call."""
        L = _cabi.lib()
        nplan = int(L.fa_workspace_plan_bytes(ctypes.byref(self.p)))
        if not nplan or self.workspace is not None:
            return
        self.workspace = plan_state if plan_state is not None else torch.empty(nplan, dtype=torch.uint8, device=device)
        self.p.workspace = self.workspace.data_ptr()
        self.p.workspace_bytes = self.workspace.numel()
        nscr = int(L.fa_workspace_scratch_bytes(ctypes.byref(self.p)))
        # (a pointer of its own even when nothing is split, so that the plan part alone is a valid workspace)
        self.scratch = torch.empty(max(nscr, 256), dtype=torch.uint8, device=device)
        self.p.split_scratch = self.scratch.data_ptr()
        self.p.split_scratch_bytes = self.scratch.numel()
        if plan_state is None:
            _cabi.check(L.fa_mask_plan(ctypes.byref(self.p), _stream_ptr(device)), "fa_mask_plan")


def _prep_ids(e, name):
    assert e.dim() == 3, f"{name} must be [bs, H, L]"
    if e.dtype not in _ID_DTYPES:
        assert not e.dtype.is_floating_point and e.dtype != torch.bool, f"{name} must be an integer tensor"
        e = e.to(torch.int32) if e.dtype in (torch.int8, torch.int16, torch.uint8) else e.to(torch.int64)
    return e


def _check_same_device(ref, **others):
    """Every tensor whose address is handed to a kernel lives on the device the kernels run on (a host
    or foreign pointer would be a memory fault on the GPU, not an error)."""
    for name, t in others.items():
        assert t is None or t.device == ref.device, f"{name} is on {t.device}, q is on {ref.device}: all operands must share q's device"


def _short_query_long_key(B, H, M, N, dtype):
    """No ids, fewer query tiles than half the chip has CUs, and a key range long enough to be cut (16-bit types)."""
    return dtype != torch.float32 and B * H * ((M + 127) // 128) <= 128 and N >= 8192


class _Impl:
    """Forward and backward shared by the two autograd functions below."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, eq, ek, score_func_mode, window=0, prefix=0, qpos=None):
        # -- checks of flash_triton.py:510-530, same order and messages --
        Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
        assert Dq == Dk and Dk == Dv, "feature size of q, k, v should be equal"
        assert Dk in {16, 32, 64, 128}
        B, H, M, D = q.shape
        N = k.shape[2]
        Hk, Hv = k.shape[1], v.shape[1]
        assert Hk == Hv, "num of heads in k and v should be equal"
        assert H % Hk == 0, "number of heads in q must be a multiple of that in k & v"
        num_groups = H // Hk
        assert (N >= M) or (not causal) or (qpos is not None), "KV length should be larger than M length in causal mode!"
        MN_GAP = max(0, N - M)
        if sm_scale is None:
            sm_scale = 1. / math.sqrt(D)
        q, k, v = maybe_contiguous(q), maybe_contiguous(k), maybe_contiguous(v)
        assert (eq is None) == (ek is None)
        if eq is None:
            assert score_func_mode == SCORE_FUNC_MODE0_NOPE
        # -- checks the reference leaves to the Triton launcher --
        assert score_func_mode in (SCORE_FUNC_MODE0_NOPE, SCORE_FUNC_MODE1_DOC, SCORE_FUNC_MODE2_BLOCK), "unknown score_func_mode"
        window, prefix = int(window or 0), int(prefix or 0)
        assert window >= 0 and prefix >= 0 and not (window and prefix), "window and prefix exclude each other"
        assert causal or not (window or prefix), "window / prefix are causal masks"
        assert q.is_cuda and k.is_cuda and v.is_cuda, "flash_mi355 runs on the GPU only"
        _check_same_device(q, k=k, v=v)
        if score_func_mode != SCORE_FUNC_MODE2_BLOCK:   # (a block map is moved to q's device below)
            _check_same_device(q, eq=eq, ek=ek)
        assert q.dtype in _DTYPES and k.dtype == q.dtype and v.dtype == q.dtype, \
            "q, k, v must share one of torch.bfloat16 / torch.float16 / torch.float32"
        assert k.shape[0] == B and v.shape[0] == B and v.shape[2] == N
        if score_func_mode == SCORE_FUNC_MODE2_BLOCK:
            nbr, nbc = -(-M // _cabi.FA_MASK_BLOCK), -(-N // _cabi.FA_MASK_BLOCK)
            assert eq.dim() == 4 and eq.shape[0] in (1, B) and eq.shape[1] in (1, H) and tuple(eq.shape[2:]) == (nbr, nbc), \
                f"block_mask must be [bs|1, H|1, {nbr}, {nbc}] (blocks of 64 x 64)"
            eq = maybe_contiguous((eq != 0).to(torch.uint8).to(q.device)).expand(B, H, nbr, nbc)
            ek = eq
        elif score_func_mode != SCORE_FUNC_MODE0_NOPE:
            eq, ek = _prep_ids(eq, "eq"), _prep_ids(ek, "ek")
            if eq.dtype != ek.dtype:   # one id width per call
                eq, ek = eq.to(torch.int64), ek.to(torch.int64)
            assert tuple(eq.shape) == (B, H, M), "eq must be [bs, H, Lq]"
            assert tuple(ek.shape) == (B, H, N), "ek must be [bs, H, Lk]"
        else:
            eq = ek = None
            if _short_query_long_key(B, H, M, N, q.dtype):
                # Few query tiles against a long key range (decoding, the tail of a long prompt): a launch of
                # B*H*ceil(M/128) workgroups leaves most of the chip idle while each walks every key.  Rows whose
                # id is >= 0 see every key (flash_triton.py:114), and the kernels cut the key range of such rows
                # into chunks that separate workgroups process and merge: the same mask, more parallelism.
                zero = torch.zeros((1, 1, 1), dtype=torch.int32, device=q.device)   # every stride 0: one id for all
                eq, ek = zero.expand(B, H, M), zero.expand(B, H, N)
                score_func_mode = SCORE_FUNC_MODE1_DOC
        if qpos is not None:
            assert causal and score_func_mode == SCORE_FUNC_MODE1_DOC and not prefix, \
                "qpos (per-row causal positions) needs causal=True and eq / ek, and excludes prefix"
            assert qpos.dim() == 2 and qpos.shape[0] in (1, B) and qpos.shape[1] == M and not qpos.dtype.is_floating_point, \
                "qpos must be an integer tensor [bs|1, Lq]"
            _check_same_device(q, qpos=qpos)
            qpos = qpos.to(torch.int32).contiguous()
        ctx.nothing_to_do = B == 0 or H == 0 or M == 0 or N == 0
        if ctx.nothing_to_do:
            # No rows, or rows without a single key: nothing is launched (the C ABI refuses sizes <= 0).  A row
            # without keys gives O = 0, LSE = -inf and no gradient, as a row whose keys are all masked does.
            # (The reference launches an empty grid for Lq = 0, which its launcher refuses, and divides 0 by 0 for Lk = 0.)
            ctx.like = (q.new_empty(0), k.shape, v.shape)
            ctx.qshape = q.shape
            return torch.zeros_like(q), torch.full((B, H, M), -math.inf, device=q.device, dtype=torch.float32)
        q, k, v = _aligned(q), _aligned(k), _aligned(v)

        L = _cabi.lib()
        with torch.cuda.device(q.device):
            plan = _Plan(q, k, v, causal, sm_scale, eq, ek, score_func_mode, window, prefix, qpos)
            Out = torch.empty_like(q)   # q's layout when q is dense (flash_triton.py:539), contiguous otherwise
            lse = torch.empty((B, H, M), device=q.device, dtype=torch.float32)
            p = plan.p
            p.o, p.lse = Out.data_ptr(), lse.data_ptr()
            _set4(p.o_stride, Out)
            plan.ensure_workspace(q.device)
            _cabi.check(L.fa_fwd(ctypes.byref(p), _stream_ptr(q.device)), "fa_fwd")
        ctx.save_for_backward(q, k, v, Out, lse, eq, ek, plan.workspace, qpos)
        ctx.sm_scale = sm_scale
        ctx.causal = causal
        ctx.shapes = (B, H, M, D, N, Hk, num_groups, MN_GAP)
        ctx.score_func_info = (score_func_mode, window, prefix)
        return Out, lse

    @staticmethod
    def backward(ctx, do, dlse):
        if ctx.nothing_to_do:
            like, kshape, vshape = ctx.like
            dq = like.new_zeros(ctx.qshape)
            return dq, like.new_zeros(kshape), like.new_zeros(vshape), None, None, None, None, None, None, None, None
        q, k, v, o, lse, eq, ek, workspace, qpos = ctx.saved_tensors
        B, H, M, D, N, Hk, num_groups, MN_GAP = ctx.shapes
        score_func_mode, window, prefix = ctx.score_func_info
        L = _cabi.lib()
        if do is None:   # only LSE was used
            do = torch.zeros_like(o)
        do = _aligned(maybe_contiguous(do))
        _check_same_device(q, do=do, dlse=dlse)
        with torch.cuda.device(q.device):
            plan = _Plan(q, k, v, ctx.causal, ctx.sm_scale, eq, ek, score_func_mode, window, prefix, qpos)
            p = plan.p
            if workspace is not None:   # the forward's mask plan is used in place (flash_triton.py:557-562 saves, copies nothing)
                plan.ensure_workspace(q.device, plan_state=workspace)
            delta = torch.empty_like(lse)
            dq = torch.empty_like(q)
            # the dk/dv kernel walks the query heads of a group itself and writes the group sum
            # (the reference writes per query head and sums afterwards, flash_triton.py:594-595,635-637)
            dk = torch.empty((B, Hk, N, D), dtype=k.dtype, device=q.device)
            dv = torch.empty((B, Hk, N, D), dtype=v.dtype, device=q.device)
            p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
            p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
            _set4(p.o_stride, o); _set4(p.do_stride, do)
            _set4(p.dq_stride, dq); _set4(p.dk_stride, dk); _set4(p.dv_stride, dv)
            stream = _stream_ptr(q.device)
            if dlse is None:
                # two launches instead of the reference's three (flash_triton.py:585-634): the dq kernel
                # forms delta = rowsum(O * dO) from rows it holds anyway and leaves it for the dk/dv kernel
                p.flags = _cabi.FA_FLAG_DQ_DELTA
                _cabi.check(L.fa_bwd_dq(ctypes.byref(p), stream), "fa_bwd_dq")
                _cabi.check(L.fa_bwd_dkdv(ctypes.byref(p), stream), "fa_bwd_dkdv")
            else:
                _cabi.check(L.fa_bwd_delta(ctypes.byref(p), stream), "fa_bwd_delta")
                if dlse is not None:
                    # dS = P * (dP - delta) + dLSE * P: a gradient arriving at LSE only shifts delta
                    delta.sub_(torch.where(torch.isinf(lse), torch.zeros_like(lse), dlse.to(torch.float32)))
                _cabi.check(L.fa_bwd_dkdv(ctypes.byref(p), stream), "fa_bwd_dkdv")
                _cabi.check(L.fa_bwd_dq(ctypes.byref(p), stream), "fa_bwd_dq")
        return dq, dk, dv, None, None, None, None, None, None, None, None


_forward, _backward = _Impl.forward, _Impl.backward


class FlashAttention(torch.autograd.Function):
    """Mirror of the reference autograd function (flash_triton.py:506-638)."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, eq, ek, score_func_mode, window=0, prefix=0, qpos=None):
        return _forward(ctx, q, k, v, causal, sm_scale, eq, ek, score_func_mode, window, prefix, qpos)[0]

    @staticmethod
    def backward(ctx, do):
        return _backward(ctx, do, None)


class FlashAttentionWithLse(torch.autograd.Function):
    """Same operator returning (Out, LSE), LSE in natural-log units, both differentiable -- what a
    caller needs to merge partial attentions over key shards (no counterpart in the reference, whose
    entry point returns Out only, flash_triton.py:564)."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, eq, ek, score_func_mode, window=0, prefix=0, qpos=None):
        out, lse = _forward(ctx, q, k, v, causal, sm_scale, eq, ek, score_func_mode, window, prefix, qpos)
        ctx.set_materialize_grads(False)   # a result that is not used arrives as None, not as zeros
        return out, lse * math.log(2.0)

    @staticmethod
    def backward(ctx, do, dlse):
        return _backward(ctx, do, dlse)


def _block_args(block_mask, eq, ek, score_func_mode):
    if block_mask is None:
        return eq, ek, score_func_mode
    assert eq is None and ek is None and score_func_mode == SCORE_FUNC_MODE0_NOPE, "block_mask excludes eq / ek"
    return block_mask, block_mask, SCORE_FUNC_MODE2_BLOCK


def attention(q, k, v, causal=False, sm_scale=None, eq=None, ek=None, score_func_mode=SCORE_FUNC_MODE0_NOPE,
              *, window=0, prefix=0, block_mask=None, qpos=None):
    """flash_triton.py:640-641.  Keyword-only additions (no counterpart in the reference):
    window = W: sliding window, a row sees only its last W keys up to the diagonal (causal only);
    prefix = P: prefix-LM, the first P keys are seen by every row (causal only, excludes window);
    block_mask: block-sparse attention -- a bool / integer tensor [bs|1, H|1, ceil(Lq/64), ceil(Lk/64)];
    a (row, key) pair is kept iff its 64 x 64 block is non-zero (and the causal terms hold); blocks that
    are switched off are never visited.  Excludes eq / ek.
    qpos: per-row causal positions, an integer tensor [bs|1, Lq] -- row i has its diagonal at key
    qpos[i] (it sees keys j <= qpos[i]) instead of max(0, Lk - Lq) + i; needs causal=True and eq / ek
    (the ids confine a row to its sequence, qpos aligns each sequence on its own), excludes prefix."""
    eq, ek, score_func_mode = _block_args(block_mask, eq, ek, score_func_mode)
    return FlashAttention.apply(q, k, v, causal, sm_scale, eq, ek, score_func_mode, window, prefix, qpos)


# ---------------------------------------------------------------------------
# Accessors for tests and benchmarks (not part of the reference's surface).
# ---------------------------------------------------------------------------
def attention_with_lse(q, k, v, causal=False, sm_scale=None, eq=None, ek=None,
                       score_func_mode=SCORE_FUNC_MODE0_NOPE, *, window=0, prefix=0, block_mask=None, qpos=None):
    """(O, LSE) with LSE in natural-log units (-inf for rows without a kept key); differentiable
    through both results."""
    eq, ek, score_func_mode = _block_args(block_mask, eq, ek, score_func_mode)
    return FlashAttentionWithLse.apply(q, k, v, causal, sm_scale, eq, ek, score_func_mode, window, prefix, qpos)


def varlen_ids(cu_seqlens: torch.Tensor, total: int) -> torch.Tensor:
    """Document ids of a packed batch: token t of sequence s (cu_seqlens[s] <= t < cu_seqlens[s+1])
    gets the local id -(s+1); tokens behind the last boundary get the id of a further sequence of
    their own.  int32, shape [total]."""
    pos = torch.arange(total, device=cu_seqlens.device, dtype=cu_seqlens.dtype)
    seq = torch.bucketize(pos, cu_seqlens[1:].contiguous(), right=True)
    return (-(seq + 1)).to(torch.int32)


def varlen_positions(cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, total_q: int) -> torch.Tensor:
    """Causal positions of a packed batch whose query and key boundaries differ: every sequence is
    aligned bottom-right on its own (its last query sees its last key, flash_triton.py:521 applied per
    sequence), so packed row i of sequence s has its diagonal at packed key i + (cu_k[s+1] - cu_q[s+1]).
    A sequence with fewer keys than queries leaves its first rows without a key (positions before the
    sequence's first key; output 0).  int32, shape [total_q]; computed on the device, no host sync."""
    pos = torch.arange(total_q, device=cu_seqlens_q.device, dtype=torch.int64)
    nseq = cu_seqlens_q.numel() - 1
    seq = torch.bucketize(pos, cu_seqlens_q[1:].contiguous().to(torch.int64), right=True).clamp_(max=max(nseq - 1, 0))
    shift = (cu_seqlens_k[1:].to(torch.int64) - cu_seqlens_q[1:].to(torch.int64))[seq]
    return (pos + shift).clamp_(min=-1).to(torch.int32)


def attention_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k=None, causal=False, sm_scale=None, *, window=0):
    """Packed variable-length batch (the calling convention of varlen flash-attention kernels):
    q [total_q, H, D], k and v [total_k, Hk, D], cu_seqlens_* int tensors [S+1] of cumulative
    sequence lengths starting at 0.  Token i of sequence s attends to the keys of sequence s
    only.  Returns [total_q, H, D]; differentiable.

    The packed batch IS the document mask of the operator: one (batch) row of total_* tokens whose
    ids are the negated sequence numbers, so no padding and no copy -- q, k, v are passed as
    [1, H, total, D] views, one launch per kernel whatever the number of sequences.  Causal with
    different boundaries (queries that are the tail of a longer key sequence: chunked prefill,
    decoding) aligns every sequence bottom-right on its own, which is not one offset of the packed
    row: the rows then carry their own causal positions (varlen_positions, the qpos argument of the
    operator).  Nothing is read back to the host.
    (No counterpart in the reference, which takes eq/ek directly, flash_triton.py:506.)"""
    assert q.dim() == 3 and k.dim() == 3 and v.dim() == 3, "q, k, v must be [total, heads, D]"
    same = cu_seqlens_k is None or cu_seqlens_k is cu_seqlens_q
    Tq, H, _ = q.shape
    Tk = k.shape[0]
    # the boundaries may live on the host (the ids and positions are built on q's device either way)
    cu_seqlens_q = cu_seqlens_q.to(q.device)
    cu_seqlens_k = cu_seqlens_q if same else cu_seqlens_k.to(q.device)
    assert not same or Tk == Tq, "cu_seqlens_k is needed when k holds a different number of tokens than q"
    qpos = None
    if not same:
        assert cu_seqlens_q.shape == cu_seqlens_k.shape, "cu_seqlens_q and cu_seqlens_k must describe the same sequences"
        if causal:
            qpos = varlen_positions(cu_seqlens_q, cu_seqlens_k, Tq).view(1, Tq)
    eq = varlen_ids(cu_seqlens_q, Tq)
    ek = eq if same else varlen_ids(cu_seqlens_k, Tk)
    q4, k4, v4 = (t.transpose(0, 1).unsqueeze(0) for t in (q, k, v))
    out = attention(q4, k4, v4, causal, sm_scale, eq.view(1, 1, Tq).expand(1, H, Tq), ek.view(1, 1, Tk).expand(1, H, Tk),
                    SCORE_FUNC_MODE1_DOC, window=window, qpos=qpos)
    return out.squeeze(0).transpose(0, 1)


def mask_dump(B, H, M, N, causal, eq=None, ek=None, score_func_mode=SCORE_FUNC_MODE0_NOPE, device="cuda", window=0, prefix=0,
              qpos=None):
    """keep(i, j) as a bool tensor [B, H, M, N], evaluated by the device mask routine."""
    L = _cabi.lib()
    device = torch.device(device)
    p = _cabi.FaParams()
    p.B, p.H, p.Hk, p.M, p.N, p.D = B, H, H, M, N, 64
    p.causal = 1 if causal else 0
    p.score_mode = int(score_func_mode)
    p.window, p.prefix = int(window), int(prefix)
    p.dtype = _cabi.FA_DTYPE_BF16
    keep = []
    with torch.cuda.device(device):
        if score_func_mode == SCORE_FUNC_MODE2_BLOCK:   # eq: the block map [B|1, H|1, ceil(M/64), ceil(N/64)]
            nbr, nbc = -(-M // _cabi.FA_MASK_BLOCK), -(-N // _cabi.FA_MASK_BLOCK)
            bm = maybe_contiguous((eq != 0).to(torch.uint8).to(device)).expand(B, H, nbr, nbc)
            p.eq = bm.data_ptr()
            _set3(p.eq_stride, bm)
            keep += [bm]
        elif score_func_mode != SCORE_FUNC_MODE0_NOPE:
            eq, ek = _prep_ids(eq, "eq").to(device), _prep_ids(ek, "ek").to(device)
            if eq.dtype != ek.dtype:
                eq, ek = eq.to(torch.int64), ek.to(torch.int64)
            p.eq, p.ek = eq.data_ptr(), ek.data_ptr()
            _set3(p.eq_stride, eq); _set3(p.ek_stride, ek)
            p.id_dtype = _ID_DTYPES[eq.dtype]
            nbytes = int(L.fa_workspace_bytes(ctypes.byref(p)))
            ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
            p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
            keep += [eq, ek, ws]
            if qpos is not None:
                qpos = qpos.to(device).to(torch.int32).contiguous()
                p.qpos, p.qpos_stride = qpos.data_ptr(), (qpos.stride(0) if qpos.shape[0] > 1 else 0)
                keep += [qpos]
            _cabi.check(L.fa_mask_plan(ctypes.byref(p), _stream_ptr(device)), "fa_mask_plan")
        out = torch.empty((B, H, M, N), dtype=torch.uint8, device=device)
        _cabi.check(L.fa_mask_dump(ctypes.byref(p), out.data_ptr(), _stream_ptr(device)), "fa_mask_dump")
    return out.bool()
