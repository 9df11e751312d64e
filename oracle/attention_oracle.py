"""CPU oracle for the flexible-mask attention operator.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain numpy / torch on the CPU, the mathematics that the
reference operator implements.  It is the checker for the HIP kernels: only the
test-suite, the smoke check and the benchmark's ``cpu_baseline`` leg may import it.
Nothing in the shipped operator calls into this module.

What is restated (reference file:line):

* ``keep_mask``             -- the boolean mask: causal ``(MN_GAP + i) >= j``
                               (flash_triton.py:107,254,406; testing.py:36-41,
                               bottom-right aligned), document mode
                               ``(eq_i >= 0) | (eq_i == ek_j)`` (flash_triton.py:114,
                               279,413; README.md:16; testing.py:114), AND-ed
                               (flash_triton.py:103-116).
* ``attention_closed_form`` -- ``softmax(q k^T * scale + mask) v`` with the softmax
                               in floating point of the chosen width (testing.py:32-47)
                               plus the log-sum-exp the kernel stores
                               (flash_triton.py:133, there in log2 units).
* ``attention_grads``       -- the explicit gradient formulas the split backward
                               evaluates: delta = rowsum(O*dO) (flash_triton.py:165),
                               dV = P^T dO (:291), dP = dO V^T (:299),
                               dS = P*(dP - delta) (:301,400), dQ = scale dS K
                               (:420,425), dK = scale dS^T Q (:308,313), and the
                               grouped-query reduction (:635-637).
* ``attention_tiled``       -- the tiled online-softmax forward and the split
                               backward exactly as the reference kernels iterate
                               (flash_triton.py:94-133, 250-313, 387-425), in numpy,
                               for small shapes only.

Pinned by (see tests/test_oracle.py): brute-force integer loops for the mask,
torch.nn.functional.scaled_dot_product_attention and torch.logsumexp for the
forward, torch autograd + fp64 gradcheck for the gradients, block-diagonal and
shift invariants, and agreement between the closed form and the tiled restatement.
The reference ships no golden vectors for this path; the committed fixtures under
tests/golden were produced by this oracle and guard it against regressions only.

Rows whose every key is masked: the reference math yields NaN there
(testing.py:43-44) and the reference never tests that case; this oracle (and the
HIP operator) define O = 0, LSE = -inf and zero gradient for such rows.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

SCORE_FUNC_MODE0_NOPE = 0  # flash_triton.py:20
SCORE_FUNC_MODE1_DOC = 1   # flash_triton.py:22
SCORE_FUNC_MODE2_BLOCK = 2  # the library's block mask (no counterpart in the reference): eq = [B|1, H|1, ceil(Lq/64), ceil(Lk/64)]
MASK_BLOCK = 64
LOG2E = 1.4426950408889634


def keep_mask(Lq: int, Lk: int, causal: bool, eq=None, ek=None,
              score_func_mode: int = SCORE_FUNC_MODE0_NOPE, window: int = 0, prefix: int = 0, qpos=None) -> np.ndarray:
    """Boolean keep-mask, broadcastable to [B, H, Lq, Lk] (True = attend).

    causal: keep iff (max(0, Lk-Lq) + i) >= j     (flash_triton.py:107,521)
    doc   : keep iff eq[i] >= 0 or eq[i] == ek[j] (flash_triton.py:114)
    Two causal variants the library adds (the reference has neither; README.md:17-18 names such masks
    as its extension point), both need causal and exclude each other:
    window > 0: sliding window, additionally j > gap + i - window (a row sees its last `window` keys)
    prefix > 0: prefix-LM, the causal term becomes (gap + i >= j) or (j < prefix)
    qpos [B|1, Lq]: per-row causal positions (the library's; no counterpart in the reference): the
    diagonal of row i sits at key qpos[i] instead of gap + i, i.e. the one offset of
    flash_triton.py:521 becomes a per-row one -- what a packed batch needs when every sequence is
    bottom-right aligned on its own.  Needs causal, excludes prefix.
    """
    assert window >= 0 and prefix >= 0 and not (window and prefix)
    assert causal or not (window or prefix)
    assert qpos is None or (causal and not prefix)
    keep = np.ones((1, 1, Lq, Lk), dtype=bool)
    if causal:
        gap = max(0, Lk - Lq)
        j = np.arange(Lk, dtype=np.int64)[None, :]
        if qpos is None:
            pos = (gap + np.arange(Lq, dtype=np.int64))[None, :, None]            # [1, Lq, 1]
        else:
            pos = np.asarray(qpos).astype(np.int64).reshape(-1, Lq)[:, :, None]   # [B|1, Lq, 1]
        c = pos >= j
        if prefix:
            c = c | (j < prefix)
        if window:
            c = c & (j > pos - window)
        keep = keep & c[:, None]
    if score_func_mode == SCORE_FUNC_MODE1_DOC:
        eq = np.asarray(eq).astype(np.int64)
        ek = np.asarray(ek).astype(np.int64)
        assert eq.ndim == 3 and ek.ndim == 3
        doc = (eq[..., :, None] >= 0) | (eq[..., :, None] == ek[..., None, :])
        keep = keep & doc
    elif score_func_mode == SCORE_FUNC_MODE2_BLOCK:
        # keep iff the block (i // 64, j // 64) is switched on; eq carries the block map, ek is not used
        bm = np.asarray(eq) != 0
        assert bm.ndim == 4 and bm.shape[2] == -(-Lq // MASK_BLOCK) and bm.shape[3] == -(-Lk // MASK_BLOCK)
        i = np.arange(Lq) // MASK_BLOCK
        j = np.arange(Lk) // MASK_BLOCK
        keep = keep & bm[:, :, i[:, None], j[None, :]]
    elif score_func_mode != SCORE_FUNC_MODE0_NOPE:
        raise ValueError(f"unknown score_func_mode {score_func_mode}")
    return keep


def _expand_kv(x: torch.Tensor, H: int) -> torch.Tensor:
    """Grouped-query: q head h reads kv head h // (H // Hk) (flash_triton.py:53)."""
    Hk = x.shape[1]
    if Hk == H:
        return x
    assert H % Hk == 0
    return x.repeat_interleave(H // Hk, dim=1)


def attention_closed_form(q, k, v, causal=False, sm_scale=None, eq=None, ek=None,
                          score_func_mode=SCORE_FUNC_MODE0_NOPE,
                          dtype=torch.float32, window=0, prefix=0, qpos=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(O, LSE) with O = softmax(q k^T * scale + mask) v, LSE natural-log.

    Follows testing.py:32-47 with every operand up-cast to ``dtype`` first.
    Differentiable w.r.t. q, k, v through torch autograd.
    """
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)  # flash_triton.py:523-524
    qf, kf, vf = q.to(dtype), _expand_kv(k.to(dtype), H), _expand_kv(v.to(dtype), H)
    s = torch.matmul(qf, kf.transpose(-1, -2)) * sm_scale
    keep = torch.from_numpy(keep_mask(
        Lq, Lk, causal,
        None if eq is None else eq.detach().cpu().numpy(),
        None if ek is None else ek.detach().cpu().numpy(), score_func_mode, window, prefix,
        None if qpos is None else qpos.detach().cpu().numpy()))
    s = torch.where(keep, s, torch.full((), float("-inf"), dtype=dtype))
    lse = torch.logsumexp(s, dim=-1)                       # -inf on fully masked rows
    p = torch.exp(s - torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)[..., None])
    p = torch.where(keep, p, torch.zeros((), dtype=dtype))  # kills exp(-inf - 0) = 0 anyway
    o = torch.matmul(p, vf)
    return o, lse


def attention_grads(q, k, v, do, causal=False, sm_scale=None, eq=None, ek=None,
                    score_func_mode=SCORE_FUNC_MODE0_NOPE, dtype=torch.float64, window=0, prefix=0, store_dtype=None, qpos=None):
    """Explicit-formula (O, LSE, delta, dQ, dK, dV); dK, dV reduced over the GQA group.

    store_dtype (torch.bfloat16 / torch.float16, default None = exact): round where the reference's
    kernels round to the tensors' element type -- P before P V and P^T dO (flash_triton.py:126,291),
    O as it is stored and read back for delta (:539,165), dS before dS K and dS^T Q (:306,417).
    Everything else stays in ``dtype``.  Shows what error those storage roundings alone put into the
    gradients (an implementation that follows the reference cannot be closer to the exact gradients
    than this); with store_dtype=None the exact formulas are evaluated."""
    rnd = (lambda x: x) if store_dtype is None else (lambda x: x.to(store_dtype).to(dtype))
    B, H, Lq, D = q.shape
    Hk, Lk = k.shape[1], k.shape[2]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    with torch.no_grad():
        qf, kf, vf = q.to(dtype), _expand_kv(k.to(dtype), H), _expand_kv(v.to(dtype), H)
        dof = do.to(dtype)
        o, lse = attention_closed_form(q, k, v, causal, sm_scale, eq, ek, score_func_mode, dtype, window, prefix, qpos)
        keep = torch.from_numpy(keep_mask(
            Lq, Lk, causal,
            None if eq is None else eq.detach().cpu().numpy(),
            None if ek is None else ek.detach().cpu().numpy(), score_func_mode, window, prefix,
            None if qpos is None else qpos.detach().cpu().numpy()))
        s = torch.matmul(qf, kf.transpose(-1, -2)) * sm_scale
        lse0 = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)
        p = torch.where(keep, torch.exp(s - lse0[..., None]), torch.zeros((), dtype=dtype))
        if store_dtype is not None:
            o = rnd(torch.matmul(rnd(p), vf))                       # :126, stored :539
        delta = (o * dof).sum(-1)                                   # flash_triton.py:165
        dv = torch.matmul(rnd(p).transpose(-1, -2), dof)            # :291
        dp = torch.matmul(dof, vf.transpose(-1, -2))                # :299
        ds = rnd(p * (dp - delta[..., None]))                       # :301,306
        dq = torch.matmul(ds, kf) * sm_scale                        # :420,425
        dk = torch.matmul(ds.transpose(-1, -2), qf) * sm_scale      # :308,313
        if Hk != H:                                                 # :635-637
            G = H // Hk
            dk = dk.reshape(B, Hk, G, Lk, D).sum(2)
            dv = dv.reshape(B, Hk, G, Lk, D).sum(2)
    return o, lse, delta, dq, dk, dv


def attention_autograd(q, k, v, do, causal=False, sm_scale=None, eq=None, ek=None,
                       score_func_mode=SCORE_FUNC_MODE0_NOPE, dtype=torch.float32, window=0, prefix=0, qpos=None):
    """(O, LSE, dQ, dK, dV) via torch autograd through the closed form."""
    qd = q.detach().to(dtype).requires_grad_(True)
    kd = k.detach().to(dtype).requires_grad_(True)
    vd = v.detach().to(dtype).requires_grad_(True)
    o, lse = attention_closed_form(qd, kd, vd, causal, sm_scale, eq, ek, score_func_mode, dtype, window, prefix, qpos)
    o.backward(do.to(dtype))
    return o.detach(), lse.detach(), qd.grad, kd.grad, vd.grad


def attention_tiled(q, k, v, do, causal, sm_scale, eq, ek, score_func_mode,
                    BLOCK_M=16, BLOCK_N=16):
    """numpy fp64 restatement of the reference's tiled kernels (single kv head per q head).

    Forward: running max / sum in the exp2 domain (flash_triton.py:94-133).
    Backward: delta (:165), the dk/dv kernel looping query tiles for one key tile
    (:250-313) and the dq kernel looping key tiles for one query tile (:387-425).
    Returns (O, L2, dQ, dK, dV) with L2 the log2-domain log-sum-exp the kernel stores.
    Small shapes only (python loops).
    """
    q = np.asarray(q, np.float64); k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64); do = np.asarray(do, np.float64)
    B, H, M, D = q.shape
    N = k.shape[2]
    G = H // k.shape[1]
    gap = max(0, N - M)
    qk_scale = sm_scale * LOG2E
    doc = score_func_mode == SCORE_FUNC_MODE1_DOC
    O = np.zeros_like(q); L2 = np.zeros((B, H, M))
    dQ = np.zeros_like(q); dK = np.zeros((B, H, N, D)); dV = np.zeros((B, H, N, D))

    def tile_mask(b, h, m0, m1, n0, n1):
        i = np.arange(m0, m1)[:, None]; j = np.arange(n0, n1)[None, :]
        keep = np.ones((m1 - m0, n1 - n0), bool)
        if causal:
            keep &= (gap + i) >= j
        if doc:
            e_q = np.asarray(eq[b, h, m0:m1]).astype(np.int64)[:, None]
            e_k = np.asarray(ek[b, h, n0:n1]).astype(np.int64)[None, :]
            keep &= (e_q >= 0) | (e_q == e_k)
        return keep

    for b in range(B):
        for h in range(H):
            hk = h // G
            for m0 in range(0, M, BLOCK_M):
                m1 = min(M, m0 + BLOCK_M)
                qt = q[b, h, m0:m1] * qk_scale
                m_i = np.full(m1 - m0, -np.inf); l_i = np.zeros(m1 - m0)
                acc = np.zeros((m1 - m0, D))
                hi = min(N, gap + m1) if causal else N
                for n0 in range(0, hi, BLOCK_N):
                    n1 = min(N, n0 + BLOCK_N)
                    s = qt @ k[b, hk, n0:n1].T
                    s = np.where(tile_mask(b, h, m0, m1, n0, n1), s, -np.inf)
                    m_new = np.maximum(m_i, s.max(1))
                    m_safe = np.where(np.isinf(m_new), 0.0, m_new)
                    alpha = np.exp2(np.where(np.isinf(m_i), -np.inf, m_i - m_safe))
                    p = np.exp2(s - m_safe[:, None])
                    l_i = l_i * alpha + p.sum(1)
                    acc = acc * alpha[:, None] + p @ v[b, hk, n0:n1]
                    m_i = m_new
                dead = l_i == 0
                O[b, h, m0:m1] = np.where(dead[:, None], 0.0, acc / np.where(dead, 1.0, l_i)[:, None])
                with np.errstate(divide="ignore"):
                    L2[b, h, m0:m1] = np.where(dead, -np.inf, m_i + np.log2(np.where(dead, 1.0, l_i)))
            delta = (O[b, h] * do[b, h]).sum(-1)
            L2s = np.where(np.isinf(L2[b, h]), 0.0, L2[b, h])
            # dk/dv: one key tile resident, loop query tiles
            for n0 in range(0, N, BLOCK_N):
                n1 = min(N, n0 + BLOCK_N)
                lo = (max(n0 - gap, 0) // BLOCK_M) * BLOCK_M if causal else 0
                dk_t = np.zeros((n1 - n0, D)); dv_t = np.zeros((n1 - n0, D))
                for m0 in range(lo, M, BLOCK_M):
                    m1 = min(M, m0 + BLOCK_M)
                    s = q[b, h, m0:m1] @ k[b, hk, n0:n1].T
                    p = np.exp2(s * qk_scale - L2s[m0:m1, None])
                    p = np.where(tile_mask(b, h, m0, m1, n0, n1), p, 0.0)
                    dv_t += p.T @ do[b, h, m0:m1]
                    dp = do[b, h, m0:m1] @ v[b, hk, n0:n1].T
                    ds = p * (dp - delta[m0:m1, None])
                    dk_t += ds.T @ q[b, h, m0:m1]
                dK[b, h, n0:n1] = dk_t * sm_scale
                dV[b, h, n0:n1] = dv_t
            # dq: one query tile resident, loop key tiles
            for m0 in range(0, M, BLOCK_M):
                m1 = min(M, m0 + BLOCK_M)
                hi = min(N, gap + m1) if causal else N
                dq_t = np.zeros((m1 - m0, D))
                for n0 in range(0, hi, BLOCK_N):
                    n1 = min(N, n0 + BLOCK_N)
                    s = (q[b, h, m0:m1] * qk_scale) @ k[b, hk, n0:n1].T
                    p = np.exp2(s - L2s[m0:m1, None])
                    dp = do[b, h, m0:m1] @ v[b, hk, n0:n1].T
                    ds = p * (dp - delta[m0:m1, None])
                    ds = np.where(tile_mask(b, h, m0, m1, n0, n1), ds, 0.0)
                    dq_t += ds @ k[b, hk, n0:n1]
                dQ[b, h, m0:m1] = dq_t * sm_scale
    if G > 1:
        Hk = H // G
        dK = dK.reshape(B, Hk, G, N, D).sum(2)
        dV = dV.reshape(B, Hk, G, N, D).sum(2)
    return O, L2, dQ, dK, dV


def eager_attention_cpu(q, k, v, causal, attn_keep=None):
    """The reference's eager mask-materialising path (testing.py:32-47) on CPU tensors.

    Used for the benchmark's CPU baseline: scores in the tensors' own dtype, causal
    bias bottom-right aligned, ``where(mask)``, fp32 softmax cast back, times v.
    Differentiable; the backward is torch autograd, as in the reference.
    """
    Lq, Lk = q.size(-2), k.size(-2)
    w = q @ k.transpose(-2, -1) * (1.0 / math.sqrt(q.size(-1)))
    if causal:
        pq = torch.arange(Lq)
        pk = torch.arange(Lk) - (Lk - Lq)
        bias = torch.where(pq[:, None] >= pk[None, :], 0.0, float("-inf")).to(w.dtype)
        w = w + bias
    if attn_keep is not None:
        w = torch.where(attn_keep, w, float("-inf"))
    w = torch.softmax(w, dim=-1, dtype=torch.float32).to(v.dtype)
    return w @ v
