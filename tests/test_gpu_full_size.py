"""The headline configurations at their full sizes.

Two kinds of checks:
* every (batch, head) at once through properties that do not depend on the size: with V = 1 every
  row that sees a key must come out as exactly one; with dO = 1 the column sums of dV over the keys
  equal the number of such rows; with all keys equal the softmax is flat over the kept keys, so
  every row of dS sums to zero against identical keys and dQ vanishes;
* selected (batch, head) slices against the CPU oracle on the same inputs (the oracle needs about
  a gigabyte per temporary at 16K x 16K, so a slice at a time), tolerances as in test_gpu_parity.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL_O = 2e-2
TOL_LSE = 1e-3


def _workload_tensors(name, seed=0):
    from flash_mi355 import workloads as W
    w = W.make_workload(name)
    dt = {"bf16": torch.bfloat16, "fp16": torch.float16}[w.dtype]
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(w.B, w.H, w.Lq, w.D, generator=g).to(dt)
    k = torch.randn(w.B, w.Hk, w.Lk, w.D, generator=g).to(dt)
    v = torch.randn(w.B, w.Hk, w.Lk, w.D, generator=g).to(dt)
    do = torch.randn(w.B, w.H, w.Lq, w.D, generator=g).to(dt)
    eq = torch.from_numpy(w.eq)[:, None, :].expand(w.B, w.H, w.Lq)
    ek = torch.from_numpy(w.ek)[:, None, :].expand(w.B, w.H, w.Lk)
    return w, q, k, v, do, eq, ek


def _live_rows(w):
    """[B, Lq] bool: rows with at least one kept key (host, from the ids)."""
    from oracle import attention_oracle as O
    live = np.zeros((w.B, w.Lq), bool)
    step = 2048
    for b in range(w.B):
        for r0 in range(0, w.Lq, step):   # the mask a block of rows at a time: it is Lq x Lk bytes
            r1 = min(w.Lq, r0 + step)
            gap = max(0, w.Lk - w.Lq)
            i = np.arange(r0, r1)[:, None]
            j = np.arange(w.Lk)[None, :]
            keep = (gap + i >= j) if w.causal else np.ones((r1 - r0, w.Lk), bool)
            e_q, e_k = w.eq[b, r0:r1, None], w.ek[b][None, :]
            keep = keep & ((e_q >= 0) | (e_q == e_k))
            live[b, r0:r1] = keep.any(axis=1)
    # the oracle's mask agrees on a small corner (guards this restatement)
    ref = O.keep_mask(w.Lq, w.Lk, w.causal, w.eq[:1, None, :], w.ek[:1, None, :], 1)[0, 0, :64]
    assert np.array_equal(ref.any(axis=1), live[0, :64])
    return torch.from_numpy(live)


@pytest.mark.parametrize("name", ["cfg4_doc_causal_16k", "cfg3_doc_causal_4k", "cfg5_rect_fp16"])
def test_size_independent_properties(name):
    from flash_mi355 import attention, SCORE_FUNC_MODE1_DOC
    w, q, k, v, do, eq, ek = _workload_tensors(name)
    print(f"case properties {name}", flush=True)
    live = _live_rows(w)                                   # [B, Lq]
    n_live = live.sum(dim=1).float()                       # [B]
    qd, kd = q.cuda(), k.cuda()
    eqd, ekd = eq.cuda(), ek.cuda()
    G = w.H // w.Hk

    # V = 1: every row that sees a key is a convex combination of ones; dO = 1: dV[j] = sum_i P[i, j]
    ones_v = torch.ones_like(v).cuda().requires_grad_(True)
    out = attention(qd, kd, ones_v, w.causal, None, eqd, ekd, SCORE_FUNC_MODE1_DOC)
    o = out.detach().float().cpu()
    lv = live[:, None, :, None].expand_as(o)
    assert (o[lv] - 1.0).abs().max().item() <= 2 ** -7
    assert o[~lv].abs().max().item() == 0.0 if (~lv).any() else True
    out.backward(torch.ones_like(out))
    dv = ones_v.grad.float().cpu()                          # [B, Hk, Lk, D]
    col = dv.sum(dim=2)                                     # [B, Hk, D]: sum over keys of the column sums of P
    want = (n_live * G)[:, None, None].expand_as(col)
    assert ((col - want).abs() / want.clamp(min=1)).max().item() <= 5e-3

    # all keys equal: flat softmax over the kept keys -> dS rows vanish -> dQ = 0, and O = mean of kept V
    k_const = k[:, :, :1, :].expand_as(k).contiguous().cuda()
    qg = qd.clone().requires_grad_(True)
    vd = v.cuda()
    out2 = attention(qg, k_const, vd, w.causal, None, eqd, ekd, SCORE_FUNC_MODE1_DOC)
    out2.backward(do.cuda())
    scale = max(1.0, do.float().abs().max().item())
    assert qg.grad.float().abs().max().item() <= 2e-2 * scale
    assert not torch.isnan(out2).any()


@pytest.mark.parametrize("name,slices", [("cfg4_doc_causal_16k", [(0, 0), (0, 21)]),
                                          ("cfg3_doc_causal_4k", [(0, 3), (1, 30)]),
                                          ("cfg5_rect_fp16", [(2, 1), (7, 6)])])
def test_slices_against_the_oracle(name, slices):
    from flash_mi355 import attention_with_lse, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    w, q, k, v, do, eq, ek = _workload_tensors(name, seed=1)
    print(f"case slices {name}", flush=True)
    G = w.H // w.Hk
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out, lse = attention_with_lse(qd, kd, vd, w.causal, None, eq.cuda(), ek.cuda(), SCORE_FUNC_MODE1_DOC)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    assert G == 1   # the configurations here are multi-head; dK / dV of a slice need no group sum
    for (b, h) in slices:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ro, rl, rdq, rdk, rdv = O.attention_autograd(q[sl], k[sl], v[sl], do[sl], w.causal, None, eq[sl], ek[sl], 1)
        dead = torch.isinf(rl)
        got_l = lse.detach()[sl].cpu()
        assert torch.equal(torch.isinf(got_l), dead)
        assert (got_l[~dead] - rl[~dead]).abs().max().item() <= TOL_LSE
        assert (out.detach()[sl].float().cpu() - ro).abs().max().item() <= TOL_O
        for nm, got, ref in (("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
            err = (got[sl].float().cpu() - ref).abs().max().item()
            assert err <= TOL_O * max(1.0, ref.abs().max().item() / 4), (name, b, h, nm, err)
