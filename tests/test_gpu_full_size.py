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

from tests._tol import check_close, worst_ratio

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


# (batch, head) slices that meet the oracle, per configuration: every one of the 64 of cfg3 and cfg5, every other head
# of cfg4 (the first and the last included; a slice of it keeps the host busy for seven seconds), in groups that each
# stay well inside a minute
SLICES = {
    "cfg4_doc_causal_16k": [(0, h) for h in (0, 31, 2, 4, 6, 8, 10, 12, 14, 16, 18, 20, 22, 24, 26, 28)],
    "cfg3_doc_causal_4k": [(b, h) for b in range(2) for h in range(32)],
    "cfg5_rect_fp16": [(b, h) for b in range(8) for h in range(8)],
}
_GROUP = {"cfg4_doc_causal_16k": 4, "cfg3_doc_causal_4k": 32, "cfg5_rect_fp16": 32}
# Per-element bound of the gradients (tests/_tol.py) times this, where the run over every slice needs it.  cfg3: its 64 slices
# hold 100 million gradient elements; a dQ or dK element is a sum over up to 4096 products of a dS that was rounded to bf16
# (flash_triton.py:306,417), and the tail of that error distribution reaches the bound of 2e-2.  Measured over the 64 slices
# (seed 1): this library has one dQ element at 1.039 of the bound (slice (0,12)) and one dK element at 1.032 ((1,16)); the CPU
# model of the reference's own storage roundings (oracle.attention_grads(store_dtype=bfloat16), result rounded too) has four
# tensors over the bound on the same inputs, the worst at 1.142 (dK of slice (0,0)): no implementation that rounds where the
# reference rounds meets the bound on every element here.  The ceilings sit just above what was measured; dV, O and LSE of
# cfg3 and everything of cfg4 and cfg5 (fp16: 0.14 of the bound at most) are held to the plain bound.
SLICE_CEILINGS = {"cfg3_doc_causal_4k": {"dq": 1.1, "dk": 1.1}}
_gpu_results = {}


def _gpu_step(name):
    """One forward + backward of the configuration on the GPU (seed 1), kept on the host for the slice groups."""
    if name not in _gpu_results:
        from flash_mi355 import attention_with_lse, SCORE_FUNC_MODE1_DOC
        _gpu_results.clear()   # one configuration's tensors at a time
        w, q, k, v, do, eq, ek = _workload_tensors(name, seed=1)
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        out, lse = attention_with_lse(qd, kd, vd, w.causal, None, eq.cuda(), ek.cuda(), SCORE_FUNC_MODE1_DOC)
        out.backward(do.cuda())
        torch.cuda.synchronize()
        _gpu_results[name] = (w, q, k, v, do, eq, ek, out.detach().cpu(), lse.detach().cpu(),
                              qd.grad.cpu(), kd.grad.cpu(), vd.grad.cpu())
    return _gpu_results[name]


@pytest.mark.parametrize("name,group", [(n, g) for n in SLICES for g in range(len(SLICES[n]) // _GROUP[n])])
def test_slices_against_the_oracle(name, group):
    from oracle import attention_oracle as O
    w, q, k, v, do, eq, ek, out, lse, dq, dk, dv = _gpu_step(name)
    slices = SLICES[name][group * _GROUP[name]:(group + 1) * _GROUP[name]]
    print(f"case slices {name} {slices}", flush=True)
    assert w.H == w.Hk   # the configurations here are multi-head; dK / dV of a slice need no group sum
    worst = {}
    for (b, h) in slices:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ro, rl, rdq, rdk, rdv = O.attention_autograd(q[sl], k[sl], v[sl], do[sl], w.causal, None, eq[sl], ek[sl], 1)
        dead = torch.isinf(rl)
        got_l = lse[sl]
        assert torch.equal(torch.isinf(got_l), dead)
        assert (got_l[~dead] - rl[~dead]).abs().max().item() <= TOL_LSE
        assert (out[sl].float() - ro).abs().max().item() <= TOL_O
        for nm, got, ref in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
            r, err, at = worst_ratio(got[sl], ref)
            worst[nm] = max(worst.get(nm, 0.0), r)
            if r > 0.9:
                print(f"  {name} slice ({b},{h}) {nm}: worst err/bound {r:.3f} (err {err:.4g} at ref {at:.4g})", flush=True)
            assert r <= SLICE_CEILINGS.get(name, {}).get(nm, 1.0), \
                f"{name} slice ({b},{h}) {nm}: error {err:.5g} at reference value {at:.5g} is {r:.3f} x the bound"
    print(f"  {name} group {group}: worst err/bound over {len(slices)} slices:", {n: round(r, 3) for n, r in worst.items()}, flush=True)


def test_cfg2_plain_every_head_against_the_oracle():
    """The plain configuration (no mask, not causal, D = 64, bf16) at its full size, every one of its
    64 (batch, head) slices against the oracle, a few heads at a time (scores are 16 MB per head)."""
    from flash_mi355 import attention_with_lse, workloads as W
    from oracle import attention_oracle as O
    w = W.make_workload("cfg2_plain")
    assert (w.B, w.H, w.Lq, w.Lk, w.D, w.dtype, w.causal, w.doc) == (4, 16, 2048, 2048, 64, "bf16", False, False)
    g = torch.Generator().manual_seed(2)
    q, k, v, do = (torch.randn(w.B, w.H, w.Lq, w.D, generator=g).to(torch.bfloat16) for _ in range(4))
    print("case cfg2_plain full size", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out, lse = attention_with_lse(qd, kd, vd, False, None)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    o, l = out.detach().float().cpu(), lse.detach().cpu()
    dq, dk, dv = (t.grad.float().cpu() for t in (qd, kd, vd))
    worst = {}
    for b in range(w.B):
        for h0 in range(0, w.H, 4):
            sl = (slice(b, b + 1), slice(h0, h0 + 4))
            ro, rl, rdq, rdk, rdv = O.attention_autograd(q[sl], k[sl], v[sl], do[sl], False, None, None, None, 0)
            assert (l[sl] - rl).abs().max().item() <= TOL_LSE
            assert (o[sl] - ro).abs().max().item() <= TOL_O
            for nm, got, ref in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
                worst[nm] = max(worst.get(nm, 0.0), check_close(f"cfg2 b{b} h{h0}..{h0 + 3} {nm}", got[sl], ref, quiet=True))
    print("  cfg2_plain worst err/bound:", {n: round(r, 3) for n, r in worst.items()}, flush=True)


def test_cfg1_fp32_doc_causal_in_full():
    """The CPU-sized configuration (fp32, B=2 H=4 L=512 D=64, causal + document mask with the ids of its
    definition: documents of 32..256 tokens, 5 % global) on the fp32 kernels, every element."""
    from flash_mi355 import attention_with_lse, workloads as W, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    w = W.make_workload("cfg1_cpu_doc_causal")
    assert (w.B, w.H, w.Lq, w.D, w.dtype, w.causal, w.doc) == (2, 4, 512, 64, "fp32", True, True)
    g = torch.Generator().manual_seed(3)
    q, k, v, do = (torch.randn(w.B, w.H, w.Lq, w.D, generator=g) for _ in range(4))
    eq = torch.from_numpy(w.eq)[:, None, :].expand(w.B, w.H, w.Lq)
    print("case cfg1_cpu_doc_causal full size", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out, lse = attention_with_lse(qd, kd, vd, True, None, eq.cuda(), eq.cuda(), SCORE_FUNC_MODE1_DOC)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    ro, rl, rdq, rdk, rdv = O.attention_autograd(q, k, v, do, True, None, eq, eq, 1)
    tol = 2e-4   # fp32 products and accumulation throughout
    assert not torch.isinf(rl).any()
    assert (lse.detach().cpu() - rl).abs().max().item() <= tol
    for nm, got, ref in (("o", out, ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        err = (got.detach().float().cpu() - ref).abs().max().item()
        assert err <= tol * max(1.0, ref.abs().max().item()), (nm, err)


def test_packed_prefill_with_per_sequence_alignment_at_16k_keys():
    """A packed causal batch at the headline key length whose sequences have more keys than queries
    (chunked prefill: the queries are the tail of every sequence), one launch per kernel: ragged
    sequence lengths, 8192 queries against 16384 keys, 8 heads over the 8 XCDs.  Properties over every
    head (V = 1 => O = 1 wherever a row exists), and three sequences -- the first, a middle one and the
    last -- against the oracle run on that sequence alone (the reference's rectangular causal case,
    flash_triton.py:520-521)."""
    from flash_mi355 import attention_varlen
    from oracle import attention_oracle as O
    rng = np.random.default_rng(5)
    S = 12
    lq = rng.multinomial(8192 - 16 * S, np.ones(S) / S) + 16
    lk = lq + (rng.multinomial(8192 - 8 * S, np.ones(S) / S) + 8)
    cq = np.concatenate([[0], np.cumsum(lq)]); ck = np.concatenate([[0], np.cumsum(lk)])
    Tq, Tk, H, D = int(cq[-1]), int(ck[-1]), 8, 128
    assert (Tq, Tk) == (8192, 16384)
    g = torch.Generator().manual_seed(6)
    q, do = (torch.randn(Tq, H, D, generator=g).to(torch.bfloat16) for _ in range(2))
    k, v = (torch.randn(Tk, H, D, generator=g).to(torch.bfloat16) for _ in range(2))
    print(f"case packed prefill lq={lq.tolist()} lk={lk.tolist()}", flush=True)
    cuq, cuk = torch.from_numpy(cq).to(torch.int32).cuda(), torch.from_numpy(ck).to(torch.int32).cuda()
    ones = attention_varlen(q.cuda(), k.cuda(), torch.ones_like(v).cuda(), cuq, cuk, causal=True)
    assert torch.equal(ones, torch.ones_like(ones))
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = attention_varlen(qd, kd, vd, cuq, cuk, causal=True)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    for s in (0, S // 2, S - 1):
        a, b, c, d = int(cq[s]), int(cq[s + 1]), int(ck[s]), int(ck[s + 1])
        sq = lambda t: t[a:b].transpose(0, 1)[None]
        sk = lambda t: t[c:d].transpose(0, 1)[None]
        ro, _, rdq, rdk, rdv = O.attention_autograd(sq(q), sk(k), sk(v), sq(do), True, None, None, None, 0)
        assert (sq(out.detach().float().cpu()) - ro).abs().max().item() <= TOL_O
        for nm, got, ref, sl in (("dq", qd.grad, rdq, sq), ("dk", kd.grad, rdk, sk), ("dv", vd.grad, rdv, sk)):
            check_close(f"sequence {s} {nm}", sl(got.float().cpu()), ref)


def test_tensors_larger_than_4_gib():
    """Every tensor of the call larger than 4 GiB (B=34, H=32, L=16384, D=128, bf16: 4.56 GB each; causal + the
    headline configuration's ids): an index that was formed in 32 bits somewhere would land in the wrong
    (batch, head).  Every head through the size-independent properties, with and without ids, evaluated on the GPU (V = 1 and
    dO = 1: O is one on every row, the column sums of dV add up to the number of rows), and four slices --
    the first, one whose offset lies past 2^31 bytes, one past 2^31 elements and the very last -- against the oracle."""
    from flash_mi355 import attention, attention_with_lse, workloads as W, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    w = W.make_workload("cfg4_doc_causal_16k")
    B, H, L, D = 34, 32, w.Lq, w.D
    assert B * H * L * D * 2 > 2 ** 32 and (L, D) == (16384, 128)
    free, _ = torch.cuda.mem_get_info()
    if free < 60 * 2 ** 30:
        pytest.skip("needs 60 GB of free device memory")
    dev = torch.device("cuda")
    print(f"case tensors of {B * H * L * D * 2 / 2 ** 30:.2f} GiB", flush=True)
    ids = torch.from_numpy(w.eq[0]).to(dev)[None, None, :].expand(B, H, L)
    g = torch.Generator(device=dev).manual_seed(11)
    q = torch.randn(B, H, L, D, device=dev, dtype=torch.bfloat16, generator=g)
    k = torch.randn(B, H, L, D, device=dev, dtype=torch.bfloat16, generator=g)

    ones_v = torch.ones(B, H, L, D, device=dev, dtype=torch.bfloat16).requires_grad_(True)
    out = attention(q, k, ones_v, True, None, ids, ids, SCORE_FUNC_MODE1_DOC)
    assert (out.detach().float() - 1.0).abs().amax().item() <= 2 ** -7   # causal with ids: every row sees itself
    out.backward(torch.ones_like(out))
    col = ones_v.grad.float().sum(dim=2)                               # [B, H, D]
    assert ((col - L).abs() / L).amax().item() <= 5e-3
    # the same without ids (the dense forms of the three kernels)
    ones_v.grad = None
    out = attention(q, k, ones_v, True, None)
    assert (out.detach().float() - 1.0).abs().amax().item() <= 2 ** -7
    out.backward(torch.ones_like(out))
    col = ones_v.grad.float().sum(dim=2)
    assert ((col - L).abs() / L).amax().item() <= 5e-3
    del out, col, ones_v
    torch.cuda.empty_cache()

    v = torch.randn(B, H, L, D, device=dev, dtype=torch.bfloat16, generator=g)
    do = torch.randn(B, H, L, D, device=dev, dtype=torch.bfloat16, generator=g)
    qd, kd, vd = (t.requires_grad_(True) for t in (q, k, v))
    out, lse = attention_with_lse(qd, kd, vd, True, None, ids, ids, SCORE_FUNC_MODE1_DOC)
    out.backward(do)
    torch.cuda.synchronize()
    eq1 = torch.from_numpy(w.eq[0])[None, None, :]
    assert (16 * H + 13) * L * D * 2 > 2 ** 31 and (32 * H + 5) * L * D > 2 ** 31
    for (b, h) in ((0, 0), (16, 13), (32, 5), (B - 1, H - 1)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        print(f"  slice ({b},{h})", flush=True)
        ro, rl, rdq, rdk, rdv = O.attention_autograd(q[sl].detach().cpu(), k[sl].detach().cpu(), v[sl].detach().cpu(), do[sl].cpu(),
                                                      True, None, eq1, eq1, 1)
        assert not torch.isinf(rl).any()
        assert (lse[sl].detach().cpu() - rl).abs().max().item() <= TOL_LSE
        assert (out[sl].detach().float().cpu() - ro).abs().max().item() <= TOL_O
        for nm, got, ref in (("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
            check_close(f"4 GiB tensors, slice ({b},{h}) {nm}", got[sl].cpu(), ref)
