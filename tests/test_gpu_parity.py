"""GPU parity: the HIP operator (through the C ABI) against the CPU oracle on the
same seeded inputs.  Tolerances (bf16/fp16 inputs, fp32 oracle on the same
rounded inputs): O, dQ, dK, dV max-abs <= 2e-2; LSE max-abs <= 1e-3; mask bit-exact.
"""
import math

import numpy as np
import pytest
import torch

from tests._tol import check_close

pytestmark = pytest.mark.gpu

TOL_O = 2e-2
TOL_LSE = 1e-3


def _ids(rng, B, H, L, kind):
    from flash_mi355 import workloads as W
    if kind == "uniform":
        ids = np.stack([W.doc_ids_uniform(rng, L, 8, 96, 0.08) for _ in range(B)])
    elif kind == "allglobal":
        ids = np.zeros((B, L), np.int32)
    elif kind == "alllocal":
        ids = np.stack([W.doc_ids_uniform(rng, L, 8, 96, 0.0) for _ in range(B)])
    else:
        raise KeyError(kind)
    return ids


def _run_case(B, H, Hk, M, N, D, dtype, causal, doc, seed, ids_kind="uniform", per_head_ids=False,
              id_dtype=torch.int32, sm_scale=None, check_bwd=True, tol_o=TOL_O, tol_lse=TOL_LSE, window=0, prefix=0,
              qpos=None, ceilings=None):
    from flash_mi355 import attention, attention_with_lse, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    q = torch.randn(B, H, M, D, generator=g).to(dtype)
    k = torch.randn(B, Hk, N, D, generator=g).to(dtype)
    v = torch.randn(B, Hk, N, D, generator=g).to(dtype)
    do = torch.randn(B, H, M, D, generator=g).to(dtype)
    eq = ek = None
    mode = 0
    if doc:
        mode = SCORE_FUNC_MODE1_DOC
        if per_head_ids:
            ekn = np.stack([_ids(rng, B, H, N, ids_kind) for _ in range(H)], axis=1)  # [B,H,N]
            ek = torch.from_numpy(ekn).to(id_dtype)
        else:
            ek = torch.from_numpy(_ids(rng, B, H, N, ids_kind)).to(id_dtype)[:, None, :].expand(B, H, N)
        if N >= M:
            eq = ek[:, :, N - M:]  # queries are the last M positions (self-attention when M == N)
        else:                      # more queries than keys (only with per-row positions): ids of their own
            eq = torch.from_numpy(_ids(rng, B, H, M, ids_kind)).to(id_dtype)[:, None, :].expand(B, H, M)
    if isinstance(qpos, str):      # per-row causal positions: "random" (any order, -1 = sees nothing) or "steps" (packed sequences)
        if qpos == "random":
            qpos = rng.integers(-1, N + 4, (B, M))
        else:
            qpos = np.minimum(np.arange(M)[None] + np.cumsum(rng.random((1, M)) < 0.02, axis=1) * 37, N + 3)
        qpos = torch.from_numpy(qpos).to(torch.int32)
    print(f"case B{B} H{H}/{Hk} M{M} N{N} D{D} {dtype} causal={causal} doc={doc} seed={seed} ids={ids_kind} "
          f"window={window} prefix={prefix} qpos={None if qpos is None else tuple(qpos.shape)}", flush=True)
    qposd = None if qpos is None else qpos.cuda()

    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    eqd = eq.cuda() if eq is not None else None
    ekd = ek.cuda() if ek is not None else None
    if eqd is not None and not per_head_ids:
        eqd = eq[:, :1].contiguous().cuda().expand(B, H, M)
        ekd = ek[:, :1].contiguous().cuda().expand(B, H, N)
    out, lse = attention_with_lse(qd.detach(), kd.detach(), vd.detach(), causal, sm_scale, eqd, ekd, mode,
                                  window=window, prefix=prefix, qpos=qposd)
    torch.cuda.synchronize()
    ref_o, ref_lse, ref_dq, ref_dk, ref_dv = O.attention_autograd(q, k, v, do, causal, sm_scale, eq, ek, mode,
                                                                   window=window, prefix=prefix, qpos=qpos)
    # rows without any kept key: O = 0, LSE = -inf on both sides
    dead = torch.isinf(ref_lse)
    assert torch.equal(torch.isinf(lse.cpu()), dead)
    lse_err = (lse.cpu()[~dead] - ref_lse[~dead]).abs().max().item() if (~dead).any() else 0.0
    o_err = (out.float().cpu() - ref_o).abs().max().item()
    assert not torch.isnan(out).any()
    assert lse_err <= tol_lse, f"LSE err {lse_err}"
    assert o_err <= tol_o, f"O err {o_err}"
    if not check_bwd:
        return
    out2 = attention(qd, kd, vd, causal, sm_scale, eqd, ekd, mode, window=window, prefix=prefix, qpos=qposd)
    out2.backward(do.cuda())
    torch.cuda.synchronize()
    assert torch.equal(out2.detach(), out)
    for name, got, ref in (("dq", qd.grad, ref_dq), ("dk", kd.grad, ref_dk), ("dv", vd.grad, ref_dv)):
        assert got.shape == ref.shape, name
        assert not torch.isnan(got).any(), name
        # per element: 2e-2 where |ref| <= 4, one bf16 ulp of the reference value above (tests/_tol.py).
        # The bound is stated for N(0,1) inputs at the default scale D^-0.5.  A caller-given scale s times
        # the default sharpens the softmax, and the error that the 16-bit storage of O puts into delta (the
        # reference forms delta from the stored O too, flash_triton.py:165) reaches dQ and dK multiplied by
        # sm_scale: such stress cases get 2e-2 * s (tests/test_oracle.py::
        # test_storage_rounding_sets_the_gradient_error_floor shows the floor on the CPU).
        sharp = 1.0 if sm_scale is None else max(1.0, abs(sm_scale) * math.sqrt(D))
        check_close(name, got, ref, tol_o * sharp * (ceilings or {}).get(name, 1.0))


CASES = [
    # B, H, Hk, M, N, D, dtype, causal, doc
    (1, 2, 2, 128, 128, 128, torch.bfloat16, False, False),
    (1, 2, 2, 256, 256, 128, torch.bfloat16, True, False),
    (2, 2, 2, 256, 256, 128, torch.bfloat16, True, True),
    (1, 2, 2, 384, 384, 64, torch.bfloat16, True, True),
    (1, 2, 2, 256, 256, 64, torch.float16, False, True),
    (1, 4, 2, 256, 256, 128, torch.bfloat16, True, True),      # grouped-query
    (1, 2, 2, 128, 512, 128, torch.float16, True, True),       # rectangular, bottom-right causal
    (1, 2, 2, 200, 200, 128, torch.bfloat16, True, True),      # ragged lengths
    (1, 2, 2, 77, 333, 64, torch.bfloat16, True, True),        # ragged + rectangular
    (1, 2, 2, 256, 256, 32, torch.bfloat16, True, True),
    (1, 1, 1, 1024, 1024, 128, torch.bfloat16, True, True),
    (1, 2, 2, 256, 256, 16, torch.bfloat16, True, True),
    (2, 2, 1, 100, 300, 16, torch.float16, True, True),
    (1, 2, 2, 192, 192, 64, torch.bfloat16, False, False),
    (1, 1, 1, 2048, 2048, 128, torch.bfloat16, False, False),  # long tile stream: the 128-key dk/dv form without ids
    (1, 2, 1, 2100, 4300, 128, torch.float16, True, False),    # the same under a causal mask, grouped and ragged
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d-H%d_%d-M%d-N%d-D%d-%s-c%d-d%d" % (
    c[0], c[1], c[2], c[3], c[4], c[5], str(c[6]).split(".")[-1], c[7], c[8]))
def test_fwd_bwd_parity(case):
    _run_case(*case, seed=1234)


QPOS_CASES = [
    # B, H, Hk, M, N, D, dtype, window, positions, ids
    (1, 2, 2, 300, 300, 128, torch.bfloat16, 0, "random", "uniform"),
    (2, 2, 1, 200, 520, 64, torch.float16, 0, "random", "uniform"),
    (1, 2, 2, 333, 77, 128, torch.bfloat16, 0, "random", "uniform"),     # more queries than keys
    (1, 2, 2, 700, 900, 128, torch.bfloat16, 0, "steps", "uniform"),
    (1, 2, 2, 700, 900, 64, torch.bfloat16, 40, "steps", "alllocal"),    # with a sliding window
    (1, 1, 1, 260, 2200, 128, torch.bfloat16, 0, "random", "allglobal"), # split key ranges of global rows
    (1, 2, 2, 130, 190, 16, torch.bfloat16, 7, "random", "uniform"),
    (1, 2, 2, 257, 257, 32, torch.float16, 0, "steps", "uniform"),
]


@pytest.mark.parametrize("case", QPOS_CASES, ids=lambda c: "M%d-N%d-D%d-w%d-%s-%s" % (c[3], c[4], c[5], c[7], c[8], c[9]))
def test_per_row_causal_positions(case):
    """qpos: every row carries the key position of its own diagonal (arbitrary order, -1 = the row sees
    nothing, more queries than keys allowed); forward, LSE and all gradients against the oracle."""
    B, H, Hk, M, N, D, dtype, window, kind, ids = case
    _run_case(B, H, Hk, M, N, D, dtype, True, True, seed=4321 + M, ids_kind=ids, window=window, qpos=kind)


def test_per_row_positions_mask_bit_exact():
    from flash_mi355 import mask_dump, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    rng = np.random.default_rng(11)
    for (B, H, M, N, window) in [(2, 2, 200, 260, 0), (1, 3, 150, 90, 0), (2, 1, 129, 129, 9)]:
        ek = torch.from_numpy(np.stack([_ids(rng, B, H, N, "uniform") for _ in range(H)], axis=1))
        eq = torch.from_numpy(np.stack([_ids(rng, B, H, M, "uniform") for _ in range(H)], axis=1))
        for pos in (rng.integers(-3, N + 4, (B, M)), rng.integers(-1, N, (1, M))):
            got = mask_dump(B, H, M, N, True, eq.cuda(), ek.cuda(), SCORE_FUNC_MODE1_DOC, window=window,
                            qpos=torch.from_numpy(pos).cuda()).cpu().numpy()
            ref = np.broadcast_to(O.keep_mask(M, N, True, eq.numpy(), ek.numpy(), 1, window=window, qpos=np.maximum(pos, -1)), (B, H, M, N))
            assert np.array_equal(got, ref)


def test_mask_bit_exact():
    from flash_mi355 import mask_dump, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    rng = np.random.default_rng(7)
    for (B, H, M, N, causal) in [(2, 3, 200, 200, True), (1, 2, 77, 333, True), (1, 2, 130, 64, False)]:
        ek = torch.from_numpy(np.stack([_ids(rng, B, H, N, "uniform") for _ in range(H)], axis=1))
        eq = torch.from_numpy(np.stack([_ids(rng, B, H, M, "uniform") for _ in range(H)], axis=1))
        for idt in (torch.int32, torch.int64):
            got = mask_dump(B, H, M, N, causal, eq.to(idt).cuda(), ek.to(idt).cuda(), SCORE_FUNC_MODE1_DOC).cpu().numpy()
            ref = np.broadcast_to(O.keep_mask(M, N, causal, eq.numpy(), ek.numpy(), 1), (B, H, M, N))
            assert np.array_equal(got, ref)
        got = mask_dump(B, H, M, N, causal).cpu().numpy()
        ref = np.broadcast_to(O.keep_mask(M, N, causal), (B, H, M, N))
        assert np.array_equal(got, ref)


BLOCK_CASES = [
    # B, H, Hk, M, N, D, dtype, causal, window, density, broadcast (block map shared by batch and heads)
    (1, 2, 2, 512, 512, 128, torch.bfloat16, False, 0, 0.5, False),
    (2, 2, 2, 512, 512, 128, torch.bfloat16, True, 0, 0.5, False),
    (1, 4, 2, 450, 700, 128, torch.float16, True, 0, 0.6, False),     # grouped (a map per query head), ragged, rectangular
    (2, 4, 1, 260, 260, 64, torch.bfloat16, False, 0, 0.5, True),      # grouped, one map for everything
    (1, 2, 2, 300, 300, 64, torch.bfloat16, True, 0, 0.4, False),
    (1, 2, 1, 333, 520, 64, torch.float16, False, 0, 0.3, True),
    (1, 2, 2, 200, 200, 16, torch.bfloat16, True, 0, 0.5, False),
    (1, 2, 2, 640, 640, 32, torch.bfloat16, False, 0, 0.2, False),
    (1, 1, 1, 2304, 2304, 128, torch.bfloat16, True, 0, 0.3, False),   # long stream: the 128-key dk/dv form
    (1, 2, 2, 1024, 1024, 128, torch.bfloat16, True, 300, 0.7, False),  # with a sliding window
    (1, 2, 2, 192, 192, 128, torch.bfloat16, False, 0, 0.0, False),    # nothing kept at all
    (1, 2, 2, 300, 300, 64, torch.float32, True, 0, 0.5, False),       # the fp32 kernels
    (1, 4, 2, 200, 520, 128, torch.float32, False, 0, 0.4, True),
    (2, 2, 1, 450, 450, 32, torch.float32, True, 100, 0.6, False),
]


@pytest.mark.parametrize("case", BLOCK_CASES, ids=lambda c: "blk-B%d-H%d_%d-M%d-N%d-D%d-c%d-w%d" % (
    c[0], c[1], c[2], c[3], c[4], c[5], c[7], c[8]))
def test_block_mask_parity(case):
    """Block-sparse attention (64 x 64 blocks switched on and off by a byte map): mask bit-exact, O, LSE
    and the gradients against the oracle; rows whose blocks are all off give O = 0, LSE = -inf, no gradient."""
    from flash_mi355 import attention_with_lse, attention, mask_dump, SCORE_FUNC_MODE2_BLOCK
    from oracle import attention_oracle as O
    B, H, Hk, M, N, D, dtype, causal, window, density, shared = case
    rng = np.random.default_rng(M * 7 + N + D)
    g = torch.Generator().manual_seed(M + N + D)
    nbr, nbc = -(-M // 64), -(-N // 64)
    bm = torch.from_numpy((rng.random((1 if shared else B, 1 if shared else H, nbr, nbc)) < density))
    if density > 0:
        bm[..., 0, :] = False          # a row of blocks with nothing kept
    q = torch.randn(B, H, M, D, generator=g).to(dtype)
    k = torch.randn(B, Hk, N, D, generator=g).to(dtype)
    v = torch.randn(B, Hk, N, D, generator=g).to(dtype)
    do = torch.randn(B, H, M, D, generator=g).to(dtype)
    print(f"case block mask {case}", flush=True)
    keep = mask_dump(B, H, M, N, causal, bm.cuda(), None, SCORE_FUNC_MODE2_BLOCK, window=window).cpu().numpy()
    ref_keep = np.broadcast_to(O.keep_mask(M, N, causal, bm.numpy(), None, 2, window=window), (B, H, M, N))
    assert np.array_equal(keep, ref_keep)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    with torch.no_grad():
        out, lse = attention_with_lse(qd, kd, vd, causal, None, window=window, block_mask=bm.cuda())
    ref_o, ref_lse, ref_dq, ref_dk, ref_dv = O.attention_autograd(q, k, v, do, causal, None, bm, None, 2, window=window)
    tol_o, tol_lse = (TOL_F32, TOL_F32) if dtype == torch.float32 else (TOL_O, TOL_LSE)
    dead = torch.isinf(ref_lse)
    assert torch.equal(torch.isinf(lse.cpu()), dead)
    if (~dead).any():
        assert (lse.cpu()[~dead] - ref_lse[~dead]).abs().max().item() <= tol_lse
    assert not torch.isnan(out).any()
    assert (out.float().cpu() - ref_o).abs().max().item() <= tol_o
    out2 = attention(qd, kd, vd, causal, None, window=window, block_mask=bm.cuda())
    out2.backward(do.cuda())
    torch.cuda.synchronize()
    assert torch.equal(out2.detach(), out)
    for name, got, ref in (("dq", qd.grad, ref_dq), ("dk", kd.grad, ref_dk), ("dv", vd.grad, ref_dv)):
        assert not torch.isnan(got).any(), name
        if dtype == torch.float32:
            err = (got.float().cpu() - ref).abs().max().item()
            assert err <= tol_o * max(1.0, ref.abs().max().item()), f"{name} err {err}"
        else:
            check_close(name, got, ref, tol_o)


def test_all_global_and_all_local_ids():
    _run_case(1, 2, 2, 256, 256, 128, torch.bfloat16, True, True, seed=5, ids_kind="allglobal")
    _run_case(1, 2, 2, 256, 256, 128, torch.bfloat16, True, True, seed=6, ids_kind="alllocal")


def test_long_key_ranges_of_global_rows():
    # Rows with id >= 0 see long key ranges; tiles of such rows are cut into key chunks that
    # separate workgroups process and merge.  Covers 2 and 4 chunks, causal and not, a ragged
    # last key tile, and more global-row tiles than the number that is ever cut.
    _run_case(1, 2, 2, 4096, 4096, 64, torch.bfloat16, True, True, seed=21)
    _run_case(1, 2, 1, 300, 5000, 128, torch.float16, False, True, seed=22)
    _run_case(1, 1, 1, 1200, 2304, 128, torch.bfloat16, True, True, seed=23, ids_kind="allglobal")
    _run_case(2, 2, 2, 2048, 2048, 16, torch.bfloat16, True, True, seed=24)
    # few query tiles in the launch: up to 16 chunks.  6 chunks (merged eight at a time) and 12 (merged one by one)
    _run_case(1, 2, 2, 150, 6500, 128, torch.bfloat16, True, True, seed=25, ids_kind="allglobal")
    _run_case(1, 2, 1, 64, 13000, 64, torch.float16, False, True, seed=26)


def test_short_query_long_key_without_ids():
    """Few query rows against a long key range and no ids: the operator hands the call to the kernels as
    all-global rows, whose key range is cut into chunks for separate workgroups (up to 16 here)."""
    from flash_mi355 import api
    assert api._short_query_long_key(1, 2, 100, 8300, torch.bfloat16) and not api._short_query_long_key(1, 2, 100, 8300, torch.float32)
    _run_case(1, 2, 1, 100, 8300, 128, torch.bfloat16, True, False, seed=61)
    _run_case(1, 4, 2, 1, 9000, 64, torch.float16, False, False, seed=62)
    _run_case(2, 2, 2, 300, 16500, 32, torch.bfloat16, True, False, seed=63, window=5000)


def test_transposed_views_and_strided_gradients():
    """q, k, v, dO given as [B, L, H, D] storage viewed as [B, H, L, D] (cf. testing.py:59-66): the kernels
    take element strides, nothing is copied on the way in."""
    from flash_mi355 import attention, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    B, H, L, D = 2, 3, 320, 64
    g = torch.Generator().manual_seed(77)
    rng = np.random.default_rng(77)
    base = [torch.randn(B, L, H, D, generator=g).bfloat16() for _ in range(4)]
    q, k, v, do = (t.transpose(1, 2) for t in base)
    ek = torch.from_numpy(_ids(rng, B, H, L, "uniform"))[:, None, :].expand(B, H, L)
    print("case transposed views", flush=True)
    qd, kd, vd = (t.cuda().transpose(1, 2).requires_grad_(True) for t in base[:3])
    assert not qd.is_contiguous() and qd.stride(-1) == 1
    out = attention(qd, kd, vd, True, None, ek.cuda(), ek.cuda(), SCORE_FUNC_MODE1_DOC)
    out.backward(base[3].cuda().transpose(1, 2))
    ref = O.attention_autograd(q, k, v, do, True, None, ek, ek, 1)
    for name, got, want in (("o", out, ref[0]), ("dq", qd.grad, ref[2]), ("dk", kd.grad, ref[3]), ("dv", vd.grad, ref[4])):
        check_close(name, got, want)


def test_lse_output_is_differentiable():
    """loss = <O, dO> + <LSE, w>: the gradient that arrives at LSE only shifts delta in the backward."""
    from flash_mi355 import attention_with_lse, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    B, H, L, D = 1, 2, 320, 64
    g = torch.Generator().manual_seed(31)
    rng = np.random.default_rng(31)
    q, k, v, do = (torch.randn(B, H, L, D, generator=g).bfloat16() for _ in range(4))
    w = torch.randn(B, H, L, generator=g)
    ek = torch.from_numpy(_ids(rng, B, H, L, "uniform"))[:, None, :].expand(B, H, L)
    print("case differentiable lse", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out, lse = attention_with_lse(qd, kd, vd, True, None, ek.cuda(), ek.cuda(), SCORE_FUNC_MODE1_DOC)
    ((out.float() * do.cuda().float()).sum() + (lse * w.cuda()).sum()).backward()
    qr, kr, vr = (t.float().requires_grad_(True) for t in (q, k, v))
    ro, rl = O.attention_closed_form(qr, kr, vr, True, None, ek, ek, 1)
    ((ro * do.float()).sum() + (rl * w).sum()).backward()
    assert (lse.detach().cpu() - rl.detach()).abs().max().item() <= TOL_LSE
    for name, got, want in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        check_close(name, got, want)


@pytest.mark.parametrize("use", ["out", "lse"])
def test_lse_entry_point_with_one_result_used(use):
    """Only one of (O, LSE) enters the loss: the other one's gradient arrives as None."""
    from flash_mi355 import attention_with_lse
    from oracle import attention_oracle as O
    B, H, L, D = 1, 2, 200, 64
    g = torch.Generator().manual_seed(37)
    q, k, v, do = (torch.randn(B, H, L, D, generator=g).to(torch.float16) for _ in range(4))
    w = torch.randn(B, H, L, generator=g)
    print("case lse entry point, used:", use, flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out, lse = attention_with_lse(qd, kd, vd, True)
    loss = (out.float() * do.cuda().float()).sum() if use == "out" else (lse * w.cuda()).sum()
    loss.backward()
    qr, kr, vr = (t.float().requires_grad_(True) for t in (q, k, v))
    ro, rl = O.attention_closed_form(qr, kr, vr, True, None, None, None, 0)
    ((ro * do.float()).sum() if use == "out" else (rl * w).sum()).backward()
    for name, got, want in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        want = torch.zeros_like(got, dtype=torch.float32, device="cpu") if want is None else want   # LSE does not depend on v
        check_close(name, got, want)


@pytest.mark.parametrize("seed", list(range(100, 124)))
def test_random_shapes(seed):
    """Seeded draws over the whole argument space of the operator: head size, head counts and groups,
    ragged and rectangular lengths (down to a single row), causal or not, ids or not, id layouts."""
    rng = np.random.default_rng(seed)
    D = int(rng.choice([16, 32, 64, 128]))
    Hk = int(rng.choice([1, 2, 3]))
    H = Hk * int(rng.choice([1, 2, 4]))
    B = int(rng.choice([1, 2]))
    causal = bool(rng.integers(0, 2))
    doc = bool(rng.integers(0, 4) > 0)
    M = int(rng.integers(1, 420))
    N = int(rng.integers(M, 640)) if (causal or rng.integers(0, 2)) else int(rng.integers(1, 640))
    if doc and rng.integers(0, 2):
        N = M   # self-attention with one id vector is the common case
    if doc and N < M:
        N = M   # the helper takes the query ids from the tail of the key ids
    dtype = torch.bfloat16 if rng.integers(0, 2) else torch.float16
    kind = str(rng.choice(["uniform", "uniform", "alllocal", "allglobal"]))
    per_head = bool(doc and rng.integers(0, 3) == 0)
    idt = torch.int64 if rng.integers(0, 2) else torch.int32
    _run_case(B, H, Hk, M, N, D, dtype, causal, doc, seed=seed, ids_kind=kind, per_head_ids=per_head, id_dtype=idt)


def test_clock_stamp_build_gives_the_same_bits():
    """The measurement build (the same sources with -DFA_TRACE, what `bench.py --wg-trace` loads) must time the
    kernels the product runs: its forward, dq and dk/dv results equal the product library's bit for bit."""
    import ctypes
    from flash_mi355 import _cabi
    from flash_mi355.api import _Plan, _set4, _stream_ptr
    from flash_mi355.build import TRACE_LIB_PATH
    T = ctypes.CDLL(str(TRACE_LIB_PATH))
    L = _cabi.lib()
    B, H, M, D = 1, 2, 2304, 128
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(91)
    rng = np.random.default_rng(91)
    ids = torch.from_numpy(_ids(rng, B, H, M, "uniform")).to(dev)[:, None, :].expand(B, H, M)
    q, k, v, do = (torch.randn(B, H, M, D, generator=g).bfloat16().to(dev) for _ in range(4))
    results = []
    for lib in (L, T):
        o, dq, dk, dv = (torch.full_like(q, float("nan")) for _ in range(4))
        lse = torch.empty(B, H, M, device=dev, dtype=torch.float32)
        delta = torch.empty_like(lse)
        plan = _Plan(q, k, v, True, 1.0 / math.sqrt(D), ids, ids, 1)
        p = plan.p
        p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
        p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
        for f, t in (("o_stride", o), ("do_stride", do), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
            _set4(getattr(p, f), t)
        plan.ensure_workspace(dev)
        p.flags = _cabi.FA_FLAG_DQ_DELTA
        ref, stream = ctypes.byref(p), _stream_ptr(dev)
        for name in ("fa_mask_plan", "fa_fwd", "fa_bwd_dq", "fa_bwd_dkdv"):
            fn = getattr(lib, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.POINTER(_cabi.FaParams), ctypes.c_void_p]
            assert fn(ref, stream) == 0, name
        torch.cuda.synchronize()
        results.append((o, lse, dq, dk, dv))
    for a_, b_ in zip(*results):
        assert not torch.isnan(a_).any() and torch.equal(a_, b_)


def test_empty_inputs():
    """No query rows, no batch, or no keys at all: nothing is launched; O has q's shape (zeros where there are
    rows: a row without keys behaves as a row whose keys are all masked, O = 0 and LSE = -inf) and the
    gradients are zeros of the operands' shapes.  (The reference cannot run these: its launcher refuses the
    empty grid and its kernel divides 0 by 0 without keys.)"""
    from flash_mi355 import attention, attention_with_lse, SCORE_FUNC_MODE1_DOC
    dev = torch.device("cuda")
    for (B, H, Hk, M, N, causal, doc) in ((1, 2, 2, 0, 64, False, False), (0, 2, 1, 32, 32, True, True),
                                          (2, 4, 2, 48, 0, False, True), (1, 2, 2, 0, 0, True, False)):
        q = torch.randn(B, H, M, 64, device=dev).bfloat16().requires_grad_(True)
        k = torch.randn(B, Hk, N, 64, device=dev).bfloat16().requires_grad_(True)
        v = torch.randn(B, Hk, N, 64, device=dev).bfloat16().requires_grad_(True)
        eq = torch.zeros(B, H, M, dtype=torch.int32, device=dev) - 1 if doc else None
        ek = torch.zeros(B, H, N, dtype=torch.int32, device=dev) - 1 if doc else None
        out, lse = attention_with_lse(q, k, v, causal, None, eq, ek, SCORE_FUNC_MODE1_DOC if doc else 0)
        assert out.shape == q.shape and out.dtype == q.dtype and lse.shape == (B, H, M)
        assert out.abs().sum().item() == 0 and bool(torch.isinf(lse).all())
        (out.float().sum() + 0 * lse.nan_to_num(neginf=0.0).sum()).backward()
        for t in (q, k, v):
            assert t.grad is not None and t.grad.shape == t.shape and t.grad.abs().sum().item() == 0
        q.grad = None
        attention(q, k, v, causal, None, eq, ek, SCORE_FUNC_MODE1_DOC if doc else 0).sum().backward()
        assert q.grad.shape == q.shape


def test_negative_and_large_scale():
    """sm_scale < 0 (the sign moves into Q so that the running maximum stays a maximum) and a large
    scale (sharp softmax: the lazily moved reference point has to move often)."""
    _run_case(1, 2, 2, 320, 320, 64, torch.bfloat16, True, True, seed=51, sm_scale=-0.2)
    _run_case(1, 2, 2, 320, 320, 128, torch.float16, False, False, seed=52, sm_scale=-0.09)
    _run_case(1, 2, 2, 384, 384, 128, torch.bfloat16, True, True, seed=53, sm_scale=0.25)
    _run_case(1, 2, 1, 256, 2304, 64, torch.bfloat16, True, True, seed=54, sm_scale=0.3)   # split tiles + sharp softmax


def _stress_inputs(kind, B, H, M, N, D, g):
    """Inputs that push the online softmax: scores that grow or fall along the keys, outliers, a large
    common offset, single dominating keys, tiny scores, one large score at the end of every key tile."""
    q = torch.randn(B, H, M, D, generator=g)
    k = torch.randn(B, H, N, D, generator=g)
    if kind == "ramp_up":
        q[..., 0] = 4.0
        k[..., 0] = torch.linspace(-12, 12, N)[None, None]
    elif kind == "ramp_down":
        q[..., 0] = 4.0
        k[..., 0] = torch.linspace(12, -12, N)[None, None]
    elif kind == "outliers":
        q = torch.where(torch.rand(q.shape, generator=g) < 0.01, q * 20, q)
        k = torch.where(torch.rand(k.shape, generator=g) < 0.01, k * 20, k)
    elif kind == "offset":
        q, k = q + 3.0, k + 3.0
    elif kind == "peaked":
        k[:, :, ::97] *= 8.0
    elif kind == "tiny":
        q, k = q * 1e-3, k * 1e-3
    elif kind == "saw":
        q[..., 0] = 3.0
        k[..., 0] = (torch.arange(N) % 64 == 63).float()[None, None] * 30.0
    else:
        raise KeyError(kind)
    return q, k


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("kind", ["ramp_up", "ramp_down", "outliers", "offset", "peaked", "tiny", "saw"])
def test_score_distributions_that_stress_the_online_softmax(kind, dtype):
    """The reference point of the softmax moves lazily (only when a partial row sum leaves its bound), so
    inputs that are not N(0,1) matter: no NaN, rows without keys agree, O and LSE inside the usual bounds.
    The gradient bound of tests/_tol.py is stated for N(0,1) inputs; dQ = scale dS K and dK = scale dS^T Q
    carry the error floor of dS (set by the 16-bit storage of O and P) times the size of K and Q, so here the
    bound is scaled by the largest |q|, |k| element (dV: by 2, its P^T dO sums run over rows that all point at one key)."""
    from flash_mi355 import attention, attention_with_lse, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    from tests._tol import worst_ratio
    for (B, H, M, N, D, causal, doc) in ((1, 2, 384, 384, 128, True, True), (1, 2, 300, 1100, 64, True, False),
                                         (1, 1, 256, 2304, 128, False, True), (1, 2, 520, 520, 32, True, True)):
        g = torch.Generator().manual_seed(7)
        rng = np.random.default_rng(7)
        q, k = (t.to(dtype) for t in _stress_inputs(kind, B, H, M, N, D, g))
        v = torch.randn(B, H, N, D, generator=g).to(dtype)
        do = torch.randn(B, H, M, D, generator=g).to(dtype)
        eq = ek = None
        mode = 0
        if doc:
            mode = SCORE_FUNC_MODE1_DOC
            ek = torch.from_numpy(_ids(rng, B, H, N, "uniform"))[:, None, :].expand(B, H, N)
            eq = ek[:, :, N - M:]
        print(f"case {kind} {dtype} M{M} N{N} D{D} causal={causal} doc={doc}", flush=True)
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        eqd, ekd = (eq.cuda(), ek.cuda()) if doc else (None, None)
        out, lse = attention_with_lse(qd.detach(), kd.detach(), vd.detach(), causal, None, eqd, ekd, mode)
        attention(qd, kd, vd, causal, None, eqd, ekd, mode).backward(do.cuda())
        torch.cuda.synchronize()
        ref_o, ref_lse, ref_dq, ref_dk, ref_dv = O.attention_autograd(q, k, v, do, causal, None, eq, ek, mode)
        dead = torch.isinf(ref_lse)
        assert torch.equal(torch.isinf(lse.cpu()), dead)
        assert (out.float().cpu() - ref_o).abs().max().item() <= TOL_O
        rel = (lse.cpu()[~dead] - ref_lse[~dead]).abs() / ref_lse[~dead].abs().clamp(min=1.0)
        assert rel.max().item() <= TOL_LSE
        size = max(1.0, q.float().abs().max().item(), k.float().abs().max().item())
        for name, got, ref, factor in (("dq", qd.grad, ref_dq, size), ("dk", kd.grad, ref_dk, size), ("dv", vd.grad, ref_dv, 2.0)):
            assert not torch.isnan(got).any(), name
            r, err, at = worst_ratio(got, ref)
            print(f"  {name}: worst err/bound {r:.3f} of {factor:.1f} allowed (err {err:.4g} at ref {at:.4g})", flush=True)
            assert r <= factor, f"{name}: error {err:.5g} at reference value {at:.5g}"


@pytest.mark.parametrize("dq_forms_delta", [False, True])
def test_graph_capture_and_replay(dq_forms_delta):
    """The calls of a step (plan, forward, delta, dk/dv, dq -- or plan, forward, dq forming delta, dk/dv)
    captured into one HIP graph: every
    replay, with new inputs copied into the captured buffers and eager work in between, must give the
    eager result bit for bit (the library allocates nothing and clears its counters with kernels)."""
    import ctypes
    from flash_mi355 import _cabi
    from flash_mi355.api import _Plan, _set4, _stream_ptr
    L = _cabi.lib()
    B, H, M, D = 1, 4, 2304, 64          # long enough for split key ranges (36 key tiles)
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(41)
    rng = np.random.default_rng(41)
    ids = torch.from_numpy(_ids(rng, B, H, M, "uniform")).to(dev)[:, None, :].expand(B, H, M)
    q, k, v, do = (torch.randn(B, H, M, D, generator=g).bfloat16().to(dev) for _ in range(4))
    o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    lse = torch.empty(B, H, M, device=dev, dtype=torch.float32)
    delta = torch.empty_like(lse)
    plan = _Plan(q, k, v, True, 1.0 / math.sqrt(D), ids, ids, 1)
    p = plan.p
    p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
    p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    for f, t in (("o_stride", o), ("do_stride", do), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
        _set4(getattr(p, f), t)
    nbytes = int(L.fa_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
    ref = ctypes.byref(p)

    if dq_forms_delta:
        p.flags = _cabi.FA_FLAG_DQ_DELTA
    calls = ("fa_mask_plan", "fa_fwd", "fa_bwd_dq", "fa_bwd_dkdv") if dq_forms_delta else \
            ("fa_mask_plan", "fa_fwd", "fa_bwd_delta", "fa_bwd_dkdv", "fa_bwd_dq")

    def step():
        s = _stream_ptr(dev)
        for name in calls:
            _cabi.check(getattr(L, name)(ref, s), name)

    print("case graph capture, dq forms delta:", dq_forms_delta, flush=True)
    step()                       # eager once: kernel attributes are set outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for t in (q, k, v, do):
            t.copy_(torch.randn(B, H, M, D, generator=g).bfloat16())
        step()
        torch.cuda.synchronize()
        want = [t.clone() for t in (o, lse, dq, dk, dv)]
        for t in (o, lse, dq, dk, dv):
            t.zero_()
        _ = (q.float() @ k.float().transpose(-1, -2)).sum().item()   # unrelated eager work and a sync in between
        graph.replay()
        torch.cuda.synchronize()
        for name, got, w_ in zip(("o", "lse", "dq", "dk", "dv"), (o, lse, dq, dk, dv), want):
            assert torch.equal(got, w_), (rep, name)


@pytest.mark.parametrize("M,D,doc,dtype", [(2304, 64, True, torch.bfloat16), (450, 128, False, torch.float16),
                                           (1000, 128, True, torch.bfloat16), (333, 16, True, torch.float16),
                                           (450, 64, True, torch.float32), (300, 128, False, torch.float32)])
def test_dq_computes_delta(M, D, doc, dtype):
    """FA_FLAG_DQ_DELTA: fa_bwd_dq forms delta itself and leaves it for fa_bwd_dkdv; delta, dq, dk, dv
    must agree with the three-launch sequence (delta is a sum of the same products in another order:
    1e-5 relative; the gradients then differ by a rounding of the 16-bit outputs at most)."""
    import ctypes
    from flash_mi355 import _cabi
    from flash_mi355.api import _Plan, _set4, _stream_ptr
    L = _cabi.lib()
    B, H = 2, 4
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(M + D)
    rng = np.random.default_rng(M + D)
    ids = torch.from_numpy(_ids(rng, B, H, M, "uniform")).to(dev)[:, None, :].expand(B, H, M) if doc else None
    q, k, v, do = (torch.randn(B, H, M, D, generator=g).to(dtype).to(dev) for _ in range(4))
    o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    lse = torch.empty(B, H, M, device=dev, dtype=torch.float32)
    delta = torch.empty_like(lse)
    plan = _Plan(q, k, v, True, 1.0 / math.sqrt(D), ids, ids, 1 if doc else 0)
    p = plan.p
    p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
    p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    for f, t in (("o_stride", o), ("do_stride", do), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
        _set4(getattr(p, f), t)
    plan.ensure_workspace(dev)
    ref, s = ctypes.byref(p), _stream_ptr(dev)
    print("case dq computes delta", M, D, doc, dtype, flush=True)
    for name in (["fa_mask_plan"] if doc else []) + ["fa_fwd", "fa_bwd_delta", "fa_bwd_dkdv", "fa_bwd_dq"]:
        _cabi.check(getattr(L, name)(ref, s), name)
    torch.cuda.synchronize()
    want = [t.clone() for t in (delta, dq, dk, dv)]
    for t in (delta, dq, dk, dv):
        t.fill_(float("nan"))
    p.flags = _cabi.FA_FLAG_DQ_DELTA
    for name in ("fa_bwd_dq", "fa_bwd_dkdv"):
        _cabi.check(getattr(L, name)(ref, s), name)
    torch.cuda.synchronize()
    assert torch.allclose(delta, want[0], rtol=1e-5, atol=1e-5 * float(want[0].abs().max())), (delta - want[0]).abs().max()
    for name, got, w_ in zip(("dq", "dk", "dv"), (dq, dk, dv), want[1:]):
        assert not torch.isnan(got).any(), name
        err = (got.float() - w_.float()).abs().max().item()
        assert err <= (1e-4 if dtype == torch.float32 else 2.0 ** -7) * max(1.0, w_.float().abs().max().item()), (name, err)


def test_harness_cell_runs_and_agrees():
    from flash_mi355 import harness as Hn
    torch.manual_seed(5)
    checks, benches = Hn.run_attn(["torch", "mem", "mi355"], [2, 2, 256, 64], True, "bf16", True,
                                  check_times=1, bench_times=2, warmup_times=1)
    for key, diffs in checks:
        if key["func_name"] == "mi355":
            assert all(0 <= d <= 5e-2 for d in diffs), diffs
    assert len(benches) == 9 and all(float(b[1][0]) > 0 for b in benches if b[0]["func_name"] == "mi355")
    # "fp32" is one of the harness's dtypes (testing.py:158): the fp32 kernels against torch eager in fp32
    checks, _ = Hn.run_attn(["torch", "mi355"], [1, 2, 200, 64], True, "fp32", True, check_times=1, bench_times=0)
    for key, diffs in checks:
        if key["func_name"] == "mi355":
            assert all(0 <= d <= 1e-3 for d in diffs), diffs


def test_per_head_int64_ids():
    _run_case(1, 3, 3, 192, 192, 64, torch.bfloat16, True, True, seed=9, per_head_ids=True, id_dtype=torch.int64)


def test_golden_fixtures():
    """The committed fixtures (inputs + fp64 answers) through the HIP operator."""
    from pathlib import Path
    from flash_mi355 import attention, attention_with_lse, mask_dump
    for path in sorted((Path(__file__).parent / "golden").glob("*.npz")):
        z = np.load(path, allow_pickle=False)
        dt = torch.bfloat16 if "bfloat16" in str(z["dtype"]) else torch.float16
        causal, doc = bool(z["causal"]), bool(z["doc"])
        print("fixture", path.stem, flush=True)
        q, k, v, do = (torch.from_numpy(z[n]).to(dt).cuda() for n in ("q", "k", "v", "do"))
        eq = torch.from_numpy(z["eq"]).cuda() if doc else None
        ek = torch.from_numpy(z["ek"]).cuda() if doc else None
        mode = 1 if doc else 0
        if "block" in z.files:   # block mask: the map travels in the place of eq
            eq = ek = torch.from_numpy(z["block"]).cuda()
            mode = 2
        B, H, M, _ = q.shape
        N = k.shape[2]
        keep = np.unpackbits(z["keep"], axis=-1, count=N).astype(bool)
        assert np.array_equal(mask_dump(B, H, M, N, causal, eq, ek, mode).cpu().numpy(), keep)
        out, lse = attention_with_lse(q, k, v, causal, None, eq, ek, mode)
        assert (out.float().cpu().numpy() - z["o"]).__abs__().max() <= TOL_O
        dead = np.isinf(z["lse"])                      # rows without any kept key: -inf on both sides
        assert np.array_equal(np.isinf(lse.cpu().numpy()), dead)
        assert np.abs(np.where(dead, 0.0, lse.cpu().numpy() - np.where(dead, 0.0, z["lse"]))).max() <= TOL_LSE
        q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
        attention(q, k, v, causal, None, eq, ek, mode).backward(do)
        for name, got in (("dq", q.grad), ("dk", k.grad), ("dv", v.grad)):
            ref = z[name]
            check_close(name, got, torch.from_numpy(np.asarray(ref)))


def test_device_mask_plan_matches_host_restatement():
    """Workspace written by fa_mask_plan against tests/_plan_ref.py."""
    import ctypes
    from flash_mi355 import _cabi
    from flash_mi355.api import _Plan
    from tests import _plan_ref as P
    rng = np.random.default_rng(3)
    B, H, M, N, D = 2, 2, 300, 450, 64
    ek = np.stack([_ids(rng, B, H, N, "uniform") for _ in range(H)], axis=1)
    eq = np.ascontiguousarray(ek[:, :, N - M:])
    q = torch.zeros(B, H, M, D, dtype=torch.bfloat16, device="cuda")
    k = torch.zeros(B, H, N, D, dtype=torch.bfloat16, device="cuda")
    plan = _Plan(q, k, k, True, 1.0, torch.from_numpy(eq).cuda(), torch.from_numpy(ek).cuda(), 1)
    plan.ensure_workspace(q.device)
    torch.cuda.synchronize()
    ws = plan.workspace.cpu().numpy()
    r256 = lambda x: (x + 255) // 256 * 256
    Mp, Np, Pp = (M + 63) // 64 * 64, (N + 63) // 64 * 64, (M + 255) // 256 * 256 + 256
    nQs, nKs = Pp // 64, Np // 64
    off = 0
    take = lambda n: (off, off + n)
    o_eq = off; off += r256(B * H * Mp * 4)
    o_ek = off; off += r256(B * H * Np * 4)
    o_pm = off; off += r256(B * H * Pp * 4)
    o_pq = off; off += r256(B * H * Pp * 4)
    o_pp = off; off += r256(B * H * Pp * 4)
    off += r256(B * H * ((Mp + 1023) // 1024) * 4)     # per-chunk counts of the partition
    o_hd = off; off += r256(B * H * 32)
    o_qs = off; off += r256(B * H * nQs * 32)
    o_ks = off; off += r256(B * H * nKs * 32)
    # no scratch for split tiles here: N / 64 < 32 key tiles, no key range is ever cut
    assert off == ws.size
    i32 = lambda o, n: ws[o:o + 4 * n].view(np.int32)
    perm = i32(o_pm, B * H * Pp).reshape(B, H, Pp)
    peq = i32(o_pq, B * H * Pp).reshape(B, H, Pp)
    ppos = i32(o_pp, B * H * Pp).reshape(B, H, Pp)
    assert np.array_equal(ppos, np.where(perm >= 0, perm + (N - M), -1))   # diagonal positions: gap + row
    hdr = i32(o_hd, B * H * 8).reshape(B, H, 8)
    qs = i32(o_qs, B * H * nQs * 8).reshape(B, H, nQs, 8)
    ks = i32(o_ks, B * H * nKs * 8).reshape(B, H, nKs, 8)
    assert np.array_equal(i32(o_eq, B * H * Mp).reshape(B, H, Mp)[:, :, :M], eq)
    assert np.array_equal(i32(o_ek, B * H * Np).reshape(B, H, Np)[:, :, :N], ek)
    for b in range(B):
        for h in range(H):
            rp, rh, rq = P.plan_q(eq[b, h].astype(np.int64), M)
            assert np.array_equal(perm[b, h], rp)
            assert np.array_equal(peq[b, h][rp >= 0], eq[b, h][rp[rp >= 0]])
            rk = P.plan_k(ek[b, h].astype(np.int64), N)
            assert list(hdr[b, h][:4]) == [rh["nL"], rh["nG"], rh["nLp"], rh["nT128"]]
            assert hdr[b, h][4] == P.first_local_key_tile(rq, rk, True, N - M)
            for t, s_ in enumerate(rq):
                got = qs[b, h, t]
                # the device stores key positions of the rows' diagonals: gap + row without per-row positions
                assert got[5] == s_["nvalid"] and got[2] == s_["glob"] and got[4] == (s_["rmax"] + (N - M) if s_["nvalid"] else -1)
                if s_["nvalid"]:
                    assert got[3] == s_["rmin"] + (N - M)
                if s_["lo"] <= s_["hi"]:
                    assert (got[0], got[1]) == (s_["lo"], s_["hi"])
                else:
                    assert got[0] > got[1]
                # key-tile range of the plan: exactly the first / last tile the visit test admits
                cand = [kt for kt, k_ in enumerate(rk) if P.visits(s_, k_, kt, True, N - M)]
                if cand:
                    assert (got[6], got[7]) == (cand[0], cand[-1])
                else:
                    assert got[7] < got[6]
            for t, s_ in enumerate(P.plan_k(ek[b, h].astype(np.int64), N)):
                assert (ks[b, h, t, 0], ks[b, h, t, 1]) == (s_["lo"], s_["hi"])


@pytest.mark.parametrize("causal", [False, True])
def test_varlen_matches_per_sequence_oracle(causal):
    """Packed variable-length batch: every sequence against the oracle run on that sequence alone
    (plain attention, no ids), including an empty sequence, a one-token one and grouped heads."""
    from flash_mi355 import attention_varlen
    from oracle import attention_oracle as O
    lens = [5, 130, 0, 1, 64, 300, 77]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    T, H, Hk, D = int(cu[-1]), 4, 2, 64
    g = torch.Generator().manual_seed(7)
    q = torch.randn(T, H, D, generator=g).to(torch.bfloat16)
    k = torch.randn(T, Hk, D, generator=g).to(torch.bfloat16)
    v = torch.randn(T, Hk, D, generator=g).to(torch.bfloat16)
    do = torch.randn(T, H, D, generator=g).to(torch.bfloat16)
    print(f"varlen lens={lens} causal={causal}", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = attention_varlen(qd, kd, vd, cu.cuda(), causal=causal)
    assert out.shape == (T, H, D) and out.is_contiguous()
    out.backward(do.cuda())
    torch.cuda.synchronize()
    for s in range(len(lens)):
        a, b = int(cu[s]), int(cu[s + 1])
        if a == b:
            continue
        sl = lambda t: t[a:b].transpose(0, 1)[None]          # [1, heads, len, D]
        ro, _, rdq, rdk, rdv = O.attention_autograd(sl(q), sl(k), sl(v), sl(do), causal, None, None, None, 0)
        for name, got, ref in (("o", out.detach(), ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
            check_close(f"sequence {s} {name}", sl(got.float().cpu()), ref, quiet=True)


def test_varlen_causal_with_longer_key_sequences():
    """Causal packed batch whose sequences have more keys than queries (chunked prefill / decoding):
    every sequence bottom-right aligned on its own, against the oracle run on that sequence alone."""
    from flash_mi355 import attention_varlen
    from oracle import attention_oracle as O
    lq, lk = [40, 3, 0, 100, 1], [40, 200, 5, 164, 77]
    cuq = torch.tensor(np.concatenate([[0], np.cumsum(lq)]), dtype=torch.int32)
    cuk = torch.tensor(np.concatenate([[0], np.cumsum(lk)]), dtype=torch.int32)
    Tq, Tk, H, Hk, D = int(cuq[-1]), int(cuk[-1]), 4, 2, 64
    g = torch.Generator().manual_seed(23)
    q = torch.randn(Tq, H, D, generator=g).to(torch.bfloat16)
    k = torch.randn(Tk, Hk, D, generator=g).to(torch.bfloat16)
    v = torch.randn(Tk, Hk, D, generator=g).to(torch.bfloat16)
    do = torch.randn(Tq, H, D, generator=g).to(torch.bfloat16)
    print("varlen causal, longer key sequences", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = attention_varlen(qd, kd, vd, cuq.cuda(), cuk.cuda(), causal=True)
    assert out.shape == (Tq, H, D)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    for s in range(len(lq)):
        a, b, c, d = int(cuq[s]), int(cuq[s + 1]), int(cuk[s]), int(cuk[s + 1])
        if a == b:
            assert kd.grad[c:d].abs().max().item() == 0 and vd.grad[c:d].abs().max().item() == 0   # keys nobody asked for
            continue
        sq = lambda t: t[a:b].transpose(0, 1)[None]
        sk = lambda t: t[c:d].transpose(0, 1)[None]
        ro, _, rdq, rdk, rdv = O.attention_autograd(sq(q), sk(k), sk(v), sq(do), True, None, None, None, 0)
        for name, got, ref, sl in (("o", out.detach(), ro, sq), ("dq", qd.grad, rdq, sq), ("dk", kd.grad, rdk, sk), ("dv", vd.grad, rdv, sk)):
            check_close(f"sequence {s} {name}", sl(got.float().cpu()), ref, quiet=True)


def test_varlen_takes_boundaries_from_the_host_and_needs_key_boundaries_for_other_key_counts():
    """cu_seqlens on the host give the same result as on the device (they are moved to q's device), and a key
    tensor of another length without cu_seqlens_k is refused instead of reusing the query boundaries."""
    from flash_mi355 import attention_varlen
    lq, lk = [40, 3, 100, 1], [40, 200, 164, 77]
    cuq = torch.tensor(np.concatenate([[0], np.cumsum(lq)]), dtype=torch.int32)
    cuk = torch.tensor(np.concatenate([[0], np.cumsum(lk)]), dtype=torch.int32)
    g = torch.Generator().manual_seed(29)
    q = torch.randn(int(cuq[-1]), 2, 64, generator=g).to(torch.bfloat16).cuda()
    k, v = (torch.randn(int(cuk[-1]), 2, 64, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
    on_dev = attention_varlen(q, k, v, cuq.cuda(), cuk.cuda(), causal=True)
    on_host = attention_varlen(q, k, v, cuq, cuk, causal=True)
    assert torch.equal(on_dev, on_host)
    assert torch.equal(attention_varlen(q, q, q, cuq), attention_varlen(q, q, q, cuq.cuda()))
    with pytest.raises(AssertionError, match="cu_seqlens_k"):
        attention_varlen(q, k, v, cuq.cuda())


COLS_CASES = [
    # B, H, Hk, M, N, D, dtype, causal, ids, window: more keys than queries, the queries' documents at the end
    (2, 2, 2, 300, 1500, 128, torch.bfloat16, True, "uniform", 0),     # one tile of global rows
    (1, 4, 2, 300, 1700, 128, torch.float16, True, "uniform", 0),      # grouped heads: one tile per query head
    (1, 2, 2, 900, 2100, 128, torch.bfloat16, True, "uniform", 0),     # two tiles
    (1, 2, 2, 2000, 3100, 128, torch.bfloat16, True, "uniform", 0),    # three tiles: the general kernel keeps these columns
    (1, 2, 2, 300, 1500, 128, torch.bfloat16, True, "alllocal", 0),    # no global row at all: the columns get zeros
    (1, 2, 2, 300, 1501, 64, torch.float16, True, "uniform", 0),       # ragged key count, D = 64
    (2, 2, 1, 200, 1333, 16, torch.bfloat16, True, "uniform", 0),
    (1, 2, 2, 333, 1777, 32, torch.bfloat16, True, "uniform", 0),
    (1, 2, 2, 300, 1500, 128, torch.bfloat16, True, "uniform", 700),   # sliding window: global rows lose the far keys
    (1, 2, 2, 300, 1500, 128, torch.bfloat16, False, "uniform", 0),    # no causal mask
    (1, 2, 2, 64, 4100, 128, torch.bfloat16, True, "allglobal", 0),    # every row global: all key columns
]


@pytest.mark.parametrize("case", COLS_CASES, ids=lambda c: "B%d-H%d_%d-M%d-N%d-D%d-%s-c%d-%s-w%d" % (
    c[0], c[1], c[2], c[3], c[4], c[5], str(c[6]).split(".")[-1], c[7], c[8], c[9]))
def test_key_columns_that_only_global_rows_see(case):
    """dK / dV of key columns no local row can need come from a kernel of their own (the global rows'
    Q / dO tiles resident, the keys streamed) when the global rows are few; the other columns and every
    other shape stay with the general kernel.  Both against the oracle, and the seam between them."""
    B, H, Hk, M, N, D, dtype, causal, kind, window = case
    _run_case(B, H, Hk, M, N, D, dtype, causal, True, seed=77 + M + N, ids_kind=kind, window=window)


def test_delta_with_more_than_65535_batch_head_pairs():
    """fa_bwd_delta walks the (batch, head) pairs with the grid's stride (a grid dimension stops at 65535)."""
    import ctypes
    from flash_mi355 import _cabi
    from flash_mi355.api import _Plan, _set4, _stream_ptr
    L = _cabi.lib()
    dev = torch.device("cuda")
    for dtype in (torch.bfloat16, torch.float32):
        B, H, M, D = 70, 1000, 8, 16
        g = torch.Generator().manual_seed(3)
        o = torch.randn(B, H, M, D, generator=g).to(dtype).to(dev)
        do = torch.randn(B, H, M, D, generator=g).to(dtype).to(dev)
        plan = _Plan(o, o, o, False, 0.25, None, None, 0)
        p = plan.p
        delta = torch.full((B, H, M), float("nan"), device=dev, dtype=torch.float32)
        dq, dk, dv = (torch.empty_like(o) for _ in range(3))
        lse = torch.zeros(B, H, M, device=dev, dtype=torch.float32)
        p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
        p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
        for f, t in (("o_stride", o), ("do_stride", do), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
            _set4(getattr(p, f), t)
        print(f"case delta with B*H = {B * H}, {dtype}", flush=True)
        _cabi.check(L.fa_bwd_delta(ctypes.byref(p), _stream_ptr(dev)), "fa_bwd_delta")
        torch.cuda.synchronize()
        ref = (o.float() * do.float()).sum(-1)
        assert (delta - ref).abs().max().item() <= 1e-4 * max(1.0, ref.abs().max().item())


def test_varlen_causal_sequence_with_fewer_keys_than_queries():
    """A sequence with fewer keys than queries, bottom-right aligned: its first rows see no key
    (O = 0, no gradient), the others the keys up to their diagonal; the whole packed problem against
    the oracle with the same ids and positions, and the short sequence against its own closed form."""
    from flash_mi355 import attention_varlen, varlen_ids, varlen_positions
    from oracle import attention_oracle as O
    lq, lk = [40, 30, 100], [40, 12, 164]
    cuq = torch.tensor(np.concatenate([[0], np.cumsum(lq)]), dtype=torch.int32)
    cuk = torch.tensor(np.concatenate([[0], np.cumsum(lk)]), dtype=torch.int32)
    Tq, Tk, H, D = int(cuq[-1]), int(cuk[-1]), 2, 64
    g = torch.Generator().manual_seed(29)
    q, do = (torch.randn(Tq, H, D, generator=g).to(torch.bfloat16) for _ in range(2))
    k, v = (torch.randn(Tk, H, D, generator=g).to(torch.bfloat16) for _ in range(2))
    print("varlen causal, a sequence with fewer keys than queries", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = attention_varlen(qd, kd, vd, cuq.cuda(), cuk.cuda(), causal=True)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    assert out[40:40 + 18].abs().max().item() == 0 and qd.grad[40:40 + 18].abs().max().item() == 0   # rows 0..17 of sequence 1: no key
    t4 = lambda t: t.transpose(0, 1)[None]
    eq = varlen_ids(cuq, Tq).view(1, 1, Tq).expand(1, H, Tq)
    ek = varlen_ids(cuk, Tk).view(1, 1, Tk).expand(1, H, Tk)
    ro, _, rdq, rdk, rdv = O.attention_autograd(t4(q), t4(k), t4(v), t4(do), True, None, eq, ek, 1,
                                                qpos=varlen_positions(cuq, cuk, Tq).view(1, Tq))
    for name, got, ref in (("o", out.detach(), ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        check_close(name, t4(got.float().cpu()), ref, quiet=True)
    # rows 18..29 of sequence 1 against that sequence alone: local row 18 + t sees local keys 0..t
    keep = torch.tril(torch.ones(12, 12, dtype=torch.bool))
    qs, ks, vs = (t4(x).float() for x in (q[58:70], k[40:52], v[40:52]))
    sc = (qs @ ks.transpose(-1, -2)) / math.sqrt(D)
    ref = torch.softmax(sc.masked_fill(~keep, float("-inf")), -1) @ vs
    assert (t4(out.detach()[58:70].float().cpu()) - ref).abs().max().item() <= TOL_O


def test_varlen_cross_attention():
    """Different query and key boundaries (non-causal): each query sequence sees the keys of the
    sequence with the same number."""
    from flash_mi355 import attention_varlen
    from oracle import attention_oracle as O
    lq, lk = [40, 3, 100], [17, 200, 64]
    cuq = torch.tensor(np.concatenate([[0], np.cumsum(lq)]), dtype=torch.int32)
    cuk = torch.tensor(np.concatenate([[0], np.cumsum(lk)]), dtype=torch.int32)
    Tq, Tk, H, D = int(cuq[-1]), int(cuk[-1]), 2, 128
    g = torch.Generator().manual_seed(11)
    q = torch.randn(Tq, H, D, generator=g).to(torch.float16)
    k = torch.randn(Tk, H, D, generator=g).to(torch.float16)
    v = torch.randn(Tk, H, D, generator=g).to(torch.float16)
    print("varlen cross", flush=True)
    out = attention_varlen(q.cuda(), k.cuda(), v.cuda(), cuq.cuda(), cuk.cuda())
    torch.cuda.synchronize()
    for s in range(3):
        qs = q[int(cuq[s]):int(cuq[s + 1])].transpose(0, 1)[None]
        ks = k[int(cuk[s]):int(cuk[s + 1])].transpose(0, 1)[None]
        vs = v[int(cuk[s]):int(cuk[s + 1])].transpose(0, 1)[None]
        ro, _ = O.attention_closed_form(qs, ks, vs, False, None, None, None, 0)
        got = out[int(cuq[s]):int(cuq[s + 1])].transpose(0, 1)[None].float().cpu()
        assert (got - ro).abs().max().item() <= TOL_O


# fp32 tensors run on fp32 MFMAs: the oracle is fp32 too, so the bound is a few ulps of the
# accumulated sums, not the 16-bit rounding of the other cases
TOL_F32 = 2e-4
FP32_CASES = [
    # B, H, Hk, M, N, D, causal, doc
    (2, 4, 4, 512, 512, 64, True, True),       # the reference's own CPU-runnable configuration
    (1, 2, 2, 256, 256, 128, True, False),
    (1, 2, 2, 200, 200, 128, False, True),     # ragged
    (1, 4, 2, 130, 130, 128, True, True),      # grouped-query, ragged
    (1, 2, 2, 77, 333, 64, True, True),        # rectangular, bottom-right causal
    (1, 2, 2, 96, 96, 32, True, True),
    (2, 2, 1, 100, 300, 16, True, True),
    (1, 1, 1, 1, 1, 16, False, False),
]


@pytest.mark.parametrize("case", FP32_CASES, ids=lambda c: "f32-B%d-H%d-%d-M%d-N%d-D%d-c%d-d%d" % tuple(int(x) for x in c))
def test_fp32_tensors(case):
    B, H, Hk, M, N, D, causal, doc = case
    _run_case(B, H, Hk, M, N, D, torch.float32, causal, doc, seed=5, tol_o=TOL_F32, tol_lse=TOL_F32)


@pytest.mark.parametrize("M,N,D,window,kind", [(300, 300, 64, 0, "random"), (333, 77, 128, 0, "random"), (700, 900, 128, 40, "steps"),
                                              (130, 190, 16, 7, "random"), (1300, 1300, 32, 0, "steps")])
def test_fp32_per_row_causal_positions(M, N, D, window, kind):
    """fp32 kernels with ids walk the permuted order of the plan and take the rows' diagonals from it."""
    _run_case(1, 2, 1, M, N, D, torch.float32, True, True, seed=8 + M, window=window, qpos=kind, tol_o=TOL_F32, tol_lse=TOL_F32)


def test_fp32_packed_documents_multi_tile():
    """fp32 with ids over several 128-row tiles per group (local tiles, a padded boundary, global tiles),
    per-head ids and grouped heads; causal and not."""
    _run_case(1, 4, 2, 1100, 1100, 64, torch.float32, True, True, seed=31, tol_o=TOL_F32, tol_lse=TOL_F32)
    _run_case(2, 2, 2, 700, 1000, 128, torch.float32, False, True, seed=32, per_head_ids=True, tol_o=TOL_F32, tol_lse=TOL_F32)
    _run_case(1, 2, 2, 900, 900, 32, torch.float32, True, True, seed=33, ids_kind="alllocal", tol_o=TOL_F32, tol_lse=TOL_F32)


def test_fp32_all_global_and_all_local_ids():
    _run_case(1, 2, 2, 160, 160, 64, torch.float32, True, True, seed=6, ids_kind="allglobal", tol_o=TOL_F32, tol_lse=TOL_F32)
    _run_case(1, 2, 2, 160, 160, 64, torch.float32, False, True, seed=6, ids_kind="alllocal", tol_o=TOL_F32, tol_lse=TOL_F32)


# Sliding window and prefix-LM (causal masks the library adds; no counterpart in the reference):
# checked against the oracle's closed form like every other case.
BAND_CASES = [
    # B, H, Hk, M, N, D, dtype, doc, window, prefix
    (1, 2, 2, 512, 512, 128, torch.bfloat16, False, 100, 0),
    (1, 2, 2, 512, 512, 128, torch.bfloat16, False, 1, 0),
    (1, 2, 2, 512, 512, 128, torch.bfloat16, False, 64, 0),
    (1, 2, 2, 300, 300, 64, torch.bfloat16, True, 77, 0),      # window + ids, ragged
    (1, 4, 2, 200, 456, 128, torch.float16, True, 130, 0),     # window + ids, rectangular, grouped-query
    (1, 2, 2, 2048, 2048, 64, torch.bfloat16, False, 256, 0),  # many key tiles before the window
    (1, 2, 2, 2048, 2048, 128, torch.bfloat16, True, 300, 0),
    (1, 2, 2, 512, 512, 128, torch.bfloat16, False, 0, 200),
    (1, 2, 2, 512, 512, 64, torch.bfloat16, False, 0, 1),
    (1, 2, 2, 300, 300, 128, torch.bfloat16, True, 0, 150),    # prefix + ids
    (1, 2, 2, 128, 512, 128, torch.float16, True, 0, 450),     # prefix reaching past the first rows' diagonal, rectangular
    (1, 2, 2, 256, 256, 32, torch.bfloat16, True, 0, 256),     # everything is prefix
    (1, 2, 2, 256, 256, 16, torch.bfloat16, True, 33, 0),
    (1, 2, 2, 333, 333, 64, torch.float32, True, 50, 0),
    (1, 2, 2, 333, 333, 128, torch.float32, False, 0, 100),
    (1, 4, 2, 100, 260, 32, torch.float32, True, 0, 200),
]


@pytest.mark.parametrize("case", BAND_CASES, ids=lambda c: "B%d-H%d_%d-M%d-N%d-D%d-%s-d%d-w%d-p%d" % (
    c[0], c[1], c[2], c[3], c[4], c[5], str(c[6]).split(".")[-1], c[7], c[8], c[9]))
def test_sliding_window_and_prefix(case):
    B, H, Hk, M, N, D, dtype, doc, window, prefix = case
    tol = TOL_F32 if dtype == torch.float32 else TOL_O
    _run_case(B, H, Hk, M, N, D, dtype, True, doc, seed=77, window=window, prefix=prefix, tol_o=tol,
              tol_lse=TOL_F32 if dtype == torch.float32 else TOL_LSE)


def test_window_and_prefix_mask_bit_exact():
    from flash_mi355 import mask_dump, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    rng = np.random.default_rng(9)
    for (B, H, M, N) in [(1, 2, 200, 200), (1, 2, 77, 333)]:
        ek = torch.from_numpy(np.stack([_ids(rng, B, H, N, "uniform") for _ in range(H)], axis=1))
        eq = torch.from_numpy(np.stack([_ids(rng, B, H, M, "uniform") for _ in range(H)], axis=1))
        for kw in ({"window": 1}, {"window": 40}, {"window": 1000}, {"prefix": 1}, {"prefix": 90}, {"prefix": 1000}):
            got = mask_dump(B, H, M, N, True, eq.cuda(), ek.cuda(), SCORE_FUNC_MODE1_DOC, **kw).cpu().numpy()
            ref = np.broadcast_to(O.keep_mask(M, N, True, eq.numpy(), ek.numpy(), 1, **kw), (B, H, M, N))
            assert np.array_equal(got, ref), kw
            got = mask_dump(B, H, M, N, True, **kw).cpu().numpy()
            assert np.array_equal(got, np.broadcast_to(O.keep_mask(M, N, True, **kw), (B, H, M, N))), kw


def test_window_needs_causal():
    from flash_mi355 import attention
    q = torch.randn(1, 1, 64, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        attention(q, q, q, False, window=8)
    with pytest.raises(AssertionError):
        attention(q, q, q, True, window=8, prefix=8)


@pytest.mark.parametrize("seed", list(range(300, 324)))
def test_random_shapes_with_per_row_positions(seed):
    """Third seeded sweep: per-row causal positions (any order, or the steps of a packed batch) over the
    three element types, all head sizes, more or fewer queries than keys, windows, id layouts."""
    rng = np.random.default_rng(seed)
    D = int(rng.choice([16, 32, 64, 128]))
    dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
    B = int(rng.integers(1, 3)); Hk = int(rng.integers(1, 3)); H = Hk * int(rng.integers(1, 3))
    M = int(rng.integers(1, 700))
    N = int(rng.integers(2000, 2600)) if rng.random() < 0.2 else int(rng.integers(1, 1500))
    window = int(rng.choice([0, 0, 0, 5, 64, 300]))
    f32 = dtype == torch.float32
    _run_case(B, H, Hk, M, N, D, dtype, True, True, seed=seed, ids_kind=str(rng.choice(["uniform", "uniform", "allglobal", "alllocal"])),
              per_head_ids=bool(rng.random() < 0.3), window=window, qpos=str(rng.choice(["random", "steps"])),
              tol_o=TOL_F32 if f32 else TOL_O, tol_lse=TOL_F32 if f32 else TOL_LSE)


def test_p_crosses_the_wave_pair_as_fp16():
    """In the role-split dk/dv form (D = 128) the gradient wave forms dS = P (dP - delta) from the P that the
    score wave hands over through LDS.  While that copy was in the element type, bf16 tensors carried one
    rounding more than the reference (which multiplies its fp32 P, flash_triton.py:301), and a sweep of random
    cases found dK elements up to 19 % over the per-element bound (this case: 0.0206 against 0.02 at an exact
    value of -3.2081; grouped heads, local ids, window 876).  P <= 1 crosses as fp16 now, for either element
    type: 11 significant bits in the same two bytes.  The case sits at 0.65 of the bound."""
    _run_case(1, 4, 2, 243, 1419, 128, torch.bfloat16, True, True, seed=5012, ids_kind="alllocal", window=876)
    _run_case(2, 2, 1, 651, 617, 128, torch.bfloat16, False, True, seed=5086, ids_kind="alllocal")
    _run_case(2, 4, 2, 248, 1297, 128, torch.bfloat16, True, True, seed=5210, ids_kind="alllocal", prefix=530)


FLOOR_CASES = [
    # B, H, Hk, M, N, D, seed, window, per-head ids, positions
    (2, 4, 2, 563, 879, 128, 5128, 96, False, None),
    (2, 2, 1, 180, 5, 64, 1429, 0, True, "steps"),
    (2, 2, 2, 215, 4, 128, 1433, 64, False, "steps"),
    (1, 2, 1, 499, 4, 64, 1307, 64, False, "steps"),
]


# Ceilings of the four cases, as multiples of the per-element bound: what was measured (dK 1.17, 1.09, 1.09, 1.92;
# in the last case also dV 2.52, exactly where the model of the reference's roundings puts it) plus a small margin;
# every other tensor of these cases is held to the plain bound, and a regression past the documented floor fails.
FLOOR_CEILINGS = {5128: {"dk": 1.25}, 1429: {"dk": 1.25}, 1433: {"dk": 1.25}, 1307: {"dk": 2.0, "dv": 2.75}}


@pytest.mark.parametrize("case", FLOOR_CASES, ids=lambda c: "M%d-N%d-D%d-seed%d" % (c[3], c[4], c[5], c[6]))
def test_case_found_outside_the_bound(case):
    """Found by sweeps of about 3500 random cases outside this suite (bf16, local ids).  What they share: rows
    that keep very few keys, so P is close to 1, and dK elements that sum over many such rows.  O, LSE and dQ
    of these cases meet the plain bound (dV too, except in the fourth); dK is held to a pinned ceiling just above
    what was measured (FLOOR_CEILINGS), so that these known exceedances stay visible and cannot grow unnoticed.
    First case (documents of 8-96 tokens, window 96): one element of dK comes out as 0.9727 where the exact
    value is 0.9492 (0.0235 against the bound of 0.02).  The error that the 16-bit storage of O puts into
    delta = rowsum(O dO) reaches dS = P (dP - delta) undamped when P is large; the reference forms delta from
    the stored O as well (flash_triton.py:165).  The CPU model of the reference's storage roundings
    (oracle.attention_grads(store_dtype=...), output rounded too) reaches 0.92 of the bound on the same inputs
    at another element; the kernel's O differs from the model's by one bf16 step in places (other summation
    order), which makes its delta another draw from the same error distribution: here the kernel is less
    accurate than an implementation that rounds exactly where the reference rounds.  Recomputed on the CPU with
    the kernel's own O, the excess comes from one element of dS: magnitude 10 (dP - delta = 27.8, P = 0.359),
    1.5e-4 away from a bf16 rounding tie (9.9686 between 9.9375 and 10.0).  Its half-step error of 0.031 is worth
    0.0083 in dK, 40 % of the bound, whichever way it falls: with the exact P it falls down and cancels the delta
    error of the other 135 rows of that column, with P rounded to the 11 bits of the fp16 hand-over between the
    wave pair (or to 8) it falls up and adds to it.  The hand-over is the one place where this kernel rounds and the
    reference does not (flash_triton.py:301 keeps P in fp32), but it acts as the tie-breaker of a rounding of dS
    that the reference performs too (flash_triton.py:306).
    Second and third case (5 and 4 keys in all, 180 and 215 query rows with per-row positions, 1.0-1.6 kept keys
    per row, 55 rows per key): 1.09 of the bound -- and the CPU model of the reference's roundings is itself at
    1.06 and 1.09 of it there: no implementation that rounds where the reference rounds meets the bound on
    these inputs.  Fourth case (4 keys, 499 rows, two query heads per key head, every id global: 4 kept keys per
    row, a thousand terms per dK element): 1.92 of the bound, where the model of the reference's roundings is
    at 2.40 for dK and 2.52 for dV -- the kernel's dV sits at that same 2.52: 998 products of a bf16-rounded P per
    element, flash_triton.py:291 -- (the reference rounds each head's dK, dV before the group sum,
    flash_triton.py:635-637; the kernel sums the group in fp32).  Every other element of these cases, and every
    case of the suite, is inside the bound; the bound is not widened for any other case."""
    B, H, Hk, M, N, D, seed, window, per_head, qpos = case
    _run_case(B, H, Hk, M, N, D, torch.bfloat16, True, True, seed=seed, ids_kind="allglobal" if seed == 1307 else "alllocal",
              window=window, per_head_ids=per_head, qpos=qpos, ceilings=FLOOR_CEILINGS[seed])


def test_the_reference_call_shape_through_the_drop_in_module():
    """The reference's own call, argument for argument: `from flash_triton import attention`, called as
    testing.py:84 calls it (positional q, k, v, causal, scale; eq / ek / score_func_mode by keyword) and
    as flash_triton.py:640-641 forwards it -- FlashAttention.apply with exactly eight positional
    arguments -- with the ids the reference's sampler makes (testing.py:110-120: an int64 document
    counter shifted so that the first third of the documents is local, expanded over the heads with
    stride 0, the same tensor for eq and ek), then `.backward(do)` (the reference's backward returns an
    8-tuple, flash_triton.py:638).  All four results against the oracle."""
    import flash_triton
    from flash_triton import FlashAttention, attention, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    from pathlib import Path
    assert Path(flash_triton.__file__).resolve().parent.name == "triton-flash-attention-with-flexible-masks_amd"
    B, H, L, D = 2, 4, 1024, 128
    shape = (B, H, L, D)
    g = torch.Generator().manual_seed(4242)
    q, k, v, do = (torch.randn(shape, generator=g).to(torch.bfloat16) for _ in range(4))
    ids = (torch.rand([B, L], generator=g) <= 0.05).cumsum(-1)          # testing.py:112
    ids = ids - ids[:, -1:] // 3                                         # testing.py:113
    assert ids.dtype == torch.int64 and (ids < 0).any() and (ids >= 0).any()
    eq_host = ids[:, None, :].expand(shape[:-1])                         # testing.py:118
    eq = ids.cuda()[:, None, :].expand(shape[:-1])
    assert eq.stride(1) == 0
    print("case reference call shape", flush=True)
    ref_o, _, ref_dq, ref_dk, ref_dv = O.attention_autograd(q, k, v, do, True, None, eq_host, eq_host, 1)
    for form in ("apply", "attention"):
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        if form == "apply":
            out = FlashAttention.apply(qd, kd, vd, True, None, eq, eq, SCORE_FUNC_MODE1_DOC)   # flash_triton.py:641
        else:
            out = attention(qd, kd, vd, True, qd.shape[-1] ** (-0.5), eq=eq, ek=eq, score_func_mode=1)   # testing.py:84,179
        assert isinstance(out, torch.Tensor) and out.shape == qd.shape and out.dtype == qd.dtype   # Out only, flash_triton.py:564
        out.backward(do.cuda())
        torch.cuda.synchronize()
        assert (out.detach().float().cpu() - ref_o).abs().max().item() <= TOL_O
        for name, got, ref in (("dq", qd.grad, ref_dq), ("dk", kd.grad, ref_dk), ("dv", vd.grad, ref_dv)):
            check_close(f"{form} {name}", got, ref)


@pytest.mark.parametrize("seed", list(range(200, 232)))
def test_random_shapes_all_types_and_masks(seed):
    """Second seeded sweep: the three element types, and on causal draws a sliding window or a
    prefix of random size (from a single key to longer than the sequence), with and without ids."""
    rng = np.random.default_rng(seed)
    D = int(rng.choice([16, 32, 64, 128]))
    Hk = int(rng.choice([1, 2]))
    H = Hk * int(rng.choice([1, 2, 3]))
    B = int(rng.choice([1, 2]))
    causal = bool(rng.integers(0, 3) > 0)
    doc = bool(rng.integers(0, 2))
    M = int(rng.integers(1, 700))
    N = int(rng.integers(M, 900)) if (causal or doc or rng.integers(0, 2)) else int(rng.integers(1, 900))
    dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
    window = prefix = 0
    if causal:
        which = int(rng.integers(0, 3))
        if which == 1:
            window = int(rng.choice([1, 2, 31, 64, 65, 200, N, N + 50])) if rng.integers(0, 2) else int(rng.integers(1, N + 1))
        elif which == 2:
            prefix = int(rng.choice([1, 63, 64, 129, N, N + 7])) if rng.integers(0, 2) else int(rng.integers(1, N + 1))
    kind = str(rng.choice(["uniform", "uniform", "alllocal", "allglobal"]))
    f32 = dtype == torch.float32
    _run_case(B, H, Hk, M, N, D, dtype, causal, doc, seed=seed, ids_kind=kind, window=window, prefix=prefix,
              tol_o=TOL_F32 if f32 else TOL_O, tol_lse=TOL_F32 if f32 else TOL_LSE)


@pytest.mark.parametrize("B,H,Hk", [(1, 1, 1), (3, 1, 1), (1, 5, 5), (1, 6, 3), (7, 1, 1), (3, 3, 1), (1, 12, 4), (5, 2, 2)])
def test_head_counts_that_do_not_fill_the_xcds_evenly(B, H, Hk):
    """Batch x head counts that are not multiples of 8 (the workgroup -> XCD map has three cases:
    whole heads per XCD, a head shared by several XCDs, (slot, head) pairs dealt round-robin), with
    enough query tiles per head that every case deals more than one round, with and without ids."""
    _run_case(B, H, Hk, 450, 450, 64, torch.bfloat16, True, True, seed=B * 100 + H)
    _run_case(B, H, Hk, 520, 840, 128, torch.float16, True, False, seed=B * 100 + H + 1)


def test_varlen_with_sliding_window():
    """Packed sequences with a sliding window: inside every sequence the window counts that
    sequence's own positions (the packed row's causal offset is the same for query and key)."""
    from flash_mi355 import attention_varlen
    from oracle import attention_oracle as O
    lens, W_ = [150, 9, 260, 64], 48
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    T, H, D = int(cu[-1]), 2, 128
    g = torch.Generator().manual_seed(13)
    q, k, v, do = (torch.randn(T, H, D, generator=g).to(torch.bfloat16) for _ in range(4))
    print("varlen window", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = attention_varlen(qd, kd, vd, cu.cuda(), causal=True, window=W_)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    for s in range(len(lens)):
        a, b = int(cu[s]), int(cu[s + 1])
        sl = lambda t: t[a:b].transpose(0, 1)[None]
        ro, _, rdq, rdk, rdv = O.attention_autograd(sl(q), sl(k), sl(v), sl(do), True, None, None, None, 0, window=W_)
        for name, got, ref in (("o", out.detach(), ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
            check_close(f"sequence {s} {name}", sl(got.float().cpu()), ref, quiet=True)


def test_varlen_fp32():
    """Packed sequences in fp32 (the fp32 kernels skip whole tiles by the plan's id summaries)."""
    from flash_mi355 import attention_varlen
    from oracle import attention_oracle as O
    lens = [300, 40, 129, 500, 31]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    T, H, Hk, D = int(cu[-1]), 2, 1, 64
    g = torch.Generator().manual_seed(17)
    q = torch.randn(T, H, D, generator=g); k = torch.randn(T, Hk, D, generator=g); v = torch.randn(T, Hk, D, generator=g)
    do = torch.randn(T, H, D, generator=g)
    for causal in (True, False):
        print(f"varlen fp32 causal={causal}", flush=True)
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        out = attention_varlen(qd, kd, vd, cu.cuda(), causal=causal)
        out.backward(do.cuda())
        torch.cuda.synchronize()
        for s in range(len(lens)):
            a, b = int(cu[s]), int(cu[s + 1])
            sl = lambda t: t[a:b].transpose(0, 1)[None]
            ro, _, rdq, rdk, rdv = O.attention_autograd(sl(q), sl(k), sl(v), sl(do), causal, None, None, None, 0)
            for name, got, ref in (("o", out.detach(), ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
                err = (sl(got.float().cpu()) - ref).abs().max().item()
                assert err <= TOL_F32 * max(1.0, ref.abs().max().item()), f"sequence {s} {name} err {err}"


def test_varlen_fp32_causal_with_longer_key_sequences():
    """The one-launch causal packed batch with different boundaries on the fp32 kernels."""
    from flash_mi355 import attention_varlen
    from oracle import attention_oracle as O
    lq, lk = [40, 3, 0, 100, 1, 200], [40, 200, 5, 164, 77, 333]
    cuq = torch.tensor(np.concatenate([[0], np.cumsum(lq)]), dtype=torch.int32)
    cuk = torch.tensor(np.concatenate([[0], np.cumsum(lk)]), dtype=torch.int32)
    Tq, Tk, H, Hk, D = int(cuq[-1]), int(cuk[-1]), 2, 1, 64
    g = torch.Generator().manual_seed(41)
    q = torch.randn(Tq, H, D, generator=g); do = torch.randn(Tq, H, D, generator=g)
    k = torch.randn(Tk, Hk, D, generator=g); v = torch.randn(Tk, Hk, D, generator=g)
    print("varlen fp32 causal, longer key sequences", flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = attention_varlen(qd, kd, vd, cuq.cuda(), cuk.cuda(), causal=True)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    for s in range(len(lq)):
        a, b, c, d = int(cuq[s]), int(cuq[s + 1]), int(cuk[s]), int(cuk[s + 1])
        if a == b:
            assert kd.grad[c:d].abs().max().item() == 0 and vd.grad[c:d].abs().max().item() == 0
            continue
        sq = lambda t: t[a:b].transpose(0, 1)[None]
        sk = lambda t: t[c:d].transpose(0, 1)[None]
        ro, _, rdq, rdk, rdv = O.attention_autograd(sq(q), sk(k), sk(v), sq(do), True, None, None, None, 0)
        for name, got, ref, sl in (("o", out.detach(), ro, sq), ("dq", qd.grad, rdq, sq), ("dk", kd.grad, rdk, sk), ("dv", vd.grad, rdv, sk)):
            err = (sl(got.float().cpu()) - ref).abs().max().item()
            assert err <= TOL_F32 * max(1.0, ref.abs().max().item()), f"sequence {s} {name} err {err}"


@pytest.mark.parametrize("D", [16, 128])
@pytest.mark.parametrize("doc", [False, True])
def test_rows_past_the_end_of_a_slice_are_never_read(D, doc):
    """q, k, v, dO are views of larger buffers whose other rows are NaN: behind the last row of every
    (batch, head) slice there is no finite value anywhere, so a tile load that reached past the slice
    (the ragged last tile relies on the range check of the buffer loads, whose row term travels in the
    scalar offset) would put NaN into the products (0 * NaN).  Lengths are ragged on both sides."""
    from flash_mi355 import attention, SCORE_FUNC_MODE1_DOC
    from oracle import attention_oracle as O
    B, H, Hk, M, N = 2, 2, 2, 77, 65 + 128
    pad = 192   # rows of NaN behind every slice: more than any tile reaches
    g = torch.Generator().manual_seed(900 + D)
    rng = np.random.default_rng(900 + D)

    def padded(heads, L):
        buf = torch.full((B, heads, L + pad, D), float("nan"))
        buf[:, :, :L] = torch.randn(B, heads, L, D, generator=g)
        return buf.bfloat16()
    bq, bk, bv, bdo = padded(H, M), padded(Hk, N), padded(Hk, N), padded(H, M)
    q, k, v, do = bq[:, :, :M], bk[:, :, :N], bv[:, :, :N], bdo[:, :, :M]
    eq = ek = None
    if doc:
        ek = torch.from_numpy(_ids(rng, B, H, N, "uniform"))[:, None, :].expand(B, H, N)
        eq = ek[:, :, N - M:]
    print(f"case NaN behind every slice D={D} doc={doc}", flush=True)
    qd, kd, vd = (t.cuda()[:, :, :L].requires_grad_(True) for t, L in ((bq, M), (bk, N), (bv, N)))
    assert not qd.is_contiguous() and torch.isnan(bq.cuda()[:, :, M:]).all()
    mode = SCORE_FUNC_MODE1_DOC if doc else 0
    out = attention(qd, kd, vd, True, None, eq.cuda() if doc else None, ek.cuda() if doc else None, mode)
    out.backward(bdo.cuda()[:, :, :M])
    torch.cuda.synchronize()
    ref = O.attention_autograd(q.contiguous(), k.contiguous(), v.contiguous(), do.contiguous(), True, None, eq, ek, mode)
    for name, got, want in (("o", out, ref[0]), ("dq", qd.grad, ref[2]), ("dk", kd.grad, ref[3]), ("dv", vd.grad, ref[4])):
        assert not torch.isnan(got).any(), name
        check_close(name, got, want)


@pytest.mark.parametrize("doc", [False, True])
def test_expired_pair_wait_is_reported_in_dk(doc):
    """fa_bwd_dkdv at D = 128: the wave that polls for its partner's P has a bounded wait.  With the
    diagnostic flag the poll budget is zero, so waits expire although every wave still runs to its end;
    the waves concerned must say so by writing NaN into their dK rows.  dV (which does not depend on the
    wait) stays exact, and the same call without the flag gives finite dK again."""
    import ctypes
    from flash_mi355 import _cabi
    from flash_mi355.api import _Plan, _set4, _stream_ptr
    L = _cabi.lib()
    B, H, M, D = 1, 4, 1024, 128
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(515)
    rng = np.random.default_rng(515)
    ids = torch.from_numpy(_ids(rng, B, H, M, "uniform")).to(dev)[:, None, :].expand(B, H, M) if doc else None
    q, k, v, do = (torch.randn(B, H, M, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(4))
    o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    lse = torch.empty(B, H, M, device=dev, dtype=torch.float32)
    delta = torch.empty_like(lse)
    plan = _Plan(q, k, v, True, 1.0 / math.sqrt(D), ids, ids, 1 if doc else 0)
    p = plan.p
    p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
    p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    for f, t in (("o_stride", o), ("do_stride", do), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
        _set4(getattr(p, f), t)
    plan.ensure_workspace(dev)
    ref, s = ctypes.byref(p), _stream_ptr(dev)
    print("case expired pair wait, doc =", doc, flush=True)
    for name in (["fa_mask_plan"] if doc else []) + ["fa_fwd", "fa_bwd_delta", "fa_bwd_dkdv"]:
        _cabi.check(getattr(L, name)(ref, s), name)
    torch.cuda.synchronize()
    assert not torch.isnan(dk).any() and not torch.isnan(dv).any()
    good_dk, good_dv = dk.clone(), dv.clone()
    n0, n1 = ctypes.c_uint64(0), ctypes.c_uint64(0)
    _cabi.check(L.fa_pair_wait_expired(ctypes.byref(n0)), "fa_pair_wait_expired")
    p.flags = _cabi.FA_FLAG_DEBUG_NO_PAIR_WAIT
    # the diagnostic belongs to fa_bwd_dkdv alone: every other entry point refuses it
    for name in ("fa_fwd", "fa_bwd_dq", "fa_bwd_delta", "fa_mask_plan"):
        assert getattr(L, name)(ref, s) == -7, name
    _cabi.check(L.fa_bwd_dkdv(ref, s), "fa_bwd_dkdv")
    torch.cuda.synchronize()
    bad_rows = torch.isnan(dk.float()).any(dim=-1)           # [B, H, N]
    # At least one expiry is expected: a gradient wave reaches its first poll after two dP products, the
    # score wave publishes P only after S, the exponentials, the masks and the conversions, and with a
    # budget of zero a single failed poll is an expiry.
    assert bad_rows.any(), "no wait expired with a poll budget of zero: the report path was not exercised"
    # ... and the host is told without looking at dk: one count per wave that reported
    _cabi.check(L.fa_pair_wait_expired(ctypes.byref(n1)), "fa_pair_wait_expired")
    assert n1.value - n0.value == int(bad_rows.sum().item()) // 32
    # the report covers whole 32-key blocks of a wave, and every row that is not reported is right
    blocks = bad_rows.view(B, H, M // 32, 32)
    assert torch.equal(blocks.all(dim=-1), blocks.any(dim=-1))
    assert torch.equal(dk[~bad_rows], good_dk[~bad_rows])
    assert torch.equal(dv, good_dv)
    p.flags = 0
    _cabi.check(L.fa_bwd_dkdv(ref, s), "fa_bwd_dkdv")
    torch.cuda.synchronize()
    assert torch.equal(dk, good_dk) and torch.equal(dv, good_dv)
    n2 = ctypes.c_uint64(0)
    _cabi.check(L.fa_pair_wait_expired(ctypes.byref(n2)), "fa_pair_wait_expired")
    assert n2.value == n1.value   # a healthy launch counts nothing
