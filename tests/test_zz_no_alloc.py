"""fa_fwd_static: the forward whose mask plan and split scratch live in a static device array inside
the library (for callers that cannot allocate).  Checked through the C ABI against fa_mask_plan +
fa_fwd with a caller's workspace, on two calls in a row, the second with a smaller input (the array
keeps the first call's contents), then a third that needs split key ranges."""
import ctypes
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _problem(B, H, M, N, D, dtype, seed):
    from flash_mi355 import workloads as W
    from flash_mi355.api import _Plan, _set4
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    q = torch.randn(B, H, M, D, generator=g).to(dtype).to(dev)
    k = torch.randn(B, H, N, D, generator=g).to(dtype).to(dev)
    v = torch.randn(B, H, N, D, generator=g).to(dtype).to(dev)
    ids = np.stack([W.doc_ids_uniform(rng, N, 8, 96, 0.08) for _ in range(B)])
    ek = torch.from_numpy(ids).to(dev)[:, None, :].expand(B, H, N)
    eq = ek[:, :, N - M:]
    plan = _Plan(q, k, v, True, 1.0 / math.sqrt(D), eq, ek, 1)
    o = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, M), float("nan"), device=dev, dtype=torch.float32)
    plan.p.o, plan.p.lse = o.data_ptr(), lse.data_ptr()
    _set4(plan.p.o_stride, o)
    return plan, o, lse


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_forward_matches_the_workspace_forward(dtype):
    from flash_mi355 import _cabi
    from flash_mi355.api import _stream_ptr
    L = _cabi.lib()
    dev = torch.device("cuda")
    s = _stream_ptr(dev)
    tol_o, tol_l = (2e-4, 2e-4) if dtype == torch.float32 else (2e-2, 1e-3)
    # large, then smaller (stale contents of the first call behind and inside the second's plan), then a
    # long key range whose global-row tiles are cut into chunks (arrival counters and partial results in
    # the static array), then the small one again
    shapes = [(2, 4, 1000, 1000, 64), (1, 2, 200, 333, 64), (1, 2, 2304, 4608, 128), (1, 2, 200, 333, 64)]
    for i, (B, H, M, N, D) in enumerate(shapes):
        print(f"case static scratch {dtype} call {i}: B{B} H{H} M{M} N{N} D{D}", flush=True)
        plan, o, lse = _problem(B, H, M, N, D, dtype, 40 + i)
        p = plan.p
        assert p.workspace is None or p.workspace == 0
        _cabi.check(L.fa_fwd_static(ctypes.byref(p), s), "fa_fwd_static")
        torch.cuda.synchronize()
        got_o, got_l = o.clone(), lse.clone()
        o.fill_(float("nan")); lse.fill_(float("nan"))
        plan.ensure_workspace(dev)                      # the existing entry points: caller's workspace
        _cabi.check(L.fa_fwd(ctypes.byref(p), s), "fa_fwd")
        torch.cuda.synchronize()
        assert not torch.isnan(got_o).any() and not torch.isnan(got_l).any()
        dead = torch.isinf(lse)
        assert torch.equal(torch.isinf(got_l), dead)
        assert (got_l[~dead] - lse[~dead]).abs().max().item() <= tol_l
        assert (got_o.float() - o.float()).abs().max().item() <= tol_o
        if N < 2048:   # no key range is split at these sizes: the same kernels on the same plan, bit for bit
            assert torch.equal(got_o, o) and torch.equal(got_l, lse)


def test_static_scratch_forward_against_the_oracle():
    """The entry point against the CPU oracle itself (not only against fa_fwd): a key range long enough
    that the global rows' tiles are cut into chunks whose partial results live in the static array."""
    from flash_mi355 import _cabi
    from flash_mi355.api import _stream_ptr
    from oracle import attention_oracle as O
    L = _cabi.lib()
    dev = torch.device("cuda")
    B, H, M, N, D = 1, 2, 700, 2500, 128
    plan, o, lse = _problem(B, H, M, N, D, torch.bfloat16, 77)
    print(f"case static scratch against the oracle: B{B} H{H} M{M} N{N} D{D}", flush=True)
    _cabi.check(L.fa_fwd_static(ctypes.byref(plan.p), _stream_ptr(dev)), "fa_fwd_static")
    torch.cuda.synchronize()
    q, k, v, eq, ek = plan.keep[:5]
    ro, rl = O.attention_closed_form(q.cpu(), k.cpu(), v.cpu(), True, None, eq.cpu(), ek.cpu(), 1)[:2]
    dead = torch.isinf(rl)
    got_l = lse.cpu() * math.log(2.0)      # the C ABI stores log2 units (flash_triton.py:133)
    assert torch.equal(torch.isinf(got_l), dead)
    assert (got_l[~dead] - rl[~dead]).abs().max().item() <= 1e-3
    assert (o.float().cpu() - ro).abs().max().item() <= 2e-2


def test_static_scratch_allocates_nothing_and_replays_from_a_graph():
    """What the entry point is for.  (1) A warm call leaves the free device memory as it found it (no
    hipMalloc behind the caller's back, no torch allocation).  (2) It can be captured into a HIP graph:
    the first call on a device looks the static array's address up, so it is made BEFORE the capture
    (the documented order); the captured call is then replayed several times, with other eager work and
    synchronisations in between, on inputs that change between the replays, and every replay must give
    the eager result bit for bit (the plan kernels clear their counters themselves; no memset node)."""
    from flash_mi355 import _cabi
    from flash_mi355.api import _stream_ptr
    L = _cabi.lib()
    dev = torch.device("cuda")
    B, H, M, N, D = 1, 4, 600, 2300, 128
    plan, o, lse = _problem(B, H, M, N, D, torch.bfloat16, 91)
    p = plan.p
    q = plan.keep[0]
    print("case static scratch: memory and graph replay", flush=True)
    _cabi.check(L.fa_fwd_static(ctypes.byref(p), _stream_ptr(dev)), "fa_fwd_static")   # warm: address looked up
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info(dev)[0]
    reserved0 = torch.cuda.memory_reserved(dev)
    for _ in range(3):
        _cabi.check(L.fa_fwd_static(ctypes.byref(p), _stream_ptr(dev)), "fa_fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free0 and torch.cuda.memory_reserved(dev) == reserved0
    eager_o, eager_l = o.clone(), lse.clone()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _cabi.check(L.fa_fwd_static(ctypes.byref(p), _stream_ptr(dev)), "fa_fwd_static (captured)")
    q0 = q.clone()
    for rep in range(4):
        if rep % 2 == 1:
            q.copy_(q0.flip(2))             # other inputs in the same buffers
        else:
            q.copy_(q0)
        o.fill_(float("nan")); lse.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_l = o.clone(), lse.clone()
        o.fill_(float("nan")); lse.fill_(float("nan"))
        _cabi.check(L.fa_fwd_static(ctypes.byref(p), _stream_ptr(dev)), "fa_fwd_static")   # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got_o, o) and torch.equal(got_l, lse), rep
        if rep % 2 == 0:
            assert torch.equal(got_o, eager_o) and torch.equal(got_l, eager_l)


def test_static_scratch_refuses_what_does_not_fit():
    from flash_mi355 import _cabi
    from flash_mi355.api import _stream_ptr
    L = _cabi.lib()
    dev = torch.device("cuda")
    # per-head ids of a long sequence: the plan alone exceeds the static array
    B, H, M, D = 1, 64, 32768, 16
    q = torch.zeros(B, H, M, D, dtype=torch.bfloat16, device=dev)
    ids = torch.zeros(B, H, M, dtype=torch.int32, device=dev)
    from flash_mi355.api import _Plan, _set4
    plan = _Plan(q, q, q, True, 0.25, ids, ids, 1)
    o = torch.empty_like(q)
    lse = torch.empty(B, H, M, device=dev, dtype=torch.float32)
    plan.p.o, plan.p.lse = o.data_ptr(), lse.data_ptr()
    _set4(plan.p.o_stride, o)
    assert L.fa_workspace_plan_bytes(ctypes.byref(plan.p)) > _cabi.FA_STATIC_WS_BYTES
    rc = L.fa_fwd_static(ctypes.byref(plan.p), _stream_ptr(dev))
    assert rc == -8, rc   # FA_ERR_WORKSPACE
    with pytest.raises(_cabi.FlashMI355Error, match="workspace"):
        _cabi.check(rc, "fa_fwd_static")
