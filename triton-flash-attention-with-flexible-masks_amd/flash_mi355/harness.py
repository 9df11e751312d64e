"""Check-and-benchmark matrix in the shape of the reference's script (testing.py:156-243, 264-293):
for every (shape, causal, dtype) it compares the outputs and gradients of several attention
implementations against the first one and then times forward, backward and forward+backward,
printing the reference's two line formats

    Compare[<shape>,<causal>,<dtype>,<rid>,<mode>,<name>]: diff=[O, dQ, dK, dV max-abs]
    Throughput(tflops/s)[<shape>,<causal>,<dtype>,<mode>,<name>]: mean/max/min=[...]

Implementations (``--funcs``):
    torch   eager attention with an fp32 softmax (testing.py:32-47), on the GPU
    math    torch SDPA, math backend           (testing.py:49-56)
    mem     torch SDPA, memory-efficient backend
    flash   torch SDPA, flash backend (no arbitrary mask: reported as ERR with ids)
    mi355   this library (alias ``triton_triton``, the name the reference gives its kernels)

FLOP convention: testing.py:92-107 (dense-equivalent, x0.5 when causal, backward = 2.0 forward for
eager implementations and 2.5 for fused ones).  Timing: HIP events around single calls after a
warm-up, gradients reset between calls, median and 20 % / 80 % quantiles (what triton's
``do_bench(quantiles=[0.5, 0.2, 0.8])`` reports in the reference).

    python -m flash_mi355.harness --lens 1 2 4 8 16 --dim 128 --funcs mem math torch mi355
"""
from __future__ import annotations

import argparse
import math
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from .api import SCORE_FUNC_MODE1_DOC, attention

EAGER = ("math", "torch")


def attn_torch(q, k, v, is_causal: bool, attn_mask=None):
    """softmax(q k^T / sqrt(D) + mask) v with the softmax in fp32 (testing.py:32-47)."""
    D = q.shape[-1]
    s = torch.matmul(q, k.transpose(-1, -2)) * (D ** -0.5)
    Lq, Lk = s.shape[-2:]
    if is_causal:  # bottom-right aligned
        i = torch.arange(Lq, device=q.device)[:, None] + (Lk - Lq)
        j = torch.arange(Lk, device=q.device)[None, :]
        s = s.masked_fill(i < j, float("-inf"))
    if attn_mask is not None:
        s = s.masked_fill(~attn_mask, float("-inf"))
    p = torch.softmax(s.float(), dim=-1).to(q.dtype)
    return torch.matmul(p, v)


def _sdpa(backend_name: str) -> Callable:
    from torch.nn.attention import SDPBackend, sdpa_kernel
    backend = {"math": SDPBackend.MATH, "mem": SDPBackend.EFFICIENT_ATTENTION,
               "flash": SDPBackend.FLASH_ATTENTION}[backend_name]

    def run(q, k, v, is_causal: bool, attn_mask=None):
        with sdpa_kernel(backend):
            return torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=is_causal,
                                                                    attn_mask=attn_mask)
    return run


def attn_mi355(q, k, v, is_causal: bool, **kw):
    return attention(q, k, v, is_causal, q.shape[-1] ** -0.5, **kw)


def implementations() -> Dict[str, Callable]:
    return {"torch": attn_torch, "math": _sdpa("math"), "mem": _sdpa("mem"), "flash": _sdpa("flash"),
            "mi355": attn_mi355, "triton_triton": attn_mi355}


def attention_flops(shape: Sequence[int], is_causal: bool, mode: str, name: str) -> float:
    """testing.py:92-107."""
    B, H, L, D = shape
    total = 2 * (2.0 * B * H * L * L * D) * (0.5 if is_causal else 1.0)
    if mode == "fwd":
        return total
    f = total * (2.0 + (0.0 if name in EAGER else 0.5))
    return f + total if mode == "fb" else f


def sample_doc_ids(shape: Sequence[int], device, is_causal: bool, boundary_rate: float = 0.05):
    """Ids as the reference draws them (testing.py:110-120): a running document counter shifted so
    that the first third of the documents gets negative (local) ids and the rest ids >= 0 (global).
    Returns (eq, ek, boolean keep mask [B,1,L,L] with the causal part folded in)."""
    B, H, L, _ = shape
    ids = (torch.rand(B, L, device=device) <= boundary_rate).cumsum(-1)
    ids = ids - ids[:, -1:] // 3
    keep = ((ids[:, :, None] >= 0) | (ids[:, :, None] == ids[:, None, :]))[:, None]
    if is_causal:
        pos = torch.arange(L, device=device)
        keep = keep & (pos[:, None] >= pos[None, :])
    e = ids[:, None, :].expand(B, H, L)
    return e, e, keep


def _kwargs_for(name: str, is_causal: bool, ids) -> dict:
    if ids is None:
        return {"is_causal": is_causal}
    eq, ek, keep = ids
    if name in ("mi355", "triton_triton"):
        return {"is_causal": is_causal, "eq": eq, "ek": ek, "score_func_mode": SCORE_FUNC_MODE1_DOC}
    return {"is_causal": False, "attn_mask": keep}  # the mask already holds the causal part


def _time_ms(fn: Callable[[], None], grads: Sequence[torch.Tensor], warmup: int, reps: int) -> Tuple[float, float, float]:
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(reps):
        for t in grads:
            t.grad = None
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    qs = torch.quantile(torch.tensor(times), torch.tensor([0.5, 0.2, 0.8]))
    return tuple(qs.tolist())


def run_attn(func_names: Sequence[str], shape: Sequence[int], is_causal: bool, dtype: str, mask_doc: bool,
             check_times: int = 3, bench_times: int = 50, warmup_times: int = 10, device: str = "cuda"):
    """One (shape, causal, dtype) cell of the matrix; returns (check records, bench records)."""
    impls = implementations()
    tdt = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}[dtype]   # testing.py:158
    shape = list(shape)
    checks, benches = [], []
    if check_times > 0:
        print(f"# <<<<<\n# ===== Check correctness [{shape},{is_causal},{dtype}]")
    for rid in range(check_times):
        q, k, v = (torch.randn(shape, dtype=tdt, device=device, requires_grad=True) for _ in range(3))
        do = torch.randn(shape, dtype=tdt, device=device)
        ids = sample_doc_ids(shape, device, is_causal) if mask_doc else None
        ref = None
        for name in func_names:
            tag = f"Compare[{shape},{is_causal},{dtype},{rid},bwd,{name}]"
            try:
                out = impls[name](q, k, v, **_kwargs_for(name, is_causal, ids))
                out.backward(do)
                got = [t.detach().float().cpu() for t in (out, q.grad, k.grad, v.grad)]
                q.grad = k.grad = v.grad = None
                ref = got if ref is None else ref
                diffs = [(a - b).abs().max().item() for a, b in zip(ref, got)]
                print(f"{tag}: diff={diffs}")
            except Exception as e:  # an implementation that cannot run this cell is a result, not a failure
                diffs = [-1.0] * 4
                q.grad = k.grad = v.grad = None
                print(f"{tag}: ERR={e}")
            checks.append(({"shape": shape, "is_causal": is_causal, "dtype": dtype, "rid": rid, "mode": "bwd",
                            "func_name": name}, diffs))
    if bench_times > 0:
        print(f"# <<<<<\n# ===== Benchmark [{shape},{is_causal},{dtype}]")
        for mode in ("fwd", "bwd", "fb"):
            for name in func_names:
                tag = f"Throughput(tflops/s)[{shape},{is_causal},{dtype},{mode},{name}]"
                need_grad = mode != "fwd"
                try:
                    q, k, v = (torch.randn(shape, dtype=tdt, device=device, requires_grad=need_grad) for _ in range(3))
                    do = torch.randn(shape, dtype=tdt, device=device)
                    ids = sample_doc_ids(shape, device, is_causal) if mask_doc else None
                    kw = _kwargs_for(name, is_causal, ids)
                    f = impls[name]
                    if mode == "fwd":
                        fn = lambda: f(q, k, v, **kw)
                    elif mode == "bwd":
                        o = f(q, k, v, **kw)
                        fn = lambda: o.backward(do, retain_graph=True)
                    else:
                        fn = lambda: f(q, k, v, **kw).backward(do)
                    ms = _time_ms(fn, (q, k, v) if need_grad else (), warmup_times, bench_times)
                    flops = attention_flops(shape, is_causal, mode, name)
                    tf = [f"{flops / z * 1e-9:.2f}" for z in ms]
                    print(f"{tag}: mean/max/min={tf}")
                except Exception as e:
                    tf = (-1, -1, -1)
                    print(f"{tag}: ERR={e}")
                benches.append(({"shape": shape, "is_causal": is_causal, "dtype": dtype, "mode": mode,
                                 "func_name": name}, tf))
                q = k = v = do = ids = None
                torch.cuda.empty_cache()
    print("# >>>>> Finished")
    return checks, benches


def pivot(records, entry: Callable[[list], str]) -> str:
    """Rows 'Mode,C,F', columns 'L,D' (the labels of testing.py:248-249), as plain text."""
    rows: Dict[str, Dict[str, list]] = {}
    cols: List[str] = []
    for key, val in records:
        r = f"Mode={key['mode']},C={key['is_causal']},F={key['func_name']}"
        c = f"L={key['shape'][2]:02d},D={key['dtype']}"
        rows.setdefault(r, {}).setdefault(c, []).append(val)
        if c not in cols:
            cols.append(c)
    w = max(len(r) for r in rows) if rows else 0
    lines = [" " * w + "  " + "  ".join(f"{c:>22s}" for c in cols)]
    for r, d in rows.items():
        lines.append(f"{r:<{w}s}  " + "  ".join(f"{entry(d[c]) if c in d else '-':>22s}" for c in cols))
    return "\n".join(lines)


def _entry_check(vals) -> str:
    n = len(vals)
    mean = [sum(v[i] for v in vals) / n for i in range(len(vals[0]))]
    return f"({n})" + "/".join(f"{z:.4f}" for z in mean)


def _entry_bench(vals) -> str:
    return f"{float(vals[0][0]):.2f}"


def main(argv: Optional[Sequence[str]] = None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--funcs", nargs="+", default=["mem", "math", "torch", "mi355"])
    ap.add_argument("--lens", nargs="+", type=int, default=[1, 2, 4, 8, 16],
                    help="sequence lengths in units of 1024; batch = 16 // len (testing.py:272-276)")
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--dtypes", nargs="+", default=["bf16"])
    ap.add_argument("--causal", nargs="+", type=int, default=[0, 1])
    ap.add_argument("--no-doc", action="store_true", help="no document ids (plain / causal attention)")
    ap.add_argument("--check-times", type=int, default=1)
    ap.add_argument("--bench-times", type=int, default=100)
    ap.add_argument("--warmup-times", type=int, default=10)
    args = ap.parse_args(argv)
    checks, benches = [], []
    for L in args.lens:
        shape = [max(1, 16 // L), args.heads, 1024 * L, args.dim]
        for c in args.causal:
            for dt in args.dtypes:
                a, b = run_attn(args.funcs, shape, bool(c), dt, not args.no_doc, args.check_times,
                                args.bench_times, args.warmup_times)
                checks.extend(a)
                benches.extend(b)
    if checks:
        print(pivot(checks, _entry_check))
    if benches:
        print(pivot(benches, _entry_bench))


if __name__ == "__main__":
    main()
