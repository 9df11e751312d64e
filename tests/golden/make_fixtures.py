#!/usr/bin/env python3
"""Writes the small golden fixtures under tests/golden/*.npz.

The reference ships no vectors for this path (its check script only prints differences), so
these are produced by the CPU oracle (oracle/attention_oracle.py, fp64 explicit formulas) from
seeded inputs rounded to bf16/fp16.  They guard the oracle against regressions and give the GPU
tests fixed inputs with known answers.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))
from oracle import attention_oracle as O  # noqa: E402

CASES = {
    # name: (B, H, Hk, M, N, D, dtype, causal, doc)
    "tiny_doc_causal_bf16": (1, 2, 2, 32, 32, 16, torch.bfloat16, True, True),
    "rect_doc_causal_fp16": (1, 2, 2, 16, 48, 32, torch.float16, True, True),
    "gqa_doc_causal_bf16": (1, 4, 2, 40, 40, 64, torch.bfloat16, True, True),
    "plain_noncausal_bf16": (2, 2, 2, 24, 40, 32, torch.bfloat16, False, False),
    # block mask (64 x 64 blocks, drawn per head): "doc" is False, the map is stored as "block"
    "block_causal_bf16": (1, 2, 1, 150, 200, 32, torch.bfloat16, True, False),
}
BLOCK = {"block_causal_bf16"}


def make(name):
    B, H, Hk, M, N, D, dt, causal, doc = CASES[name]
    seed = sum(map(ord, name))
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    q = torch.randn(B, H, M, D, generator=g).to(dt)
    k = torch.randn(B, Hk, N, D, generator=g).to(dt)
    v = torch.randn(B, Hk, N, D, generator=g).to(dt)
    do = torch.randn(B, H, M, D, generator=g).to(dt)
    out = dict(q=q.float().numpy(), k=k.float().numpy(), v=v.float().numpy(), do=do.float().numpy(),
               causal=np.array(causal), doc=np.array(doc), dtype=np.array(str(dt)))
    eq = ek = None
    if doc:
        ekn = -(np.cumsum(rng.random((B, H, N)) < 0.12, axis=-1) + 1)
        ekn[rng.random((B, H, N)) < 0.1] = 0
        ek = torch.from_numpy(ekn.astype(np.int32))
        eq = ek[..., N - M:].contiguous()
        out.update(eq=eq.numpy(), ek=ek.numpy())
    mode = 1 if doc else 0
    if name in BLOCK:
        bm = rng.random((B, H, -(-M // 64), -(-N // 64))) < 0.6
        bm[:, 0, 1, :] = False   # a row of blocks without any key
        eq, mode = torch.from_numpy(bm), 2
        out.update(block=bm)
    o, lse, delta, dq, dk, dv = O.attention_grads(q, k, v, do, causal, None, eq, ek, mode)
    keep = np.broadcast_to(O.keep_mask(M, N, causal, None if eq is None else eq.numpy(),
                                       None if ek is None else ek.numpy(), mode), (B, H, M, N))
    out.update(o=o.numpy(), lse=lse.numpy(), delta=delta.numpy(), dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy(),
               keep=np.packbits(keep, axis=-1), keep_shape=np.array(keep.shape))
    np.savez_compressed(Path(__file__).parent / f"{name}.npz", **out)


if __name__ == "__main__":
    for n in (sys.argv[1:] or CASES):
        make(n)
        print("wrote", n)
