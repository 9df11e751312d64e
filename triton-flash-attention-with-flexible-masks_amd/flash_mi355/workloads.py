"""Seeded synthetic workloads for the benchmark and the parity tests, and the
FLOP accounting used to report throughput.

The five named configurations follow the benchmark definition of this project
(document ids: negative = attend inside the own document only, >= 0 = attend to
everything, the id semantics of the reference's sampler, testing.py:110-120).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np


@dataclass
class Workload:
    name: str
    B: int
    H: int
    Hk: int
    Lq: int
    Lk: int
    D: int
    dtype: str            # "bf16" | "fp16" | "fp32"
    causal: bool
    doc: bool
    eq: Optional[np.ndarray] = None   # [B, Lq] int32 (shared by all heads)
    ek: Optional[np.ndarray] = None   # [B, Lk] int32
    window: int = 0       # sliding window (causal only; 0 = off)
    prefix: int = 0       # prefix-LM (causal only; 0 = off)
    block: Optional[np.ndarray] = None   # [B, ceil(Lq/64), ceil(Lk/64)] bool: block mask shared by all heads (excludes eq / ek)


def _pack_docs(rng, L, draw_len):
    """ids -(doc+1) for documents packed back to back until L tokens are covered."""
    ids = np.empty(L, dtype=np.int32)
    pos, doc = 0, 0
    while pos < L:
        n = int(draw_len(rng))
        ids[pos:pos + n] = -(doc + 1)
        pos += n
        doc += 1
    return ids


def _globalise(rng, ids, frac):
    ids = ids.copy()
    ids[rng.random(ids.shape[0]) < frac] = 0
    return ids


def doc_ids_uniform(rng, L, lo, hi, global_frac):
    return _globalise(rng, _pack_docs(rng, L, lambda r: r.integers(lo, hi + 1)), global_frac)


def doc_ids_geometric(rng, L, mean, minimum, global_frac):
    p = 1.0 / max(1.0, mean - minimum + 1)
    return _globalise(rng, _pack_docs(rng, L, lambda r: minimum - 1 + r.geometric(p)), global_frac)


def make_workload(name: str, seed: int = 0) -> Workload:
    rng = np.random.default_rng(seed)
    if name == "cfg1_cpu_doc_causal":
        B, H, L, D = 2, 4, 512, 64
        ids = np.stack([doc_ids_uniform(rng, L, 32, 256, 0.05) for _ in range(B)])
        return Workload(name, B, H, H, L, L, D, "fp32", True, True, ids, ids)
    if name == "cfg2_plain":
        return Workload(name, 4, 16, 16, 2048, 2048, 64, "bf16", False, False)
    if name == "cfg3_doc_causal_4k":
        B, H, L, D = 2, 32, 4096, 128
        ids = np.stack([doc_ids_uniform(rng, L, 128, 1024, 0.10) for _ in range(B)])
        return Workload(name, B, H, H, L, L, D, "bf16", True, True, ids, ids)
    if name == "cfg4_doc_causal_16k":
        B, H, L, D = 1, 32, 16384, 128
        ids = np.stack([doc_ids_geometric(rng, L, 512, 16, 0.02) for _ in range(B)])
        return Workload(name, B, H, H, L, L, D, "bf16", True, True, ids, ids)
    if name == "cfg5_rect_fp16":
        B, H, Lq, Lk, D = 8, 8, 1024, 8192, 128
        ek = np.repeat(-(np.arange(32, dtype=np.int32) + 1), Lk // 32)          # 32 docs of 256 keys
        ek = np.broadcast_to(ek, (B, Lk)).copy()
        eq = np.stack([_globalise(rng, ek[b, -Lq:], 0.05) for b in range(B)])   # the last 4 docs
        return Workload(name, B, H, H, Lq, Lk, D, "fp16", True, True, eq, ek)
    if name == "block25_causal_16k":    # block-sparse: the diagonal blocks and a quarter of the others, under a causal mask
        L = 16384
        blk = rng.random((1, L // 64, L // 64)) < 0.25
        blk |= np.eye(L // 64, dtype=bool)[None]
        return Workload(name, 1, 32, 32, L, L, 128, "bf16", True, False, block=blk)
    if name == "window1k_causal_16k":   # sliding window of 1024 keys over 16K tokens
        return Workload(name, 1, 32, 32, 16384, 16384, 128, "bf16", True, False, window=1024)
    if name == "fp32_causal_4k":     # the fp32 kernels at a size that fills the chip
        return Workload(name, 1, 32, 32, 4096, 4096, 128, "fp32", True, False)
    if name == "plain_causal_16k":   # no ids: the dense efficiency of the same kernels
        return Workload(name, 1, 32, 32, 16384, 16384, 128, "bf16", True, False)
    raise KeyError(name)


WORKLOADS = ("cfg1_cpu_doc_causal", "cfg2_plain", "cfg3_doc_causal_4k", "cfg4_doc_causal_16k", "cfg5_rect_fp16")


def keep_rows(w: Workload, b: int, i0: int, i1: int) -> np.ndarray:
    """keep(i, j) for rows i0..i1 of batch b as a bool array [i1-i0, Lk]."""
    i = np.arange(i0, i1, dtype=np.int64)[:, None]
    j = np.arange(w.Lk, dtype=np.int64)[None, :]
    keep = np.ones((i1 - i0, w.Lk), dtype=bool)
    if w.causal:
        gap = max(0, w.Lk - w.Lq)
        c = (gap + i) >= j
        if w.prefix:
            c |= j < w.prefix
        if w.window:
            c &= j > gap + i - w.window
        keep &= c
    if w.doc:
        e_q = w.eq[b, i0:i1].astype(np.int64)[:, None]
        e_k = w.ek[b].astype(np.int64)[None, :]
        keep &= (e_q >= 0) | (e_q == e_k)
    if w.block is not None:
        keep &= w.block[b][(i // 64), (j // 64)]
    return keep


def count_mask(w: Workload, tile: int = 128):
    """(kept elements, non-empty canonical tile x tile tiles, all tiles) summed over the batch
    (ids are shared by the heads, so per-head counts are these numbers)."""
    kept = tiles = 0
    n_tiles_k = (w.Lk + tile - 1) // tile
    for b in range(w.B):
        for i0 in range(0, w.Lq, tile):
            k = keep_rows(w, b, i0, min(w.Lq, i0 + tile))
            kept += int(k.sum())
            col_any = k.any(axis=0)
            pad = n_tiles_k * tile - w.Lk
            if pad:
                col_any = np.concatenate([col_any, np.zeros(pad, bool)])
            tiles += int(col_any.reshape(n_tiles_k, tile).any(axis=1).sum())
    total_tiles = w.B * ((w.Lq + tile - 1) // tile) * n_tiles_k
    return kept, tiles, total_tiles


def flops(w: Workload, mode: str = "fwd", kept=None, tiles=None, tile: int = 128):
    """FLOP counts under the three conventions used in the reports.

    dense : 4*B*H*Lq*Lk*D, halved when causal (testing.py:94-98; exact bottom-right
            count for rectangular shapes)
    elem  : 4*D*H*#kept elements
    tile  : 4*D*H*tile^2*#canonical tiles with at least one kept element
    backward = 2.5 x forward, forward+backward = 3.5 x (testing.py:103-105).
    """
    if kept is None or tiles is None:
        kept, tiles, _ = count_mask(w, tile)
    mult = {"fwd": 1.0, "bwd": 2.5, "fb": 3.5}[mode]
    dense_pairs = w.Lq * w.Lk
    if w.causal:
        gap = max(0, w.Lk - w.Lq)
        dense_pairs = w.Lq * gap + w.Lq * (w.Lq + 1) // 2 if w.Lq != w.Lk else w.Lq * w.Lk / 2
    return {
        "dense": 4.0 * w.B * w.H * dense_pairs * w.D * mult,
        "elem": 4.0 * w.D * w.H * kept * mult,
        "tile": 4.0 * w.D * w.H * tile * tile * tiles * mult,
    }


# ---------------------------------------------------------------------------
# Executed work: a host emulation of the tile decisions the kernels take (mask plan,
# permuted order, per-wave skip tests), so that reports can state the FLOPs the MFMA
# pipes really execute next to the algorithmic (mask-derived) counts.
# ---------------------------------------------------------------------------
_IMAX, _IMIN = 2**31 - 1, -2**31


def _summaries(ids, rows, n):
    """Per group of n entries of `rows` (row indices, -1 = none): lo/hi over local ids, glob, rmin, rmax."""
    G = len(rows) // n
    r = rows.reshape(G, n)
    valid = r >= 0
    v = np.where(valid, ids[np.maximum(r, 0)], 0)
    local = valid & (v < 0)
    lo = np.where(local, v, _IMAX).min(1)
    hi = np.where(local, v, _IMIN).max(1)
    glob = (valid & (v >= 0)).any(1)
    rmin = np.where(valid, r, _IMAX).min(1)
    rmax = np.where(valid, r, -1).max(1)
    return lo, hi, glob, rmin, rmax, valid.sum(1)


def executed_wave_steps(w: Workload):
    """(forward/dq wave steps, dk/dv wave steps) per head, summed over the batch.

    A forward (or dq) wave step is 32 query rows x 64 keys; a dk/dv wave step is 64 query rows x
    32 keys.  Both cover 2048 score elements, i.e. 2048 * 4 * D FLOPs in the forward.
    """
    gap = max(0, w.Lk - w.Lq)
    win = w.window if w.window else 2**30
    pfx_m1 = min(w.prefix, w.Lk) - 1 if w.prefix else -1
    fwd_steps = kv_steps = 0
    nK64 = (w.Lk + 63) // 64
    nK32 = (w.Lk + 31) // 32
    for b in range(w.B):
        if w.doc:
            eq = w.eq[b].astype(np.int64)
            ek = w.ek[b].astype(np.int64)
            local = np.nonzero(eq < 0)[0]
            glob = np.nonzero(eq >= 0)[0]
            nLp = (len(local) + 255) // 256 * 256
            Pp = (w.Lq + 255) // 256 * 256 + 256
            perm = np.full(Pp, -1, np.int64)
            perm[:len(local)] = local
            perm[nLp:nLp + len(glob)] = glob
        else:
            eq = np.zeros(w.Lq, np.int64)         # every row "global": no doc test
            ek = np.zeros(w.Lk, np.int64)
            Pp = (w.Lq + 127) // 128 * 128
            perm = np.where(np.arange(Pp) < w.Lq, np.arange(Pp), -1)
        pad = lambda x, n, fill: np.concatenate([x, np.full(n - len(x), fill, x.dtype)])
        k64 = pad(ek, nK64 * 64, 0).reshape(nK64, 64)
        kvalid64 = (np.arange(nK64 * 64).reshape(nK64, 64) < w.Lk)
        k64_lo = np.where(kvalid64, k64, _IMAX).min(1)
        k64_hi = np.where(kvalid64, k64, _IMIN).max(1)
        # forward / dq: waves of 32 rows against key tiles of 64
        lo, hi, g, rmin, rmax, nv = _summaries(eq, perm, 32)
        j0 = np.arange(nK64)[None, :] * 64
        vis = np.broadcast_to(nv[:, None] > 0, (len(nv), nK64)).copy()
        if w.causal:
            vis = vis & (j0 <= np.maximum(gap + rmax[:, None], pfx_m1)) & (j0 + 63 >= gap + rmin[:, None] - win + 1)
        if w.doc:
            vis = vis & (g[:, None] | ((lo[:, None] <= k64_hi[None, :]) & (k64_lo[None, :] <= hi[:, None])))
        if w.block is not None:   # a wave's 32 rows lie inside one row of blocks, a key tile is one column
            nW = len(nv)
            vis = vis & w.block[b][np.minimum(np.arange(nW) // 2, w.block.shape[1] - 1)][:, :nK64] & (np.arange(nW) // 2 < w.block.shape[1])[:, None]
        fwd_steps += int(vis.sum())
        # dk/dv: waves of 32 keys against query tiles of 64 (permuted order)
        k32 = pad(ek, nK32 * 32, 0).reshape(nK32, 32)
        kvalid32 = (np.arange(nK32 * 32).reshape(nK32, 32) < w.Lk)
        k32_lo = np.where(kvalid32, k32, _IMAX).min(1)
        k32_hi = np.where(kvalid32, k32, _IMIN).max(1)
        perm64 = pad(perm, (len(perm) + 63) // 64 * 64, -1)
        lo, hi, g, rmin, rmax, nv = _summaries(eq, perm64, 64)
        n0 = np.arange(nK32)[None, :] * 32
        vis = np.broadcast_to(nv[:, None] > 0, (len(nv), nK32)).copy()
        if w.causal:
            vis = vis & ((gap + rmax[:, None] >= n0) | (n0 <= pfx_m1)) & (gap + rmin[:, None] - win + 1 <= n0 + 31)
        if w.doc:
            vis = vis & (g[:, None] | ((lo[:, None] <= k32_hi[None, :]) & (k32_lo[None, :] <= hi[:, None])))
        if w.block is not None:   # a query tile is one row of blocks, a wave's 32 keys lie inside one column
            nT = len(nv)
            vis = vis & w.block[b][np.minimum(np.arange(nT), w.block.shape[1] - 1)][:, np.arange(nK32) // 2] & (np.arange(nT) < w.block.shape[1])[:, None]
        kv_steps += int(vis.sum())
    return fwd_steps, kv_steps


def executed_flops(w: Workload):
    """FLOPs the MFMA pipes execute per kernel: forward (2 GEMMs), dq (3), dk/dv (4)."""
    f, kv = executed_wave_steps(w)
    unit = 2048 * 4.0 * w.D * w.H     # one wave step, forward accounting
    return {"fwd": f * unit, "dq": 1.5 * f * unit, "dkdv": 2.0 * kv * unit}
