#!/usr/bin/env python3
"""Benchmark of the flexible-mask attention operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

A step is one forward + backward pass of the drop-in operator
(``attention(...)`` then ``.backward(dO)``) over one batch of the workload, with
every input already resident in HBM.  Default workload: the headline
configuration (bf16, causal + document mask, B=1 H=32 L=16384 D=128).

One JSON line is printed.  ``value`` is forward+backward throughput in TFLOP/s
under the tile-effective convention: 4*D*128*128 FLOPs for every canonical
128x128 tile of the score matrix that holds at least one kept element, times 3.5
for forward + backward (the reference's own accounting, testing.py:94-108, minus
the tiles the mask empties).  Dense-equivalent and element-effective figures,
forward and backward separately, are in ``detail``.

``roofline`` is for the longest-running kernel of the step: the FLOPs its MFMA
instructions execute (host emulation of the kernels' tile decisions; equals the
hardware's MFMA operation count) over its mean duration measured with HIP events
on the launch stream, against the 2.5 PFLOP/s bf16 MFMA peak -- a fraction of what
the matrix pipes can do, never above 1.  The mask plan lets the kernels skip most
canonical tiles, so the tile-effective rate of the same launch (what ``value``
counts) is higher and is reported beside it.  ``pct_of_mfma_peak`` is the executed
rate of the whole step; ``pct_of_mfma_peak_tile_effective`` the north-star figure.
``roofline.sustained_mfma_probe`` is what a bare MFMA loop on random bf16 operands sustains on the same box
right after the timed region (``frac_of_sustained`` = achieved over that): context only, ``frac`` is what counts.
``cpu_baseline`` times the reference's eager mask-materialising path on the host
cores for a bounded sample (a few heads) of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "triton-flash-attention-with-flexible-masks_amd"))

PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp32": 157.3}   # MI355X dense MFMA peaks
PEAK_HBM_GBS = 8000.0   # MI355X HBM3E
HBM_PEAK_GBS = 8000.0

KERNEL_OF = {"fa_fwd": "fwd_kernel", "fa_bwd_dq": "bwd_dq_kernel", "fa_bwd_dkdv": "bwd_dkdv_kernel"}


def profiled_traffic(workload, entry):
    """HBM bytes per launch of a kernel as the committed counter profile of this workload states them
    (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by a copy of known size; the commands are in
    the file).  This run does not measure traffic: the figure is quoted together with its source, or
    (None, None) when there is no profile of the workload."""
    import re
    path = ROOT / "profiles" / f"kernel_stats_{workload}.md"
    if not path.exists():
        return None, None
    text = path.read_text()
    if "## HBM traffic per launch" not in text:
        return None, None
    for row in text.split("## HBM traffic per launch")[1].splitlines():
        cells = [c.strip() for c in row.split("|")]
        if len(cells) >= 8 and KERNEL_OF[entry] in cells[1]:
            try:
                read_gb, written_gb = float(cells[3]), float(cells[6])
            except ValueError:
                continue
            return int(round((read_gb + written_gb) * 1e9)), f"profiles/{path.name}"
    return None, None


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg4_doc_causal_16k")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-heads", type=int, default=2, help="(batch, head) slices timed on the CPU")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch plain device copies of 1 GiB: the reference point that scales "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE readings to bytes")
    ap.add_argument("--only-headline", action="store_true", help="skip the short measurements of the other configurations")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="instead of the benchmark: print the sustained bf16 MFMA rate of the chip (a bare MFMA loop "
                         "with small-integer and with random operands, libfa_probe.so), four launches each")
    ap.add_argument("--wg-trace", action="store_true",
                    help="instead of the benchmark: launch forward, dQ and dK/dV of the workload from the clock-stamp "
                         "build (libflash_mi355_trace.so) and print where the workgroups spend their time")
    return ap.parse_args()


def make_inputs(w, torch):
    dt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[w.dtype]
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    q = torch.randn(w.B, w.H, w.Lq, w.D, device=dev, generator=g).to(dt)
    k = torch.randn(w.B, w.Hk, w.Lk, w.D, device=dev, generator=g).to(dt)
    v = torch.randn(w.B, w.Hk, w.Lk, w.D, device=dev, generator=g).to(dt)
    do = torch.randn(w.B, w.H, w.Lq, w.D, device=dev, generator=g).to(dt)
    eq = ek = None
    if w.doc:  # ids shared by the heads, passed head-expanded as the reference harness does (testing.py:118)
        eq = torch.from_numpy(w.eq).to(dev)[:, None, :].expand(w.B, w.H, w.Lq)
        ek = torch.from_numpy(w.ek).to(dev)[:, None, :].expand(w.B, w.H, w.Lk)
    if w.block is not None:   # block mask: the byte map travels in the place of eq (score mode 2)
        eq = ek = torch.from_numpy(w.block).to(dev)[:, None].expand(w.B, w.H, *w.block.shape[1:]).to(torch.uint8)
    return q, k, v, do, eq, ek


def time_kernels(w, q, k, v, do, eq, ek, torch, iters=20, warm=5):
    """Duration (ms) of every kernel of the step, each launched alone through the C ABI, `iters` launches
    back to back after `warm` untimed ones with a HIP event on the launch stream between any two
    (the method of testing.py:140-152).  Returns the means and, under "_quantiles", (p20, median, p80)."""
    from flash_mi355 import _cabi
    from flash_mi355.api import _Plan, _set4, _stream_ptr
    L = _cabi.lib()
    dev = q.device
    plan = _Plan(q, k, v, w.causal, 1.0 / math.sqrt(w.D), eq, ek, 1 if w.doc else (2 if w.block is not None else 0), w.window, w.prefix)
    p = plan.p
    o = torch.empty_like(q)
    lse = torch.empty(w.B, w.H, w.Lq, device=dev, dtype=torch.float32)
    delta = torch.empty_like(lse)
    dq = torch.empty_like(q)
    dk = torch.empty(w.B, w.Hk, w.Lk, w.D, device=dev, dtype=q.dtype)
    dv = torch.empty_like(dk)
    p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
    p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    for f, t in (("o_stride", o), ("do_stride", do), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
        _set4(getattr(p, f), t)
    plan.ensure_workspace(dev)
    stream = _stream_ptr(dev)
    ref = ctypes.byref(p)
    out = {}
    # the launches of the operator's backward: dq forms delta itself, then dk/dv (as api.py asks for)
    p.flags = _cabi.FA_FLAG_DQ_DELTA
    names = [("fa_fwd", L.fa_fwd), ("fa_bwd_dq", L.fa_bwd_dq), ("fa_bwd_dkdv", L.fa_bwd_dkdv)]
    if w.doc:
        names.insert(0, ("fa_mask_plan", L.fa_mask_plan))
    quant = {}
    for name, fn in names:
        for _ in range(warm):
            _cabi.check(fn(ref, stream), name)
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1)]
        ev[0].record()
        for i in range(iters):
            fn(ref, stream)
            ev[i + 1].record()
        ev[-1].synchronize()
        ts = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(iters))
        out[name] = ev[0].elapsed_time(ev[-1]) / iters
        quant[name] = [round(ts[int(f * (iters - 1))], 4) for f in (0.2, 0.5, 0.8)]
    out["_quantiles"] = quant
    return out


def wg_trace(w, q, k, v, do, eq, ek, torch):
    """Per-workgroup timeline of the three kernels from the clock-stamp build: every workgroup notes the
    100 MHz wall clock at a handful of points; this reads the stamps of one launch (after warm ones) and
    reduces them to means.  "mean_resident_per_cu" is the summed workgroup lifetime over span x 256 CUs."""
    import numpy as np
    from flash_mi355 import _cabi
    from flash_mi355.build import TRACE_LIB_PATH
    assert _cabi._lib is None, "the trace build must be the first library loaded"
    _cabi.LIB_PATH = TRACE_LIB_PATH
    L = _cabi.lib()
    L.fa_trace_read.restype = ctypes.c_int
    L.fa_trace_read.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int]
    from flash_mi355.api import _Plan, _set4, _stream_ptr
    dev = q.device
    plan = _Plan(q, k, v, w.causal, 1.0 / math.sqrt(w.D), eq, ek, 1 if w.doc else (2 if w.block is not None else 0), w.window, w.prefix)
    p = plan.p
    o = torch.empty_like(q)
    lse = torch.empty(w.B, w.H, w.Lq, device=dev, dtype=torch.float32)
    delta = torch.empty_like(lse)
    dq = torch.empty_like(q)
    dk = torch.empty(w.B, w.Hk, w.Lk, w.D, device=dev, dtype=q.dtype)
    dv = torch.empty_like(dk)
    p.o, p.lse, p.dout, p.delta = o.data_ptr(), lse.data_ptr(), do.data_ptr(), delta.data_ptr()
    p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    for f, t in (("o_stride", o), ("do_stride", do), ("dq_stride", dq), ("dk_stride", dk), ("dv_stride", dv)):
        _set4(getattr(p, f), t)
    plan.ensure_workspace(dev)
    stream = _stream_ptr(dev)
    ref = ctypes.byref(p)
    p.flags = _cabi.FA_FLAG_DQ_DELTA
    if w.doc:
        _cabi.check(L.fa_mask_plan(ref, stream), "fa_mask_plan")
    TICK_US = 0.01   # the wall clock of the stamps runs at 100 MHz
    out = {}
    # columns of the stamps: (start, set-up done, loop done, end, tiles, info)
    for which, (name, fn, cols) in enumerate((("fa_fwd", L.fa_fwd, (0, 2, 3, 4, 5, 7)),
                                              ("fa_bwd_dq", L.fa_bwd_dq, (0, 2, 3, 4, 5, 7)),
                                              ("fa_bwd_dkdv", L.fa_bwd_dkdv, (0, 3, 4, 5, 6, 7)))):
        for _ in range(16):   # the stamps of the last launch stay; the earlier ones bring the clock to its level under this kernel
            _cabi.check(fn(ref, stream), name)
        torch.cuda.synchronize()
        buf = np.zeros(8 * 65536, dtype=np.int64)
        rc = L.fa_trace_read(which, buf.ctypes.data, buf.size)
        assert rc == 0, f"fa_trace_read({which}) returned {rc}"
        t = buf.reshape(-1, 8)
        t = t[t[:, 0] != 0]
        c_start, c_setup, c_loop, c_end, c_tiles, c_info = cols
        left = t[:, c_info] == -1
        live = t[~left & (t[:, c_end] != 0) & (t[:, c_tiles] > 0)]
        idle = t[~left & (t[:, c_end] != 0) & (t[:, c_tiles] == 0)]
        span = (t[:, c_end].max() - t[:, 0].min()) * TICK_US
        life = (live[:, c_end] - live[:, c_start]) * TICK_US
        r = {
            "workgroups": int(len(t)), "left_at_once": int(left.sum()), "no_tiles": int(len(idle)),
            "with_tiles": int(len(live)),
            "span_us": round(float(span), 1),
            "mean_lifetime_us": round(float(life.mean()), 2),
            "mean_setup_us": round(float(((live[:, c_setup] - live[:, c_start]) * TICK_US).mean()), 2),
            "mean_loop_us": round(float(((live[:, c_loop] - live[:, c_setup]) * TICK_US).mean()), 2),
            "mean_drain_us": round(float(((live[:, c_end] - live[:, c_loop]) * TICK_US).mean()), 2),
            "mean_tiles": round(float(live[:, c_tiles].mean()), 2),
            "max_tiles": int(live[:, c_tiles].max()),
            "max_lifetime_us": round(float(life.max()), 1),
            "last_start_us": round(float((t[:, c_start].max() - t[:, 0].min()) * TICK_US), 1),
            "loop_us_per_tile": round(float((live[:, c_loop] - live[:, c_setup]).sum() * TICK_US / live[:, c_tiles].sum()), 3),
            "mean_resident_per_cu": round(float(life.sum() / (span * 256)), 3),
        }
        if which < 2:   # the workgroups that merged the chunks of a split tile: their drain in two parts
            mg = live[live[:, 6] != 0]
            if len(mg):
                r["merging_workgroups"] = int(len(mg))
                r["mean_store_and_arrive_us"] = round(float(((mg[:, 6] - mg[:, c_loop]) * TICK_US).mean()), 2)
                r["mean_merge_us"] = round(float(((mg[:, c_end] - mg[:, 6]) * TICK_US).mean()), 2)
                r["mean_chunks_merged"] = round(float(((mg[:, 7] >> 24) & 0xff).mean()), 2)
        if which == 2 and live[:, 1].any():   # role-split dk/dv: what its first gradient wave waits for the score wave's P
            r["mean_pair_wait_shader_clocks"] = round(float(live[:, 1].mean()), 0)
            r["mean_pair_wait_clocks_per_tile"] = round(float(live[:, 1].sum() / live[:, c_tiles].sum()), 1)
        if which == 2 and ((t[:, c_info] >> 40) == 1).any():   # workgroups of the column form share the launch: both kinds apart
            for key, sel in (("general_form", (live[:, c_info] >> 40) != 1), ("column_form", (live[:, c_info] >> 40) == 1)):
                x = live[sel]
                r[key] = {"workgroups": int(len(x)),
                          "mean_lifetime_us": round(float(((x[:, c_end] - x[:, c_start]) * TICK_US).mean()), 2),
                          "mean_setup_us": round(float(((x[:, c_setup] - x[:, c_start]) * TICK_US).mean()), 2),
                          "mean_loop_us": round(float(((x[:, c_loop] - x[:, c_setup]) * TICK_US).mean()), 2),
                          "mean_tiles": round(float(x[:, c_tiles].mean()), 2),
                          "first_start_us": round(float((x[:, c_start].min() - t[:, 0].min()) * TICK_US), 1),
                          "last_end_us": round(float((x[:, c_end].max() - t[:, 0].min()) * TICK_US), 1)}
        if len(idle):
            r["mean_lifetime_no_tiles_us"] = round(float(((idle[:, c_end] - idle[:, c_start]) * TICK_US).mean()), 2)
        out[name] = r
    return out


def measure_other_config(name, torch, steps=20, warmup=5):
    """One short operator-level measurement (forward + backward per step) of another benchmark configuration,
    same accounting as the headline line."""
    from flash_mi355 import attention, workloads as W
    w = W.make_workload(name)
    q, k, v, do, eq, ek = make_inputs(w, torch)
    mode = 1 if w.doc else (2 if w.block is not None else 0)
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)

    def step():
        q.grad = k.grad = v.grad = None
        attention(q, k, v, w.causal, 1.0 / math.sqrt(w.D), eq, ek, mode, window=w.window, prefix=w.prefix).backward(do)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    kept, tiles, _ = W.count_mask(w)
    f = W.flops(w, "fb", kept, tiles)
    ex = W.executed_flops(w) if w.dtype != "fp32" else None   # the emulation follows the 16-bit kernels' tiling
    out = {"dtype": w.dtype, "shape": [w.B, w.H, w.Lq, w.Lk, w.D], "causal": w.causal, "doc_mask": w.doc, "steps": steps,
           "ms_per_step": round(ms, 4), "tflops_tile_effective": round(f["tile"] / ms * 1e-9, 1),
           "tflops_dense_equivalent": round(f["dense"] / ms * 1e-9, 1)}
    if ex is not None:
        out["tflops_executed"] = round((ex["fwd"] + ex["dq"] + ex["dkdv"]) / ms * 1e-9, 1)
        out["pct_of_mfma_peak"] = round(100 * out["tflops_executed"] / PEAK_TFLOPS[w.dtype], 2)
    # The other roof: the bytes a step cannot avoid (every operand and result of the three kernels once:
    # forward Q K V -> O; dq Q K V dO O -> dQ; dk/dv Q dO K V -> dK dV) over the 8 TB/s HBM peak.  For a
    # configuration whose few global rows make every head stream all of K and V (cfg5) this, not the MFMA
    # share, says how far the step is from its bound.
    es = 4 if w.dtype == "fp32" else 2
    nq, nk = w.B * w.H * w.Lq * w.D * es, w.B * w.Hk * w.Lk * w.D * es
    gb = ((2 * nq + 2 * nk) + (4 * nq + 2 * nk) + (2 * nq + 4 * nk)) * 1e-9
    out["hbm_gb_min"] = round(gb, 3)
    out["pct_of_hbm_peak"] = round(100 * gb / (ms * 1e-3) / (PEAK_HBM_GBS), 2)
    return out


def cpu_baseline(w, heads, torch):
    """The reference's eager path (testing.py:32-47) on the host cores for `heads` (b, h) slices."""
    from oracle import attention_oracle as O
    from flash_mi355 import workloads as W
    cores = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    n = min(heads, w.B * w.H)
    t_total = 0.0
    for s in range(n):
        b = s % w.B
        q = torch.randn(1, 1, w.Lq, w.D, generator=g).requires_grad_(True)
        k = torch.randn(1, 1, w.Lk, w.D, generator=g).requires_grad_(True)
        v = torch.randn(1, 1, w.Lk, w.D, generator=g).requires_grad_(True)
        do = torch.randn(1, 1, w.Lq, w.D, generator=g)
        keep = None
        if w.doc:
            e_q = torch.from_numpy(w.eq[b])[:, None]
            e_k = torch.from_numpy(w.ek[b])[None, :]
            keep = ((e_q >= 0) | (e_q == e_k))[None, None]
        t0 = time.perf_counter()
        out = O.eager_attention_cpu(q, k, v, w.causal, keep)
        out.backward(do)
        t_total += time.perf_counter() - t0
        del out, q, k, v, keep
    per_slice = t_total / n
    # dense-equivalent FLOPs with the x2.0 backward factor the reference applies to eager paths (testing.py:103)
    f = W.flops(w, "fwd", kept=0, tiles=0)["dense"] / (w.B * w.H)
    return {
        "value": round(3.0 * f / per_slice * 1e-12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"{n} of {w.B * w.H} (batch, head) slices of {w.name}, fp32 eager fwd+bwd, "
                  f"{per_slice:.2f} s per slice (dense-equivalent FLOPs, backward x2.0)",
        "seconds_per_slice": round(per_slice, 3),
        "extrapolated_step_seconds": round(per_slice * w.B * w.H, 1),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this operator shards over (batch, head) with no "
              "communication and this build uses a single GPU; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.mfma_probe:
        from flash_mi355.build import PROBE_LIB_PATH
        probe = ctypes.CDLL(str(PROBE_LIB_PATH))
        probe.fa_probe_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
        out = {}
        for label, rnd in (("small_integers", 0), ("random_bf16", 1)):
            rates = []
            for _ in range(4):
                tf_ = ctypes.c_float(0)
                rc = probe.fa_probe_mfma_rate(rnd, 40000, ctypes.byref(tf_))
                assert rc == 0, f"probe failed with hipError {rc}"
                rates.append(round(tf_.value, 1))
            out[label] = rates
        # the forward's phase structure without memory: ns per round, and the rate that is for a 128 x 64 x 128 tile per workgroup
        probe.fa_probe_phase_time.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
        phase = {}
        for label, wgs, soft in (("mfma_only_1wg", 1, 0), ("mfma_only_2wg", 2, 0), ("with_softmax_1wg", 1, 1), ("with_softmax_2wg", 2, 1)):
            ns = ctypes.c_float(0)
            rc = probe.fa_probe_phase_time(wgs, soft, 20000, ctypes.byref(ns))
            assert rc == 0, f"probe failed with hipError {rc}"
            phase[label] = {"ns_per_round": round(ns.value, 1),
                            "tflops": round(256 * wgs * 4 * 32 * 32768.0 / ns.value * 1e-3, 1)}
        print(json.dumps({"probe": "v_mfma_f32_32x32x16_bf16, 8 workgroups of 4 waves per CU, 4 accumulators per wave",
                          "tflops": out, "datasheet_peak": PEAK_TFLOPS["bf16"],
                          "forward_phase_structure_without_memory": phase}))
        return
    import torch
    from flash_mi355 import attention, workloads as W

    w = W.make_workload(args.workload)
    q, k, v, do, eq, ek = make_inputs(w, torch)
    if args.wg_trace:
        print(json.dumps({"workload": w.name, "clock": "100 MHz wall clock, the last of 16 launches",
                          "kernels": wg_trace(w, q, k, v, do, eq, ek, torch)}))
        return
    mode = 1 if w.doc else (2 if w.block is not None else 0)
    scale = 1.0 / math.sqrt(w.D)
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)

    def step():
        q.grad = k.grad = v.grad = None
        out = attention(q, k, v, w.causal, scale, eq, ek, mode, window=w.window, prefix=w.prefix)
        out.backward(do)

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    kept, tiles, total_tiles = W.count_mask(w)
    f_fwd = W.flops(w, "fwd", kept, tiles)
    kt = time_kernels(w, q.detach(), k.detach(), v.detach(), do, eq, ek, torch)
    t_fwd = kt["fa_fwd"] + kt.get("fa_mask_plan", 0.0)
    t_bwd = kt.get("fa_bwd_delta", 0.0) + kt["fa_bwd_dkdv"] + kt["fa_bwd_dq"]
    peak = PEAK_TFLOPS[w.dtype]

    def tf(flops, ms):
        return flops / ms * 1e-9

    quantiles = kt.pop("_quantiles")
    detail = {"ms": {n: round(t, 4) for n, t in kt.items()}, "ms_p20_p50_p80": quantiles,
              "tiles_nonempty": tiles, "tiles_total": total_tiles,
              "kept_fraction": round(kept / (w.B * w.Lq * w.Lk), 5)}
    for conv in ("tile", "dense", "elem"):
        detail[f"fwd_tflops_{conv}"] = round(tf(f_fwd[conv], t_fwd), 1)
        detail[f"bwd_tflops_{conv}"] = round(tf(2.5 * f_fwd[conv], t_bwd), 1)
    detail["fwd_pct_peak_tile"] = round(100 * detail["fwd_tflops_tile"] / peak, 2)
    detail["bwd_pct_peak_tile"] = round(100 * detail["bwd_tflops_tile"] / peak, 2)

    # Roofline of the longest kernel.  `achieved` counts the FLOPs the kernel's MFMA instructions execute:
    # 2 * 32*32*16 per v_mfma_f32_32x32x16 over the 32 x 64 (forward, dq) or 64 x 32 (dk/dv) blocks its
    # waves do not skip, from a host emulation of the kernels' tile decisions (it reproduces the hardware
    # counter SQ_INSTS_VALU_MFMA_MOPS_BF16 x 512 of the committed profile), so `frac` is the share of the
    # matrix pipes' peak that was really used.  The mask plan lets the kernels skip most of the canonical
    # 128 x 128 tiles: the tile-effective rate (north-star accounting) of the same launch is given next to it.
    gemm_units = {"fa_fwd": 1.0, "fa_bwd_dkdv": 2.0, "fa_bwd_dq": 1.5}
    ex = W.executed_flops(w)
    executed = {"fa_fwd": ex["fwd"], "fa_bwd_dkdv": ex["dkdv"], "fa_bwd_dq": ex["dq"]}
    dom = max(gemm_units, key=lambda n: kt[n])
    traffic, traffic_src = profiled_traffic(w.name, dom)
    roofline = {"bound": "mfma", "kernel": dom, "achieved": round(tf(executed[dom], kt[dom]), 1), "peak": peak,
                "unit": "TFLOP/s", "frac": round(tf(executed[dom], kt[dom]) / peak, 4),
                "traffic": traffic, "traffic_source": traffic_src,
                "avg_launch_ms": round(kt[dom], 4),
                "flops_per_launch_executed": executed[dom],
                "tile_effective_tflops": round(tf(gemm_units[dom] * f_fwd["tile"], kt[dom]), 1),
                "all": {n: {"achieved": round(tf(executed[n], kt[n]), 1),
                            "frac": round(tf(executed[n], kt[n]) / peak, 4),
                            "avg_launch_ms": round(kt[n], 4),
                            "tile_effective_tflops": round(tf(u * f_fwd["tile"], kt[n]), 1)} for n, u in gemm_units.items()}}

    if w.dtype in ("bf16", "fp16"):
        # What the matrix pipes of THIS box sustain in a bare MFMA loop on random operands (the boxes of a pool
        # differ, and the clock follows the load): context for `frac`, which stays a share of the data-sheet peak.
        try:
            from flash_mi355.build import PROBE_LIB_PATH
            probe = ctypes.CDLL(str(PROBE_LIB_PATH))
            probe.fa_probe_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
            rate = ctypes.c_float(0)
            if probe.fa_probe_mfma_rate(1, 20000, ctypes.byref(rate)) == 0 and rate.value > 0:
                roofline["sustained_mfma_probe"] = round(rate.value, 1)
                roofline["frac_of_sustained"] = round(roofline["achieved"] / rate.value, 4)
        except OSError:
            pass

    value = tf(3.5 * f_fwd["tile"], ms_per_step)
    executed_step = ex["fwd"] + ex["dq"] + ex["dkdv"]
    line = {
        "metric": f"attention fwd+bwd TFLOP/s ({w.dtype}, {'doc+' if w.doc else ''}{'block+' if w.block is not None else ''}{'causal' if w.causal else 'no'} mask, tile-effective FLOPs)",
        "value": round(value, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.dtype, "data": "synthetic",
        "config": {"workload": w.name, "B": w.B, "H": w.H, "Hk": w.Hk, "Lq": w.Lq, "Lk": w.Lk, "D": w.D,
                   "causal": w.causal, "doc_mask": w.doc, "block_mask": w.block is not None},
        # the same step under the other two accountings, and what the matrix pipes really did
        "value_dense_equivalent": round(tf(3.5 * f_fwd["dense"], ms_per_step), 1),
        "value_executed": round(tf(executed_step, ms_per_step), 1),
        "pct_of_mfma_peak": round(100 * tf(executed_step, ms_per_step) / peak, 2),
        "pct_of_mfma_peak_tile_effective": round(100 * value / peak, 2),
        "detail": detail, "roofline": roofline,
    }
    if not args.only_headline:
        # the other configurations of the benchmark definition, measured in this same run
        del q, k, v, do, eq, ek
        torch.cuda.empty_cache()
        names = [n for n in W.WORKLOADS if n != w.name]
        line["other_configs"] = {n: measure_other_config(n, torch) for n in names}
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(w, args.cpu_heads, torch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
