#!/usr/bin/env python3
"""CLT forward benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1] [--no-cpu]

One step = one forward pass (encoder projection of all layers -> BatchTopK selection ->
sparse cross-layer decode of all targets) over one synthetic batch that is already
resident in HBM.  Prints ONE JSON line: whole-forward tokens/s, the roofline of the
dominant kernel (the sparse decode) measured with HIP events around its launch, the
per-stage figures, and a CPU baseline (the reference's dense algorithm, restated in
``oracle/``, timed on the host cores on a bounded sample of the same workload).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, GB/s
MFMA_BF16_PEAK_TF = 2500.0  # dense bf16, TFLOP/s
MFMA_FP32_PEAK_TF = 157.3


def _esize(dtype_name: str) -> int:
    return 4 if dtype_name == "float32" else 2


def _dtname(dtype_name: str) -> str:
    return {"float32": "f32", "bfloat16": "bf16", "float16": "f16"}[dtype_name]


def algorithmic_work(wl, nnz_rows_pairs: int, nnz_total: int):
    """Algorithmic flops / bytes per forward, by stage (e = bytes per element)."""
    e = _esize(wl.dtype)
    L, T, d, F = wl.num_layers, wl.tokens, wl.d_model, wl.num_features
    P = nnz_rows_pairs  # (token, feature, source->target) triples that fetch a decoder vector
    n_dec = L * (L + 1) // 2 if wl.decoder_tying == "none" else L
    return {
        "encoder_flop": 2.0 * T * d * F * L,
        "select_bytes": float(L * T * F * e + nnz_total * (4 + e)),
        "decode_gathered_bytes": float(P * d * e + P * (4 + e) + L * T * d * e),
        "decode_compulsory_bytes": float(n_dec * F * d * e + P * (4 + e) + L * T * d * e),
    }


def profiled_traffic(workload: str):
    """({kernel name: (dispatches, HBM bytes per launch)}, forwards profiled) from the counter summary kept
    under profiles/ for this workload: FETCH_SIZE and WRITE_SIZE of `rocprofv3 --pmc`, each scaled by what
    the same counter reads for the known-size copy of ``--copy-probe``.  ({}, 0) when there is no such file:
    the traffic figures are then left out rather than guessed."""
    path = os.path.join(ROOT, "profiles", f"forward_{workload}_hbm_traffic.txt")
    table, forwards = {}, 0
    try:
        for line in open(path):
            if line.startswith("forwards profiled:"):
                forwards = int(line.split(":")[1])
            elif line.startswith("k_"):
                f = line.split()
                name = " ".join(f[:-6])
                table[name] = (int(f[-6]), float(f[-1]) * 1e6)
    except (OSError, ValueError, IndexError):
        return {}, 0
    return table, forwards


def gather_yardstick(lib, dev, table_bytes: int, row_bytes: int, steps: int = 5, reps: int = 4):
    """(GB/s, spread) of a bare gather of ``row_bytes`` rows from a table of ``table_bytes`` (the piece of a
    decoder matrix one XCD works on): what the L2 -> CU path delivers to this access pattern on the GPU at
    hand, with no survivor lists, partial rows or arithmetic around it.  Four grid sizes, each timed ``reps``
    times over ``steps`` launches after a warm-up; the figure is the best run of the best grid size, and
    ``spread`` = (lowest, highest) of that grid size's runs - how far the yardstick itself moves."""
    n_rows = max(1, table_bytes // row_bytes)
    n_idx = 4_000_000 * 1536 // row_bytes
    g = torch.Generator(device=dev).manual_seed(0)
    table = torch.randint(0, 1 << 30, (n_rows * row_bytes // 4,), dtype=torch.int32, device=dev, generator=g)
    idx = torch.randint(0, n_rows, (n_idx,), dtype=torch.int32, device=dev, generator=g)
    stream = torch.cuda.current_stream().cuda_stream
    best, spread = 0.0, (0.0, 0.0)
    for blocks in (256 * 2, 256 * 4, 256 * 8, 256 * 16):
        out = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
        if lib.clt_probe_gather(table.data_ptr(), n_rows, row_bytes, idx.data_ptr(), n_idx, blocks, 0, out.data_ptr(), stream):
            return None, None
        runs = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(steps):
                lib.clt_probe_gather(table.data_ptr(), n_rows, row_bytes, idx.data_ptr(), n_idx, blocks, 0, out.data_ptr(), stream)
            b.record()
            b.synchronize()
            runs.append(n_idx * row_bytes * steps / (a.elapsed_time(b) * 1e-3) / 1e9)
        if max(runs) > best:
            best, spread = max(runs), (min(runs), max(runs))
    return best, spread


def copy_probe(dev):
    """A plain elementwise kernel that reads 256 MiB and writes 256 MiB: the yardstick the
    FETCH_SIZE / WRITE_SIZE counters of a profiled run are scaled by."""
    n = 64 * 1024 * 1024
    src = torch.ones(n, dtype=torch.int32, device=dev)
    dst = torch.empty_like(src)
    torch.neg(src, out=dst)
    torch.cuda.synchronize()
    return int(dst[0].item())


def gpu_events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def run_gpu(args):
    import crosslayer_coding_amd as cca
    from crosslayer_coding_amd import engine, synth

    wl = synth.WORKLOADS[args.workload]
    if args.topk_mode and args.topk_mode != wl.topk_mode:
        wl = wl.scaled(f"{wl.name}-{args.topk_mode}", topk_mode=args.topk_mode)
    if args.dtype and args.dtype != wl.dtype:
        wl = wl.scaled(f"{wl.name}-{_dtname(args.dtype)}", dtype=args.dtype)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cca._native.load(build_if_missing=False)
    model, inputs, slab = synth.build_model(wl, dev)
    model.eval()
    model.fuse_encode_select = not args.no_fuse
    L, T = wl.num_layers, wl.tokens

    for _ in range(args.warmup):
        out = model(inputs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = model(inputs)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    del out

    # per-stage durations: the same three launches, bracketed by events on the launch stream
    enc, dec = model.encoder_module, model.decoder_module
    ws = model._workspace()
    pre_buf = ws.typed("pre", (L, T, wl.num_features), model.dtype)
    glob = wl.topk_mode != "per_layer"
    src_mask = (1 << L) - 1
    st = {"encode": 0.0, "select": 0.0, "decode": 0.0}
    surv = None
    _, x_slab, w_slab, b_slab = enc.prepare_slab(inputs)
    fused = (wl.activation_fn == "batchtopk" and not glob and model.fuse_encode_select
             and engine.encode_collect_supported(x_slab, w_slab, b_slab, wl.k))
    theta = model.theta_manager.thresholds(model.dtype) if wl.activation_fn == "jumprelu" else None
    fused_thr = (wl.activation_fn == "jumprelu" and model.fuse_encode_select
                 and engine.encode_threshold(x_slab, w_slab, b_slab, theta, ws, model._density_ppm) is not None)
    for _ in range(args.steps):
        ev = gpu_events(4)
        ev[0].record()
        if fused:
            # encoder whose epilogue keeps the candidates only (plus the sample before it and the
            # first histogram after it), then the exact selection on the candidates
            handle = engine.encode_collect(x_slab, w_slab, b_slab, wl.k, pre_buf, ws)
            ev[1].record()
            surv = engine.collect_select(handle)
        elif fused_thr:
            # projection with the thresholds applied in the epilogue, survivor list laid out from
            # the pool: one call, all of it counted as the encoder stage
            surv = engine.encode_threshold(x_slab, w_slab, b_slab, theta, ws, model._density_ppm)
            ev[1].record()
        else:
            pre = engine.encode(x_slab, w_slab, b_slab, out=pre_buf)
            ev[1].record()
            if wl.activation_fn == "batchtopk":
                surv = engine.batchtopk_select(pre, wl.k, glob, ws)
            elif wl.activation_fn == "jumprelu":
                surv = engine.threshold_select(pre, theta, cca._native.PRED_GE_THETA, ws)
            else:
                surv = model._survivors(inputs)[2]
        ev[2].record()
        rec = dec.decode_survivors(surv, src_mask, ws=ws)
        ev[3].record()
        torch.cuda.synchronize()
        st["encode"] += ev[0].elapsed_time(ev[1])
        st["select"] += ev[1].elapsed_time(ev[2])
        st["decode"] += ev[2].elapsed_time(ev[3])
    for k in st:
        st[k] /= args.steps
    del rec

    counts = (surv.row_ptr[1:] - surv.row_ptr[:-1]).view(L, T).sum(dim=1).tolist()
    nnz_total = int(sum(counts))
    # every survivor of source s fetches one decoder vector for each target t >= s
    pairs = int(sum(counts[s] * (L - s) for s in range(L)))
    work = algorithmic_work(wl, pairs, nnz_total)
    enc_tf = work["encoder_flop"] / (st["encode"] * 1e-3) / 1e12
    sel_gbs = work["select_bytes"] / (st["select"] * 1e-3) / 1e9
    dec_gbs = work["decode_gathered_bytes"] / (st["decode"] * 1e-3) / 1e9
    dec_c_gbs = work["decode_compulsory_bytes"] / (st["decode"] * 1e-3) / 1e9
    # ---- the dominant kernel: the decode ----------------------------------------------------------------
    nat = cca._native
    e = _esize(wl.dtype)
    F, d = wl.num_features, wl.d_model
    mfma_peak = MFMA_FP32_PEAK_TF if wl.dtype == "float32" else MFMA_BF16_PEAK_TF   # fp16 and bf16: the same dense peak
    route = engine.decode_route(T, d, F, L, wl.decoder_tying, model.dtype)
    dense_first, dense_end = dec.last_route.get("dense_targets", (L, L))
    n_dense = dense_end - dense_first
    table, forwards = profiled_traffic(wl.name)
    if n_dense > 0:
        # decoders tied per target: targets [dense_first, L) are dense products on the MFMA kernel
        flop = 2.0 * T * F * d * n_dense
        tf = flop / (st["decode"] * 1e-3) / 1e12
        roofline = {
            "kernel": (f"k_encode_mfma as the decoder product summed[T,F] @ W[t].T of targets {dense_first}..{dense_end - 1} "
                       f"({n_dense} launches per step, with the scatter of the summed activations before each)"),
            "bound": "mfma", "achieved": tf, "peak": mfma_peak, "unit": "TFLOP/s", "frac": tf / mfma_peak, "traffic": None,
            "algorithmic_flop_per_launch": flop / n_dense, "avg_launch_ms": st["decode"] / n_dense,
            "launches_per_step": n_dense,
            "note": "achieved = 2 T F d per dense target / the whole decode stage (scatter kernels and any gathered targets included)",
        }
        decode_stage = {"ms": st["decode"], "bound": "mfma", "achieved": tf, "peak": mfma_peak, "unit": "TFLOP/s",
                        "frac": tf / mfma_peak}
    else:
        sliced = route in (nat.ROUTE_QUARTER, nat.ROUTE_LINE, nat.ROUTE_SLICED)
        n_dec_launch = L if sliced else 1
        kname = {nat.ROUTE_QUARTER: "k_decode_quarter", nat.ROUTE_LINE: "k_decode_line"}.get(route, "k_decode")
        # the piece of one decoder matrix that an XCD gathers from while the tokens stream past
        if route == nat.ROUTE_QUARTER:
            part_bytes = (F // 2) * (d // 4) * e
        elif route == nat.ROUTE_LINE:
            part_bytes = F * 128 // max(1, -(-F * 128 // 3407872))
        elif route in (nat.ROUTE_SLICED, nat.ROUTE_SLICED_ALL_SOURCES):
            part_bytes = (F // 8) * d * e
        else:
            part_bytes = F * d * e
        row_bytes = min(d * e, 2048) // 16 * 16
        yard, yard_spread = gather_yardstick(nat.load(), dev, part_bytes, row_bytes) if row_bytes >= 16 else (None, None)
        per_launch_s = st["decode"] / n_dec_launch * 1e-3
        hit = [v for k, v in table.items() if k.startswith(kname + "<")]
        traffic = hit[0][1] if hit else None
        comp = work["decode_compulsory_bytes"] / n_dec_launch
        roofline = {
            "kernel": (f"{kname} (sparse cross-layer decode; {n_dec_launch} launch(es) per step; the per-launch figures are "
                       "the step's decode stage divided by that count)"),
            "bound": "l2_gather (measured)",
            "achieved": dec_gbs,
            "peak": yard,
            "peak_spread": yard_spread,
            "unit": "GB/s",
            "frac": (dec_gbs / yard) if yard else None,
            "traffic": traffic,
            # the same launch against the published HBM peak (8 TB/s): on the bytes that must come from HBM at
            # least once, and on the HBM traffic the counters measured
            "hbm_compulsory_frac": dec_c_gbs / HBM_PEAK_GBS,
            "hbm_traffic_frac": (traffic / per_launch_s / 1e9 / HBM_PEAK_GBS) if traffic else None,
            "hbm": {"peak": HBM_PEAK_GBS, "compulsory_bytes_per_launch": comp, "compulsory_GBps": dec_c_gbs,
                    "compulsory_frac": dec_c_gbs / HBM_PEAK_GBS,
                    "traffic_GBps": (traffic / per_launch_s / 1e9) if traffic else None,
                    "traffic_frac": (traffic / per_launch_s / 1e9 / HBM_PEAK_GBS) if traffic else None},
            "note": ("achieved = gathered bytes (every active (token, feature, source->target) fetches one decoder row) per "
                     "launch / launch time.  The rows come from the L2s, not from HBM, so the bound is what a bare gather of "
                     f"{row_bytes}-byte rows reaches from a table the size of the piece an XCD works on ({part_bytes / 1e6:.1f} MB), "
                     "measured in this run with clt_probe_gather (best of four grid sizes).  hbm: the same launch against the "
                     "HBM peak, on the compulsory bytes (each decoder row once) and on the profiled traffic (FETCH_SIZE + "
                     "WRITE_SIZE of the counter run kept under profiles/, null when there is none)"),
            "algorithmic_bytes_per_launch": work["decode_gathered_bytes"] / n_dec_launch,
            "avg_launch_ms": st["decode"] / n_dec_launch,
            "launches_per_step": n_dec_launch,
        }
        decode_stage = {"ms": st["decode"], "bound": "l2_gather (measured)", "achieved": dec_gbs, "peak": yard,
                        "unit": "GB/s", "frac": (dec_gbs / yard) if yard else None,
                        "compulsory_GBps": dec_c_gbs, "compulsory_frac": dec_c_gbs / HBM_PEAK_GBS}
    # what the selection stage really moves, from the same counter run (it never reads the ranking values in the
    # fused path: they are compared in the encoder epilogue)
    sel_kernels = ("k_tile_emit", "k_tile_count", "k_pool_hist", "k_row_prefix", "k_select_allot", "k_select_scan",
                   "k_select_pass", "k_select_emit", "k_select_count", "k_select_level", "k_rowptr_scan")
    sel_real = sum(n * b for k, (n, b) in table.items() if k.split("<")[0] in sel_kernels) / forwards if forwards else None
    result = {
        "metric": "CLT forward tokens/sec at GPT-2-small x32 BatchTopK k=200; % of roofline per stage",
        "value": T * args.steps / wall,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": _dtname(wl.dtype),
        "data": "synthetic",
        "config": {
            "workload": f"{wl.name}: CLT forward, L={L} d_model={wl.d_model} F={wl.num_features} T={T} "
                        f"{wl.activation_fn} k={wl.k} ({wl.topk_mode}), decoders {wl.decoder_tying}",
            "global_batch_tokens": T,
            "survivors_per_layer": counts[0],
            "encode_select": ("fused (candidates collected in the encoder epilogue)" if fused else
                              "fused (thresholds applied in the encoder epilogue; the select stage is empty)"
                              if fused_thr else "separate kernels"),
        },
        "roofline": roofline,
        "stages": {
            "encoder": {"ms": st["encode"], "bound": "mfma", "achieved": enc_tf, "peak": mfma_peak,
                        "unit": "TFLOP/s", "frac": enc_tf / mfma_peak,
                        "note": ("includes the sample / cut before and the candidate histogram after the projection"
                                 if fused else "projection only")},
            "select": {"ms": st["select"], "bound": "hbm", "achieved": None if fused_thr else sel_gbs,
                       "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None if fused_thr else sel_gbs / HBM_PEAK_GBS,
                       "moved_bytes": sel_real,
                       "moved_GBps": (sel_real / (st["select"] * 1e-3) / 1e9) if sel_real and st["select"] > 0 else None,
                       "moved_frac": (sel_real / (st["select"] * 1e-3) / 1e9 / HBM_PEAK_GBS) if sel_real and st["select"] > 0 else None,
                       "note": ("achieved / frac: algorithmic bytes = one read of the ranking values + the survivor write. "
                                "In the fused path the ranking values are compared in the encoder epilogue and never reach "
                                "HBM, so this stage only touches the candidates: moved_* are the HBM bytes its kernels "
                                "really move (profiled counters, null without a counter run)") if fused else
                               "empty: the survivor list is written by the encoder stage" if fused_thr else
                               "separate streaming pass"},
            "decode": decode_stage,
        },
    }
    if args.copy_probe:
        copy_probe(dev)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(wl, model, slab, args.cpu_tokens)
    return result


def run_theta(args):
    """Post-hoc theta estimation (reference clt/models/theta.py:175-430) over ``steps`` batches of the
    workload's inputs; one step = one batch: encoder, per-feature statistics, global BatchTopK ranked
    on the z-score, per-feature minimum of the selected z-scores."""
    import crosslayer_coding_amd as cca
    from crosslayer_coding_amd import synth

    wl = synth.WORKLOADS[args.workload].scaled(args.workload + "-global", topk_mode="global")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cca._native.load(build_if_missing=False)
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    data = [(inputs, None)] * (args.warmup + args.steps)
    k, fn = model.config.batchtopk_k, model.config.activation_fn
    model.estimate_theta_posthoc(data[:args.warmup], num_batches=args.warmup)
    model.config.activation_fn, model.config.batchtopk_k = fn, k       # estimate again from the same starting point
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    model.estimate_theta_posthoc(data[:args.steps], num_batches=args.steps)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return {
        "metric": "post-hoc theta estimation tokens/sec (encoder + statistics + global BatchTopK + selected minimum)",
        "value": wl.tokens * args.steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": wall / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": _dtname(wl.dtype), "data": "synthetic",
        "config": {"workload": f"{wl.name}: theta estimation, L={wl.num_layers} d_model={wl.d_model} "
                               f"F={wl.num_features} T={wl.tokens} batchtopk k={wl.k} (global)"},
    }


def run_probe(args):
    """Calibration of the gather-bound stages: a bare gather of 1536-byte rows (the decoder row of C1)
    from tables of growing size, timed with events.  Every XCD reads the whole table, so the table
    size is each L2's working set: 2-3 MB fit the 4 MB L2, 4.7 MB is the decoder slice one XCD works on
    at C1, 64 MB fits the memory-side cache, 4 GB neither."""
    import crosslayer_coding_amd as cca

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = cca._native.load(build_if_missing=False)
    row_bytes = int(args.probe_row_bytes)
    n_idx = 5_400_000 * 1536 // row_bytes                   # one decode launch at C1 gathers 5.3 M rows of 1536 bytes
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device=dev).manual_seed(0)
    results = {}
    for label, table_bytes in (("2 MB", 2 << 20), ("3 MB", 3 << 20), ("4 MB", 4 << 20), ("4.7 MB", 4928307), ("6 MB", 6 << 20),
                               ("64 MB", 64 << 20), ("4 GB", 4 << 30)):
        n_rows = table_bytes // row_bytes
        table = torch.randint(0, 1 << 30, (n_rows * row_bytes // 4,), dtype=torch.int32, device=dev, generator=g)
        idx = torch.randint(0, n_rows, (n_idx,), dtype=torch.int32, device=dev, generator=g)
        best, best_lds = None, None
        for to_lds in ((0, 1) if row_bytes >= 1024 else (0,)):
            moved = row_bytes if not to_lds else 2048
            for blocks in (256 * 2, 256 * 4, 256 * 8, 256 * 16):
                out = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
                for _ in range(2):
                    rc = lib.clt_probe_gather(table.data_ptr(), n_rows, row_bytes, idx.data_ptr(), n_idx, blocks, to_lds,
                                              out.data_ptr(), stream)
                    assert rc == 0
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                for _ in range(args.steps):
                    lib.clt_probe_gather(table.data_ptr(), n_rows, row_bytes, idx.data_ptr(), n_idx, blocks, to_lds,
                                         out.data_ptr(), stream)
                b.record()
                b.synchronize()
                gbs = n_idx * moved * args.steps / (a.elapsed_time(b) * 1e-3) / 1e9
                if to_lds:
                    if best_lds is None or gbs > best_lds[0]:
                        best_lds = (gbs, blocks)
                elif best is None or gbs > best[0]:
                    best = (gbs, blocks)
        results[label] = {"GB/s": best[0], "blocks": best[1]}
        if best_lds is not None:
            results[label].update({"direct_to_lds_GB/s": best_lds[0], "direct_to_lds_blocks": best_lds[1]})
        del table, idx
    top = results["2 MB"]["GB/s"]
    return {"metric": f"bare gather of {row_bytes}-byte rows, best of four grid sizes", "value": top, "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": 2, "ms_per_step": n_idx * row_bytes / top / 1e6, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": f"gather probe: {n_idx / 1e6:.1f} M random rows of {row_bytes} bytes per launch"}, "tables": results}


def run_feed(args):
    """Activation-store feed (reference clt/training/data/manifest_activation_store.py:776-958): one step =
    one batch of T random rows drawn from 8 chunks of 8192 rows, gathered, normalised (mean / std) and cast
    into the [L, T, d] input and target slabs.  Timed with the chunks resident in HBM (`value`), with the
    chunks in pinned host memory read in place, and with slices arriving as wire-format bytes."""
    import numpy as np
    import crosslayer_coding_amd as cca
    from crosslayer_coding_amd import synth

    wl = synth.WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cca._native.load(build_if_missing=False)
    L, T, d = wl.num_layers, wl.tokens, wl.d_model
    dt = torch.bfloat16 if wl.dtype == "bfloat16" else torch.float32
    n_chunks, rows = 8, 8192
    g = torch.Generator().manual_seed(0)
    stats = {str(l): {k: {"mean": torch.randn(d, generator=g).tolist(), "std": (torch.rand(d, generator=g) + 0.5).tolist()}
                      for k in ("inputs", "targets")} for l in range(L)}
    chunks = [torch.randn(L, 2, rows, d, generator=g).to(dt) for _ in range(n_chunks)]
    rng = np.random.RandomState(1)
    batches = [np.stack([rng.randint(0, n_chunks, T), rng.randint(0, rows, T)], axis=1).astype(np.uint32)
               for _ in range(args.warmup + args.steps)]

    def wire(chunk_id, sorted_rows):
        return chunks[chunk_id][:, :, torch.as_tensor(sorted_rows.astype(np.int64)), :].contiguous().view(torch.uint8).numpy().tobytes()

    def timed(where):
        feed = cca.DeviceActivationFeed(L, d, dtype=dt, device=dev, normalization_method="mean_std", norm_stats=stats)
        if where != "wire":
            for c, t in enumerate(chunks):
                feed.add_chunk(c, t, where=where)
        fetch = wire if where == "wire" else None
        for b in batches[:args.warmup]:
            feed.parse_batch(b, fetch)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for b in batches[args.warmup:]:
            feed.parse_batch(b, fetch)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    sec = timed("device")
    pinned = timed("pinned")
    wire_sec = timed("wire")
    esz = 2 if dt == torch.bfloat16 else 4
    nbytes = 2 * L * T * d * (esz + esz)
    return {
        "metric": "activation-store feed tokens/sec (gather + mean/std normalisation + cast into the batch slabs)",
        "value": T / sec, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if dt == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": f"{wl.name}: store feed, L={L} d_model={d} T={T}, {n_chunks} resident chunks x {rows} rows"},
        "roofline": {"bound": "hbm", "achieved": nbytes / sec / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": nbytes / sec / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "note": "bytes = rows read + rows written, inputs and targets of all layers; wall time of a step "
                             "including the host-side grouping and 8 launches"},
        "pinned_host_ms": pinned * 1e3, "wire_bytes_ms": wire_sec * 1e3,
    }


def run_evaluator(args):
    """The evaluator's reductions (reference clt/training/evaluator.py:194-405, trainer.py:693-712) on one
    batch whose forward has already run: L0 and per-feature firing counts from the survivor list, the
    dead-feature counter update, reconstruction statistics.  One step = the reductions of one batch; the
    same quantities from dense [T, F] activations with torch ops on the GPU are timed beside it."""
    import crosslayer_coding_amd as cca
    from crosslayer_coding_amd import engine, synth

    wl = synth.WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cca._native.load(build_if_missing=False)
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    g = torch.Generator(device=dev).manual_seed(99)
    L, T, F, d = wl.num_layers, wl.tokens, wl.num_features, wl.d_model
    tgt = torch.randn(L, T, d, generator=g, device=dev).to(model.dtype)
    recs, surv = model.forward_with_survivors(inputs)
    rec = torch.stack([recs[l] for l in range(L)]).contiguous()
    tracker = cca.DeadFeatureTracker(L, F, 1000, dev)
    ws = engine.Workspace(dev)

    def one():
        nonzero, fired = engine.survivor_metrics(surv)
        tracker.update(surv, fired)
        return nonzero, fired, engine.reconstruction_stats(rec, tgt, ws=ws)

    def timed(fn, n):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    sec = timed(one, args.steps)
    dense = model.get_feature_activations(inputs)
    counter = torch.zeros(L, F, dtype=torch.long, device=dev)

    def dense_scan():
        for l, a in dense.items():
            (a != 0).float().sum(dim=-1).mean()
            fired = (a > 1e-6).float()
            fired.mean(dim=0); fired.sum(dim=0)
            hit = fired.any(dim=0)
            counter[l] += 1
            counter[l][hit] = 0
            t, r = tgt[l].float(), rec[l].float()
            torch.nn.functional.mse_loss(r, t); torch.var(t, dim=0, unbiased=False).mean()
            torch.var(t - r, dim=0, unbiased=False).mean()

    dense_sec = timed(dense_scan, max(1, args.steps // 4))
    esz = _esize(wl.dtype)
    list_bytes = surv.nnz * (4 + esz) + (L * T + 1) * 4 + L * F * (4 + 4 + 8 + 8) + 2 * L * T * d * esz
    return {
        "metric": "evaluator reductions tokens/sec (L0, firing counts, dead-feature counters, reconstruction statistics)",
        "value": T / sec, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": _dtname(wl.dtype), "data": "synthetic",
        "config": {"workload": f"{wl.name}: evaluator reductions, L={L} d_model={d} F={F} T={T} k={wl.k}"},
        "roofline": {"bound": "hbm", "achieved": list_bytes / sec / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": list_bytes / sec / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "note": "bytes = survivor list + counters + reconstructions and targets, all launches of a step"},
        "dense_torch_ms": dense_sec * 1e3,
    }


def run_dense_regime(args):
    """The workload's shape as a JumpReLU model whose encoder biases are raised by ``--dense-regime`` (1.0: about a
    quarter of the features fire per token, what a run trained from scratch starts at): forward and training step
    on the dense routes (Decoder.dense_pairs_wanted).  One line: forward ms, training-step ms, density, routes."""
    import crosslayer_coding_amd as cca
    from crosslayer_coding_amd import synth

    base = synth.WORKLOADS[args.workload]
    wl = base.scaled(f"{base.name}-jumprelu-dense", activation_fn="jumprelu", k=None)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cca._native.load(build_if_missing=False)
    model, inputs, _ = synth.build_model(wl, dev)
    with torch.no_grad():
        for enc in model.encoder_module.encoders:
            enc.bias_param.add_(args.dense_regime)
    model.eval()
    slab = synth.make_targets(wl, dev)
    targets = {l: slab[l] for l in range(wl.num_layers)}

    def timed(fn, warmup, steps):
        for _ in range(warmup):
            fn()
            torch.cuda.synchronize()       # (the density of a threshold model is known one forward late)
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    with torch.no_grad():
        acts = model.get_feature_activations(inputs)
        density = float(sum((a != 0).float().mean() for a in acts.values())) / len(acts)
        del acts
        fwd_ms = timed(lambda: model(inputs), args.warmup, args.steps)
        fwd_route = dict(model.decoder_module.last_route)
    opt = cca.CLTAdam(model, lr=1e-4)
    step_ms = timed(lambda: model.training_step(inputs, targets, opt), max(2, args.warmup // 2), max(3, args.steps // 4))
    return {
        "metric": "CLT forward and training step in the dense regime (JumpReLU, encoder biases raised)",
        "value": wl.tokens / (fwd_ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": fwd_ms, "training_step_ms": step_ms, "density": density, "forward_route": fwd_route,
        "training_route": dict(model.decoder_module.last_route), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": _dtname(wl.dtype), "data": "synthetic",
        "config": {"workload": f"{wl.name}: L={wl.num_layers} d_model={wl.d_model} F={wl.num_features} T={wl.tokens} "
                               f"jumprelu, encoder biases + {args.dense_regime}"},
    }


def run_backward(args):
    """Forward, MSE reconstruction loss and the gradients of every encoder / decoder parameter
    (CrossLayerTranscoder.loss_and_gradients); one step = one batch.  No optimizer step."""
    import crosslayer_coding_amd as cca
    from crosslayer_coding_amd import synth

    wl = synth.WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cca._native.load(build_if_missing=False)
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    slab = synth.make_targets(wl, dev)
    targets = {l: slab[l] for l in range(wl.num_layers)}
    opt = cca.CLTAdam(model, lr=1e-4) if args.train_step else None

    def one():
        if opt is not None:
            return model.training_step(inputs, targets, opt)
        loss, grads = model.loss_and_gradients(inputs, targets)
        del grads
        return loss

    for _ in range(args.warmup):
        loss = one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = one()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # one more step, stage by stage, with events on the stream the kernels run on
    from crosslayer_coding_amd import engine
    L, T, d, F = wl.num_layers, wl.tokens, wl.d_model, wl.num_features
    stages = {}

    def timed(name, fn):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        out = fn()
        b.record()
        b.synchronize()
        stages[name] = a.elapsed_time(b)
        return out

    cfg, ws, mask = model.config, model._workspace(), (1 << L) - 1
    _, _, surv = timed("forward: encode + select", lambda: model._survivors(inputs))
    rec = timed("forward: decode", lambda: model.decoder_module.decode_survivors(surv, mask, ws=ws))
    tgt = torch.stack([targets[l] for l in range(L)]).contiguous()
    loss_l, g, g_model, bias_grad = timed("loss and its gradient", lambda: engine.mse_loss_grad(rec, tgt, ws))
    dval = timed("gradient of the kept activations", lambda: engine.decode_backward_values(
        surv, model.decoder_module.packed(), g, cfg.decoder_tying, mask, ws))
    lists = timed("per-feature token lists", lambda: engine.feature_lists(surv, ws))
    fused = opt is not None and opt.fuses_decoder_step()
    dw_name = "decoder weight gradient + its Adam step in place" if fused else "decoder weight gradient"
    if fused:
        # what training_step does for untied decoders: the gradient rows go from registers into the update of the
        # moments and of the packed copy, then the checkpoint-layout parameters are rewritten from that copy
        dw_dec = None
        timed(dw_name, lambda: opt.decoder_weight_step(lists, surv, g_model))
    else:
        dw_dec = timed(dw_name, lambda: engine.decoder_weight_grad(lists, surv, g_model, cfg.decoder_tying))
    _, x_slab, _, _ = model.encoder_module.prepare_slab(inputs)
    dw_enc, db_enc = timed("encoder weight gradient", lambda: engine.encoder_weight_grad(lists, dval, x_slab.contiguous(), F))
    if opt is not None:
        dec_b = bias_grad[torch.tensor([t for s_ in range(L) for t in range(s_, L)], device=dev)].contiguous()
        timed("Adam (other parameters)" if fused else "Adam",
              lambda: opt.step({"enc_w": dw_enc, "enc_b": db_enc, "dec_w": dw_dec, "dec_b": dec_b, "theta": None}))
    esz = _esize(wl.dtype)
    pairs = L * (L + 1) // 2
    gathered = surv.nnz / L * pairs * d * esz           # one row of g per (survivor, target >= its source)
    dw_sec = stages[dw_name] * 1e-3
    # The weight-gradient gather reads rows of one layer's loss gradient (every XCD all of it), nearly all of
    # them from the L2: it is priced against what a bare gather of such rows from such a table reaches on
    # this GPU, measured now; what has to cross the HBM interface (the fp32 gradient written once, the
    # gradient slab and the lists read once) is the second figure.
    yard, _ = gather_yardstick(cca._native.load(build_if_missing=False), dev, wl.tokens * d * esz, d * esz)
    # per decoder element the fp32 gradient written once - or, with the step in place, both moments and the packed
    # copy read and written and the parameter rewritten from the copy
    hbm_bytes = pairs * F * d * ((16 + 4 * esz) if fused else 4) + L * wl.tokens * d * esz + surv.nnz * (8 + esz)
    tiled = fused and opt._dec_layout == "tiles"
    if tiled:
        # Column-tile route: the gather of the loss gradient is LDS traffic; through the HBM interface go both
        # moments (read and written: 16 bytes per decoder element), the tiled weight copy (read and written) and
        # the conversion that follows (tiles read, feature-major slab and checkpoint layout written): 5 elements.
        hbm_bytes = pairs * F * d * (16 + 5 * esz) + L * wl.tokens * d * esz + surv.nnz * (8 + esz)
        roofline = {"kernel": f"k_tile_outer_adam + k_tile_convert ({dw_name}, one launch each per step)",
                    "bound": "hbm", "achieved": hbm_bytes / dw_sec / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": hbm_bytes / dw_sec / 1e9 / HBM_PEAK_GBS, "traffic": None,
                    "lds_gather_GBps": gathered / dw_sec / 1e9,
                    "note": "achieved = compulsory HBM bytes of the stage (moments, tiled weights, converted layouts, "
                            "loss gradient, lists) / the stage's time; the kernel itself is bound by vector-instruction "
                            "issue (see the profile summary), not by this interface"}
    else:
        roofline = None
    roofline = roofline or {"kernel": f"k_feature_outer ({dw_name}, {L} launches per step)",
                "bound": "l2_gather (measured)", "achieved": gathered / dw_sec / 1e9, "peak": yard, "unit": "GB/s",
                "frac": (gathered / dw_sec / 1e9 / yard) if yard else None, "traffic": None,
                "hbm": {"compulsory_bytes": hbm_bytes, "compulsory_GBps": hbm_bytes / dw_sec / 1e9,
                        "compulsory_frac": hbm_bytes / dw_sec / 1e9 / HBM_PEAK_GBS},
                "note": "achieved = rows of the loss gradient gathered per (survivor, target) / the stage's time; peak = "
                        "clt_probe_gather on rows of this length from a table the size of one layer's gradient"}
    if opt is not None:
        # Adam is the one stage that streams: per decoder element the fp32 gradient (4), both moments read and
        # written (16), the feature-major copy read and written (2 e) and the checkpoint-layout parameter (e);
        # per encoder element gradient, moments and the parameter read and written
        n_dec, n_enc = pairs * F * d, L * F * d
        adam_bytes = (0 if fused else n_dec * (20 + 3 * esz)) + n_enc * (20 + 2 * esz)
        adam_sec = stages["Adam (other parameters)" if fused else "Adam"] * 1e-3
        roofline["adam"] = {"bound": "hbm", "bytes": adam_bytes, "achieved": adam_bytes / adam_sec / 1e9,
                            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": adam_bytes / adam_sec / 1e9 / HBM_PEAK_GBS}
    return {
        "stages_ms": stages, "roofline": roofline,
        "decoder_step_route": (("column tiles" if tiled else "rows") if fused else "gradient then Adam") if opt is not None else None,
        "metric": ("CLT training step tokens/sec (forward, MSE loss, gradients, Adam lr 1e-4 with fp32 moments)"
                   if opt is not None else "CLT forward + MSE loss + gradients tokens/sec (no optimizer step)"),
        "value": wl.tokens * args.steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": wall / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": _dtname(wl.dtype), "data": "synthetic",
        "config": {"workload": f"{wl.name}: forward + backward, L={wl.num_layers} d_model={wl.d_model} "
                               f"F={wl.num_features} T={wl.tokens} {wl.activation_fn} k={wl.k}", "loss": float(loss)},
    }


def cpu_baseline(wl, model, slab, tokens):
    """The reference's dense forward (F.linear encoder, torch.topk mask, one dense F.linear
    per decoder, sum in the model dtype) from ``oracle/``, on the first ``tokens`` tokens of
    the same batch with the same weights, on the host cores."""
    from oracle import clt_oracle as orc

    L = wl.num_layers
    dtype = getattr(torch, wl.dtype)
    sd = {k: v.detach().cpu() for k, v in model.state_dict().items()}
    enc_w = [sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)]
    enc_b = [sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)]
    from crosslayer_coding_amd import synth

    names = synth.decoder_names(wl)
    dec_w = {n: sd[f"decoder_module.decoders.{n}.weight"] for n in names}
    dec_b = {n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names}
    x = {l: slab[l, :tokens].detach().cpu() for l in range(L)}
    cores = torch.get_num_threads()
    t0 = time.perf_counter()
    orc.forward(x, enc_w=enc_w, enc_b=enc_b, dec_w=dec_w, dec_b=dec_b, activation_fn=wl.activation_fn,
                dtype=dtype, num_layers=L, d_model=wl.d_model, num_features=wl.num_features,
                tying=wl.decoder_tying, k=wl.k, topk_mode=wl.topk_mode,
                log_threshold=sd.get("theta_manager.log_threshold"), timed_baseline=True)
    dt = time.perf_counter() - t0
    return {
        "value": tokens / dt,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"one dense forward of the first {tokens} tokens of the {wl.name} batch "
                  f"(same weights, {wl.dtype}, torch {torch.__version__} CPU ops, {dt:.1f} s)",
    }


def main():
    torch.set_grad_enabled(False)      # the forward is measured as inference; the training modes compute their own gradients
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c1")
    ap.add_argument("--dtype", choices=["float32", "bfloat16", "float16"], default=None,
                    help="forward bench only: run the workload in another element type than its own")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-tokens", type=int, default=4096)
    ap.add_argument("--no-fuse", action="store_true", help="separate encoder and selection kernels")
    ap.add_argument("--topk-mode", choices=["per_layer", "global"], default=None,
                    help="override the workload's BatchTopK scope (global = the reference's default helper)")
    ap.add_argument("--theta-estimation", action="store_true",
                    help="time batches of the post-hoc theta estimation (encoder, column statistics, global "
                         "selection, per-feature minimum) instead of the forward")
    ap.add_argument("--backward", action="store_true",
                    help="time forward + MSE loss + all gradients (loss_and_gradients) instead of the forward")
    ap.add_argument("--probe-row-bytes", type=int, default=1536,
                    help="row size of --gather-probe (a multiple of 16 up to 2048; 1536 is a whole C1 decoder row, 384 a quarter)")
    ap.add_argument("--gather-probe", action="store_true",
                    help="calibration: the rate a bare row gather reaches from L2-, cache- and HBM-sized tables")
    ap.add_argument("--feed", action="store_true",
                    help="time the activation-store feed (gather + normalise + cast into the batch slabs)")
    ap.add_argument("--evaluator", action="store_true",
                    help="time the evaluator's reductions on the survivor list of one batch")
    ap.add_argument("--train-step", action="store_true",
                    help="time full optimisation steps: forward, MSE loss, gradients, Adam update")
    ap.add_argument("--dense-regime", type=float, default=None, metavar="BIAS_SHIFT",
                    help="the workload's shape as a JumpReLU model with the encoder biases raised by this much: forward "
                         "and training step at high density (the dense routes)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one 256 MiB elementwise copy (counter yardstick for profiled runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the one-GPU forward path; this build has no multi-GPU path "
              f"(asked for --gpus {args.gpus})", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(2)
    print(json.dumps(run_dense_regime(args) if args.dense_regime is not None else run_theta(args) if args.theta_estimation else run_evaluator(args) if args.evaluator else run_feed(args) if args.feed else run_probe(args) if args.gather_probe else run_backward(args) if (args.backward or args.train_step) else run_gpu(args)))


if __name__ == "__main__":
    main()
