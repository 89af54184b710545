#!/usr/bin/env python3
"""Benchmark of the LUT-AMM hot path on one MI355X.

Workload (default): the BERT-base FFN pair as LUT-AMM -- N = 8192 tokens (batch 64 x seq 128),
768 -> 3072 and 3072 -> 768, sub_vec_len 4, 16 centroids per codebook, int8 LUTs with the
reference's per-tensor fp32 scale, int32 accumulation, random-init centroids and weights.
One "step" = one pass of the pair (centroid search + LUT gather for FFN1, then for FFN2) with all
inputs, LUTs and outputs resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-model] [--no-large-layer] [--no-sweep] [--no-cpu-baseline]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0                     # MI355X HBM3E
LDS_PEAK_GBPS = 256 * 256 * 2.4            # 256 CUs x 256 B/clk (ds_read_b128) x 2.4 GHz = 157286 GB/s
MFMA_I8_PEAK_TOPS = 5000.0                 # MI355X dense int8 matrix peak
# HBM bytes per launch of the dominant gather kernel, from two rocprofv3 --pmc runs of this script
# (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch; summary: profiles/bench_ffn_pair_hbm_traffic.txt).
# Keyed by the kernel's name as a profile lists it and by the batch: the figure is only reported while the
# launch still runs that kernel on that batch, otherwise `traffic` is null until the counters are collected again.
# FETCH_SIZE is scaled by 2.0 and WRITE_SIZE by 1.0: what a streaming copy of known size reads for the same
# counters in the same runs.
MEASURED_GATHER_TRAFFIC = {
    ("gather_sparse_kernel<6, 4, 16, 4, false>", 8192, 768, 3072): {"fetch_kib": 9830.5, "write_kib": 98317.1},
    ("gather_sparse_kernel<3, 4, 64, 8, false>", 8192, 3072, 768): {"fetch_kib": 15643.5, "write_kib": 24948.0},
}
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0
# Busy fractions of the same kernels from a rocprofv3 --pmc run of this script (summary:
# profiles/bench_ffn_pair_lds_mfma_counters.txt): matrix core (SQ_VALU_MFMA_BUSY_CYCLES / SQ_BUSY_CU_CYCLES), LDS
# (SQ_LDS_IDX_ACTIVE / ...), LDS bank-conflict cycles over LDS-active cycles.  Reported only for the kernel they belong to.
MEASURED_GATHER_COUNTERS = {
    ("gather_sparse_kernel<6, 4, 16, 4, false>", 8192, 768, 3072): {
        "matrix_core_busy_frac": 0.425, "lds_active_frac": 0.368, "lds_bank_conflict_frac_of_active": 0.225, "wave_cycles_waiting_to_issue_frac": 0.37},
    ("gather_sparse_kernel<3, 4, 64, 8, false>", 8192, 3072, 768): {
        "matrix_core_busy_frac": 0.440, "lds_active_frac": 0.501, "lds_bank_conflict_frac_of_active": 0.254, "wave_cycles_waiting_to_issue_frac": 0.37},
}
CLOCK_SETTLE_S = 0.08                      # untimed pre-heat: the engine clock needs ~20 ms of this load to ramp up


def synth_amm(rng, K, v, C, M, pimdl, ctx):
    """Random-init centroids N(0,1) and weight N(0,0.02); LUT built and quantised on the GPU."""
    CB = K // v
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    W = (rng.standard_normal((K, M)) * 0.02).astype(np.float32)
    lut, scales = ctx.lutgen(cent, W, pimdl.LUT_I8, 0)
    bias = np.zeros(M, np.float32)
    return cent, lut, scales, bias


def algorithmic_bytes(N, K, v, C, M, e=1):
    CB = K // v
    ib = 0.5 if C <= 16 else 1.0
    return {
        "ccs_hbm": 4 * N * K + 4 * C * K + ib * N * CB,
        "gather_hbm": ib * N * CB + e * CB * C * M + 4 * N * M + 4 * M,
        "gather_lds": e * N * CB * M,
        "eff_ops": 2 * N * K * M,
    }


def model_forward(pimdl, ctx, iters=10):
    """The full 12-layer LUT-BERT-base encoder forward (every linear a LUT-AMM, v=4, C=16, int8 LUTs;
    N = 32 x 128 = 4096 tokens, random-init weights), timed end to end on the GPU: a secondary figure
    next to the headline metric."""
    import torch
    from pim_dl_asplos_amd import transformer as T
    p = T.TransformerParams.bert_base(batch_size=32, seq_len=128, layer_num=12)
    model = T.Transformer(ctx, pimdl, T.synth_layers(p, ctx, pimdl, seed=1), p)
    x = torch.randn((p.n, p.token_dim), device="cuda", dtype=torch.float32)
    for _ in range(3):
        model.forward(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        model.forward(x)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / iters
    # the same forward recorded once into a HIP graph and replayed (no host work between the kernels)
    graph, _sx, _sy = model.capture(x)
    for _ in range(10):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3 * iters):
        graph.replay()
    torch.cuda.synchronize()
    ms_graph = (time.perf_counter() - t0) * 1e3 / (3 * iters)
    del graph
    model.close()
    return {"layers": 12, "tokens": p.n, "ms_per_forward": ms, "tokens_per_s": p.n / (ms * 1e-3),
            "ms_per_forward_graph": ms_graph, "tokens_per_s_graph": p.n / (ms_graph * 1e-3),
            "note": "LUT-AMM linears (tanh-GELU inside the first feed-forward operator's epilogue), pimdl_layer_norm and pimdl_attention (fp32) on libpimdl; PyTorch-ROCm for tensors, streams and graph capture"}


def bert_large_layer(pimdl, ctx, iters=20):
    """One BERT-large encoder layer as a layer (hidden 1024, 16 heads x 64, feed-forward 4096, N = 64 x 128 = 8192
    tokens, every linear a LUT-AMM with v=4, C=16, int8 LUTs): time of the whole layer and of each of its stages
    launched on its own (device time between two events around `iters` launches, after the clock has settled)."""
    import torch
    from pim_dl_asplos_amd import transformer as T
    p = T.TransformerParams(128, 64, 16, 64, 1024, 4096, 1)
    for op, (k_in, m_out) in {"q": (1024, 1024), "k": (1024, 1024), "v": (1024, 1024), "o": (1024, 1024),
                              "ffn1": (1024, 4096), "ffn2": (4096, 1024)}.items():
        p.shapes[op] = T.AmmShape(k_in // 4, 16, k_in, m_out)
    layer = T.TransformerLayer(ctx, pimdl, T.synth_layers(p, ctx, pimdl, seed=2)[0], p)
    n, d = p.n, p.token_dim
    x = torch.randn((n, d), device="cuda", dtype=torch.float32)
    keep = {}
    layer.forward(x, keep)

    def timed(fn, reps):
        t_end = time.perf_counter() + 0.03          # about 30 ms of the same work first: clock ramp
        while time.perf_counter() < t_end:
            fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    ms_layer = timed(lambda: layer.forward(x), iters)
    # the same layer recorded once into a HIP graph and replayed: no host work between its kernels
    graph, _sx, _sy = T.Transformer.from_layers([layer], p).capture(x)
    ms_layer_graph = timed(graph.replay, iters)
    del graph
    qkv = torch.empty((n, 3 * d), device="cuda", dtype=torch.float32)
    out_d = torch.empty((n, d), device="cuda", dtype=torch.float32)
    out_f = torch.empty((n, p.ffn_hidden_dim), device="cuda", dtype=torch.float32)
    q, k, v = (qkv[:, i * d:(i + 1) * d] for i in range(3))
    w1, b1 = layer.norm["attention_norm"]
    stages = {}
    if layer.qkv_group is not None and layer.qkv_group.fused_cols == 3 * d:
        stages["qkv (one search, one gather into [q|k|v])"] = lambda: layer.qkv_group.run_fused_ptr(x.data_ptr(), n, qkv.data_ptr())
    for i, name in enumerate(("q", "k", "v")):   # the attention stage reads this layer's own projections
        qkv[:, i * d:(i + 1) * d].copy_(keep[name])
    stages["attention"] = lambda: ctx.attention_ptr(q.data_ptr(), k.data_ptr(), v.data_ptr(), out_d.data_ptr(), p.batch_size,
                                                    p.seq_len, p.head_num, p.head_dim, q.stride(0), d, 0.125)
    stages["o"] = lambda: layer.amm["o"].run_ptr(keep["attn"].data_ptr(), n, out_d.data_ptr())
    stages["attention_norm (+ residual)"] = lambda: ctx.layer_norm((keep["o"].data_ptr(), n, d), w1.data_ptr(), b1.data_ptr(),
                                                                   x.data_ptr(), out_d.data_ptr(), 1e-6)
    stages["ffn1 (+ GELU in the epilogue)"] = lambda: layer.amm["ffn1"].run_ptr(keep["h"].data_ptr(), n, out_f.data_ptr())
    stages["ffn2"] = lambda: layer.amm["ffn2"].run_ptr(keep["gelu"].data_ptr(), n, out_d.data_ptr())
    stages["ffn_norm (+ residual)"] = lambda: ctx.layer_norm((keep["ffn2"].data_ptr(), n, d), w1.data_ptr(), b1.data_ptr(),
                                                             keep["h"].data_ptr(), out_d.data_ptr(), 1e-6)
    per_stage = {name: round(timed(fn, iters) * 1e3, 1) for name, fn in stages.items()}
    layer.close()
    return {"tokens": n, "token_dim": d, "head_num": p.head_num, "ffn_hidden_dim": p.ffn_hidden_dim,
            "ms_per_layer": ms_layer, "tokens_per_s": n / (ms_layer * 1e-3), "ms_per_layer_graph": ms_layer_graph,
            "tokens_per_s_graph": n / (ms_layer_graph * 1e-3), "stage_us": per_stage,
            "note": "ms_per_layer: the whole forward, launched op by op from Python; ms_per_layer_graph: replayed from a HIP graph; stage_us: each stage launched on "
                    "its own, back to back with itself (inputs warm in the caches, no allocation between launches)"}


def cpu_baseline(shapes, N, warmup=10, rounds=20, budget_s=25.0):
    """The oracle's restatement of the reference's amm_cpu (test_amm.cpp:126-183) on this host's cores, on the
    full batch of both AMMs, with the reference driver's protocol (test_amm.cpp:21-22,290-314: 10 warm-up and
    20 timed rounds, mean wall time).  Bounded: if the first round says the protocol would exceed budget_s, the
    round counts shrink in proportion (and the sample string says so)."""
    import oracle

    threads = oracle.max_threads()
    rng = np.random.default_rng(1)
    work = []
    for (K, v, C, M) in shapes:
        CB = K // v
        x = rng.standard_normal((N, K), dtype=np.float32)
        cent = rng.standard_normal((CB, C, v)).astype(np.float32)
        lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
        bias = np.zeros(M, np.float32)
        scratch = (np.empty((N, CB), np.uint16), np.empty((N, M), np.int32), np.empty((N, M), np.float32))
        work.append((x, cent, lut, bias, v, scratch))

    def one_pass():
        for x, cent, lut, bias, v, scratch in work:
            oracle.amm_cpu(x, cent, lut, bias, v, 0.01, 0.0, threads=threads, scratch=scratch)

    t0 = time.perf_counter()
    one_pass()  # first warm-up round, timed only to bound the rest
    t1 = time.perf_counter() - t0
    shrink = min(1.0, budget_s / max(t1 * (warmup + rounds), 1e-9))
    warmup, rounds = max(1, int(warmup * shrink)), max(2, int(rounds * shrink))
    for _ in range(warmup - 1):
        one_pass()
    t0 = time.perf_counter()
    for _ in range(rounds):
        one_pass()
    dt = (time.perf_counter() - t0) / rounds
    eff = sum(2.0 * N * K * M for (K, _, _, M) in shapes)
    return {"value": N / dt, "unit": "tokens/s", "cores": threads, "kind": "port", "eff_gops": eff / dt / 1e9,
            "sample": f"all {N} tokens through both AMMs of the pair, {rounds} timed rounds after {warmup} warm-up "
                      f"(the reference driver's protocol is 20 after 10), oracle amm_cpu built with the reference's "
                      f"flags (-O3 -fopenmp, no -march), {threads} OpenMP threads, {dt * 1e3:.1f} ms per round"}


def check_pair(amms, shapes, x1, x2, h, y, N, sample=64):
    """Bit-compares `sample` rows of both outputs of the timed step with the oracle's amm_cpu on the same inputs
    (indices, int32 sums and the fp32 epilogue all enter the compared bits).  Raises on a mismatch."""
    import oracle
    rows = np.sort(np.random.default_rng(5).choice(N, size=sample, replace=False))
    rows[0], rows[-1] = 0, N - 1
    for amm, (K, v, C, M), x, out in zip(amms, shapes, (x1, x2), (h, y)):
        xs = x[rows].cpu().numpy()
        got = out[rows].cpu().numpy()
        want, _, _ = oracle.amm_cpu(xs, amm.h_centroids, amm.h_lut, amm.h_bias, v, float(amm.h_scales[0]), 0.0,
                                    threads=min(16, oracle.max_threads()))
        if not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
            bad = int((got.view(np.uint32) != want.view(np.uint32)).sum())
            raise SystemExit(f"bench.py: the timed {K}->{M} launch differs from the oracle in {bad} of {want.size} sampled outputs")
    return True


def settled_profile(amm, x, N, y, iters):
    """pimdl_amm_profile after enough warm-up launches (about 30 ms of them) for the engine clock to have ramped
    up again: preparing an operator on the host leaves the GPU idle for a second, and the clock drops meanwhile."""
    t = amm.profile(x.data_ptr(), N, y.data_ptr(), warmup=2, iters=2)
    warm = int(min(2000, max(5, 30.0 / max(t["total_ms"], 1e-3))))
    return amm.profile(x.data_ptr(), N, y.data_ptr(), warmup=warm, iters=iters)


def per_codebook_scale(pimdl, ctx, rng, N, shapes, iters=20):
    """The same pair with one fp32 scale per codebook (scale_group = 1), the wording of the benchmark
    configuration; the reference itself has one scale per tensor, which is what `value` measures.  A different
    scale per codebook rules out integer accumulation across codebooks: the table is resident as fp32 integers
    (already multiplied by its codebook's scale: one rounding, as the definition has it) and gathered by the
    fp32-table kernel (VALU adds), so this mode runs at that kernel's rate."""
    import torch
    out = []
    for (K, v, C, M) in shapes:
        CB = K // v
        cent = rng.standard_normal((CB, C, v)).astype(np.float32)
        W = (rng.standard_normal((K, M)) * 0.02).astype(np.float32)
        lut, scales = ctx.lutgen(cent, W, pimdl.LUT_I8, 1)
        amm = ctx.amm(cent, lut, scales, None, max_n=N, scale_group=1)
        x = torch.randn((N, K), device="cuda", dtype=torch.float32)
        y = torch.empty((N, M), device="cuda", dtype=torch.float32)
        t = settled_profile(amm, x, N, y, iters)
        out.append({"K": K, "M": M, "ccs_ms": t["ccs_ms"], "gather_ms": t["gather_ms"], "amm_ms": t["total_ms"],
                    "gather_kernel": amm.last_gather_kernel()})
        amm.close()
    total = sum(o["amm_ms"] for o in out)
    return {"scale_group": 1, "per_amm": out, "ms_per_step": total, "tokens_per_s": N / (total * 1e-3),
            "note": "extension (one scale per codebook is not in the reference); int32 sum inside a group, fp32 "
                    "across groups in ascending order; bit-identical to the oracle's statement of it"}


def vit_sweep(pimdl, ctx, iters=10):
    """ViT-Base/16 feed-forward shapes (N = 64 x 197 = 12608) over sub_vec_len x num_centroid x LUT type:
    device time of the two kernels of each operator."""
    import torch
    N = 64 * 197
    rng = np.random.default_rng(4)
    cells = []
    for (K, M) in ((768, 3072), (3072, 768)):
        x = torch.randn((N, K), device="cuda", dtype=torch.float32)
        y = torch.empty((N, M), device="cuda", dtype=torch.float32)
        for v in (2, 4, 8):
            for C in (8, 16, 32):
                CB = K // v
                cent = rng.standard_normal((CB, C, v)).astype(np.float32)
                for kind in ("i8", "f32"):
                    if kind == "i8":
                        lut, scales = rng.integers(-128, 128, (CB, C, M)).astype(np.int8), np.float32(0.01)
                    else:
                        lut, scales = rng.standard_normal((CB, C, M), dtype=np.float32), None
                    amm = ctx.amm(cent, lut, scales, None, max_n=N)
                    t = settled_profile(amm, x, N, y, iters)
                    e = 1 if kind == "i8" else 4
                    cells.append({"K": K, "M": M, "v": v, "C": C, "lut": kind, "ccs_us": round(t["ccs_ms"] * 1e3, 1),
                                  "gather_us": round(t["gather_ms"] * 1e3, 1),
                                  "mtok_per_s": round(N / (t["total_ms"] * 1e-3) / 1e6, 1),
                                  "gather_lds_frac": round(e * N * CB * M / (t["gather_ms"] * 1e-3) / 1e9 / LDS_PEAK_GBPS, 3),
                                  "gather_kernel": amm.last_gather_kernel().split("<")[0]})
                    amm.close()
                    del lut
    return {"tokens": N, "cells": cells}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--no-model", action="store_true", help="skip the 12-layer model forward timing")
    ap.add_argument("--no-large-layer", action="store_true", help="skip the BERT-large layer timing")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sweep", action="store_true", help="skip the ViT-Base sweep and the per-codebook-scale pair")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the path shards over tokens with no exchange; "
              "nothing to measure across GPUs); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from __graft_entry__ import load_package

    pimdl = load_package()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    ctx = pimdl.Context(0)
    stream = torch.cuda.current_stream()
    ctx.set_stream(stream.cuda_stream)

    N, v, C = args.tokens, 4, 16
    shapes = [(768, v, C, 3072), (3072, v, C, 768)]
    rng = np.random.default_rng(0)
    amms = []
    for (K, vv, CC, M) in shapes:
        cent, lut, scales, bias = synth_amm(rng, K, vv, CC, M, pimdl, ctx)
        amm = ctx.amm(cent, lut, scales, bias, max_n=N)
        amm.h_centroids, amm.h_lut, amm.h_scales, amm.h_bias = cent, lut, np.atleast_1d(scales), bias   # for check_pair
        amms.append(amm)

    gen = torch.Generator(device="cuda").manual_seed(0)
    x1 = torch.randn((N, 768), device="cuda", generator=gen, dtype=torch.float32)
    h = torch.empty((N, 3072), device="cuda", dtype=torch.float32)
    y = torch.empty((N, 768), device="cuda", dtype=torch.float32)
    # FFN2's input: GELU of FFN1's output, computed once outside the timed region (the activation
    # function is not part of the LUT-AMM path)
    amms[0].run_ptr(x1.data_ptr(), N, h.data_ptr())
    ctx.synchronize()
    x2 = torch.nn.functional.gelu(h).contiguous()
    torch.cuda.synchronize()

    def step():
        amms[0].run_ptr(x1.data_ptr(), N, h.data_ptr())
        amms[1].run_ptr(x2.data_ptr(), N, y.data_ptr())

    # Untimed pre-heat, whatever --warmup says: after an idle period the engine clock takes about 20 ms of this
    # load to ramp up, and until then everything runs 15-20 % slower.  Then the W warm-up steps, then exactly K
    # timed steps between two synchronisations.
    settle_steps = 0
    t_end = time.perf_counter() + CLOCK_SETTLE_S
    while time.perf_counter() < t_end:
        for _ in range(50):
            step()
        torch.cuda.synchronize()
        settle_steps += 50
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(args.steps):
        step()
    e1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ev_ms = e0.elapsed_time(e1) / args.steps
    ms_per_step = wall_ms

    # The outputs the timed steps left behind, against the oracle on a 64-row sample (rows are independent): the
    # exact launches that were timed, not a separate test run.
    checked = check_pair(amms, shapes, x1, x2, h, y, N)

    # per-kernel device times: HIP events on the launch stream, each kernel launched on its own (pimdl_amm_profile)
    prof = [amms[0].profile(x1.data_ptr(), N, h.data_ptr(), warmup=200, iters=max(50, args.steps)),
            amms[1].profile(x2.data_ptr(), N, y.data_ptr(), warmup=200, iters=max(50, args.steps))]
    per_amm = []
    for name, (K, vv, CC, M), p in zip(("ffn1", "ffn2"), shapes, prof):
        ab = algorithmic_bytes(N, K, vv, CC, M)
        per_amm.append({
            "name": name, "K": K, "M": M, "ccs_ms": p["ccs_ms"], "gather_ms": p["gather_ms"], "amm_ms": p["total_ms"],
            "tokens_per_s": N / (p["total_ms"] * 1e-3), "eff_gops": ab["eff_ops"] / (p["total_ms"] * 1e-3) / 1e9,
            "ccs_hbm_gbps": ab["ccs_hbm"] / (p["ccs_ms"] * 1e-3) / 1e9,
            "ccs_hbm_frac": ab["ccs_hbm"] / (p["ccs_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "gather_lds_gbps": ab["gather_lds"] / (p["gather_ms"] * 1e-3) / 1e9,
            "gather_lds_frac": ab["gather_lds"] / (p["gather_ms"] * 1e-3) / 1e9 / LDS_PEAK_GBPS,
            "gather_hbm_gbps": ab["gather_hbm"] / (p["gather_ms"] * 1e-3) / 1e9,
            "gather_hbm_frac": ab["gather_hbm"] / (p["gather_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "geometry": None,
        })
    for pa, amm in zip(per_amm, amms):
        pa["geometry"] = amm.geometry()
        pa["gather_kernel"] = amm.last_gather_kernel()

    # Dominant kernel: the longer of the two gathers.  Its roofline is the one the metric is worded in: LUT
    # entries gathered per second, N*CB*M algorithmic bytes per launch, over the LDS read peak.  How the kernel
    # gets there (one-hot products on the matrix cores, which execute 16 multiply-adds per gathered entry) is
    # reported beside it as utilisation of the units it occupies, not as a roofline fraction.
    dom = max(per_amm, key=lambda d: d["gather_ms"])
    K, M = dom["K"], dom["M"]
    ab = algorithmic_bytes(N, K, v, C, M)
    _, lds_measured = ctx.diag_bandwidth(copy=False, lds=True)
    mt = MEASURED_GATHER_TRAFFIC.get((dom["gather_kernel"], N, K, M))
    traffic = (mt["fetch_kib"] * FETCH_SCALE + mt["write_kib"] * WRITE_SCALE) * 1024.0 if mt else None
    sparse = dom["gather_kernel"].startswith("gather_sparse")
    cb_per_instr = 8 if sparse else 4               # codebooks one matrix instruction covers for 16 tokens x 16 columns
    instrs = N / 16 * (M / 16) * (K // v) / cb_per_instr
    simds = 4 * ctx.device_info()["compute_units"]
    roofline = {
        "kernel": f"{dom['gather_kernel']} ({dom['name']}: K={K} M={M})",
        "bound": "lds",
        "kind": "algorithmic",   # N*CB*M gathered bytes per launch over the LDS read peak: the roofline the metric is
                                 # worded in.  The kernel gathers through one-hot products on the sparse matrix
                                 # instruction and does not move those bytes through LDS; the units it does occupy are
                                 # under "matrix_core" and "lds_counters" (utilisation, not rooflines).
        "achieved": dom["gather_lds_gbps"], "peak": LDS_PEAK_GBPS, "unit": "GB/s", "frac": dom["gather_lds_frac"],
        "algorithmic_bytes_per_launch": ab["gather_lds"],
        "avg_launch_ms": dom["gather_ms"],
        "traffic": traffic,
        "traffic_source": ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this script for this kernel and batch, scaled "
                           "x2.0 / x1.0 (copy-kernel calibration); profiles/bench_ffn_pair_hbm_traffic.txt") if mt else
                          "not collected for the kernel this run launched",
        "lds_peak_measured_gbps": lds_measured,
        "frac_of_measured_lds_peak": dom["gather_lds_gbps"] / lds_measured if lds_measured else None,
        "hbm": {"achieved": dom["gather_hbm_gbps"], "peak": HBM_PEAK_GBPS, "frac": dom["gather_hbm_frac"],
                "algorithmic_bytes_per_launch": ab["gather_hbm"]},
        # utilisation, not a roofline: matrix instructions issued per launch x 16 clocks each over the SIMDs' time
        "matrix_core": {"instruction": "v_smfmac_i32_16x16x128_i8" if sparse else "v_mfma_i32_16x16x64_i8",
                        "instructions_per_launch": instrs,
                        "busy_frac": instrs * 16.0 / (simds * 2.4e9 * dom["gather_ms"] * 1e-3),
                        "dense_equivalent_tops": 2.0 * N * (K // v) * 16 * M / (dom["gather_ms"] * 1e-3) / 1e12,
                        "dense_int8_peak_tops": MFMA_I8_PEAK_TOPS},
        "north_star_target_frac": 0.5,
    }
    lc = MEASURED_GATHER_COUNTERS.get((dom["gather_kernel"], N, K, M))
    roofline["lds_counters"] = dict(lc, source="rocprofv3 --pmc of this script for this kernel and batch; "
                                    "profiles/bench_ffn_pair_lds_mfma_counters.txt") if lc else None
    # the step as a whole on the same roofline: both gathers' algorithmic bytes over the whole step (searches included)
    step_lds = sum(algorithmic_bytes(N, K_, v, C, M_)["gather_lds"] for (K_, _, _, M_) in shapes)
    roofline["step_frac"] = step_lds / (ms_per_step * 1e-3) / 1e9 / LDS_PEAK_GBPS

    total_eff_ops = sum(algorithmic_bytes(N, K_, v, C, M_)["eff_ops"] for (K_, _, _, M_) in shapes)
    result = {
        "metric": "LUT-AMM tokens/s (BERT-base FFN pair, N=8192)",
        "value": N / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "clock_settle_steps": settle_steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8", "data": "synthetic",
        "config": {"workload": "BERT-base FFN pair as LUT-AMM: N=8192 (64x128) fp32 activations N(0,1); "
                               "768->3072 and 3072->768, vec_len=4, 16 centroids/codebook, int8 LUT with the "
                               "reference's per-tensor fp32 scale, int32 accumulate, random-init centroids/weights",
                   "tokens": N, "vec_len": v, "num_centroid": C},
        "eff_gops": total_eff_ops / (ms_per_step * 1e-3) / 1e9,
        "device_ms_per_step": ev_ms,
        "per_amm": per_amm,
        "roofline": roofline,
    }
    # The same pair with pageable HOST buffers in and out (what the reference's amm_host signature hands
    # over): 25 + 100 MB up and 100 + 25 MB down per step through the context's staging buffers.
    # A labelled secondary figure; `value` above is the HBM-resident rate.
    xh = np.random.default_rng(1).standard_normal((N, 768)).astype(np.float32)
    hh, yh = np.empty((N, 3072), np.float32), np.empty((N, 768), np.float32)
    host_steps = []
    for it in range(8):
        t0 = time.perf_counter()
        amms[0].run_ptr(xh.ctypes.data, N, hh.ctypes.data)
        amms[1].run_ptr(hh.ctypes.data, N, yh.ctypes.data)
        host_steps.append((time.perf_counter() - t0) * 1e3)
    host_ms = float(np.mean(host_steps[3:]))   # the first steps fault the fresh host buffers in and size the staging ring
    legs = ctx.diag_host_copy(100 << 20)
    link_floor_ms = sum(4.0 * N * max(K_, M_) for (K_, _, _, M_) in shapes) / (min(legs["h2d_gbps"], legs["d2h_gbps"]) * 1e9) * 1e3
    host_buffers = {"ms_per_step": host_ms, "tokens_per_s": N / (host_ms * 1e-3), "steps_ms": [round(t, 2) for t in host_steps],
                    "legs_gbps": {k: round(val, 1) for k, val in legs.items()},
                    "link_floor_ms": link_floor_ms,
                    "note": "pageable host memory in and out of both AMMs (what the reference's amm_host signature hands "
                            "over), mean of the last 5 of 8 steps: chunks of tokens through pinned staging buffers, copies by the host thread "
                            "pool, transfers and kernels overlapped on three streams.  link_floor_ms: the wider side of "
                            "each AMM (100 MB) over the measured pinned-memory link rate, both directions overlapped"}
    # The large objects first, the small ones last (a reader that keeps only the end of the line keeps those).
    if not args.no_sweep:
        result["vit_base_sweep"] = vit_sweep(pimdl, ctx)
        result["per_codebook_scale"] = per_codebook_scale(pimdl, ctx, rng, N, shapes)
    result["host_buffers"] = host_buffers
    if not args.no_model:
        if not args.no_large_layer:
            result["bert_large_layer"] = bert_large_layer(pimdl, ctx)
        result["bert_base_forward"] = model_forward(pimdl, ctx)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(shapes, N)
    result["checked"] = checked
    result["summary"] = {
        "tokens_per_s": result["value"], "ms_per_step": ms_per_step, "checked_against_oracle": checked,
        "roofline_frac": roofline["frac"], "roofline_step_frac": roofline["step_frac"],
        "gather_us": [round(p["gather_ms"] * 1e3, 1) for p in per_amm], "search_us": [round(p["ccs_ms"] * 1e3, 1) for p in per_amm],
        "host_buffers_ms": round(host_ms, 2),
        "bert_base_forward_ms": round(result["bert_base_forward"]["ms_per_forward_graph"], 3) if "bert_base_forward" in result else None,
        "bert_large_layer_ms": round(result["bert_large_layer"]["ms_per_layer_graph"], 3) if "bert_large_layer" in result else None,
        "per_codebook_scale_ms": round(result["per_codebook_scale"]["ms_per_step"], 3) if "per_codebook_scale" in result else None,
        "cpu_tokens_per_s": round(result["cpu_baseline"]["value"]) if "cpu_baseline" in result else None,
    }
    for a in amms:
        a.close()
    ctx.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
