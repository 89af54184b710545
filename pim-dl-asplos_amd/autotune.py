"""Measured tile search for a LUT-AMM operator.

The reference ships an auto-tuner that enumerates DPU tilings and ranks them with an analytic latency
model of UPMEM hardware (inference-engine/src/tuner/auto_tuner.cpp:368-603; input and output are YAML files,
:793-820).  That model has no meaning on a GPU, so the counterpart here measures: for one operator shape it
builds the operator with every column-tile width the gather kernel offers, times the two kernels with
events on the device (pimdl_amm_profile) and keeps the fastest.  The result is cached in a JSON file keyed
by device and shape, and can be written in the reference's single-kernel YAML layout with the chosen tile
under kernel_params.

    python autotune.py --n 8192 --k 768 --m 3072 --vec_len 4 --ncentroids 16 [--cache tiles.json] [--yaml out.yaml]
"""
import argparse
import json
import os
import sys

import numpy as np

CANDIDATES = (0, 48, 64, 96)   # 0 = the library's own load-balance choice


def shape_key(device, n, K, v, C, M, dtype):
    return f"{device}|n={n}|k={K}|v={v}|c={C}|m={M}|{dtype}"


def tune(ctx, pimdl, n, K, v, C, M, lut_dtype="int8", seed=0, iters=20, candidates=CANDIDATES):
    """Returns (best col_block, {col_block: {"ccs_ms", "gather_ms", "total_ms"}}); widths the operator's
    kernel does not offer are skipped."""
    import torch
    rng = np.random.default_rng(seed)
    CB = K // v
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    if lut_dtype == "int8":
        lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
        scales = np.float32(0.01)
    else:
        lut = rng.standard_normal((CB, C, M)).astype(np.float32)
        scales = None
    x = torch.randn((n, K), device="cuda", dtype=torch.float32)
    y = torch.empty((n, M), device="cuda", dtype=torch.float32)
    results = {}
    for cb in candidates:
        try:
            amm = ctx.amm(cent, lut, scales, None, max_n=n, col_block=cb)
        except pimdl.PimdlError as e:
            if e.code == pimdl.ERR_INVALID:
                continue  # no kernel variant of that width for this operator
            raise
        t = amm.profile(x.data_ptr(), n, y.data_ptr(), warmup=3, iters=iters)
        geo = amm.geometry()
        results[cb] = {"ccs_ms": t["ccs_ms"], "gather_ms": t["gather_ms"], "total_ms": t["total_ms"],
                       "col_block": geo["col_block"]}
        amm.close()
    if not results:
        raise RuntimeError("no candidate could be built")
    # the fastest explicit width; "auto" (0) only documents what the library would have picked
    explicit = [c for c in results if c != 0]
    best = min(explicit, key=lambda c: results[c]["gather_ms"]) if explicit else results[0]["col_block"]
    return best, results


class TileCache:
    """JSON file {shape key: col_block}."""

    def __init__(self, path):
        self.path = path
        self.table = {}
        if path and os.path.exists(path):
            with open(path) as f:
                self.table = json.load(f)

    def get(self, key):
        return int(self.table.get(key, 0))

    def put(self, key, col_block):
        self.table[key] = int(col_block)
        if self.path:
            with open(self.path, "w") as f:
                json.dump(self.table, f, indent=1, sort_keys=True)


def write_yaml(path, n, K, v, C, M, col_block, timing):
    """The reference's single-kernel YAML layout (inference-engine/configs/single_kernel_output_example.yaml)
    with the measured choice; the DPU-only keys are left out."""
    import yaml
    doc = {"amm_shape_params": {"n": n, "input_feature_len": K, "num_codebook": K // v, "num_centroid": C,
                                "output_feature_len": M, "scale": 0.1, "bias": 0.0},
           "kernel_params": {"col_block": int(col_block), "gather_ms": float(timing["gather_ms"]),
                             "ccs_ms": float(timing["ccs_ms"])}}
    with open(path, "w") as f:
        yaml.safe_dump(doc, f, sort_keys=False)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--n", type=int, required=True)
    ap.add_argument("--k", type=int, required=True)
    ap.add_argument("--m", type=int, required=True)
    ap.add_argument("--vec_len", type=int, default=4)
    ap.add_argument("--ncentroids", type=int, default=16)
    ap.add_argument("--lut_dtype", choices=("int8", "fp32"), default="int8")
    ap.add_argument("--cache", type=str, default=None)
    ap.add_argument("--yaml", type=str, default=None)
    args = ap.parse_args(argv)
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.dirname(here))
    from __graft_entry__ import load_package
    pimdl = load_package()
    ctx = pimdl.Context(0)
    try:
        best, results = tune(ctx, pimdl, args.n, args.k, args.vec_len, args.ncentroids, args.m, args.lut_dtype)
        dev = ctx.device_info()["name"]
    finally:
        ctx.close()
    for cb, r in sorted(results.items()):
        print(f"col_block {cb if cb else 'auto(' + str(r['col_block']) + ')':>9}: search {r['ccs_ms'] * 1e3:7.1f} us, "
              f"gather {r['gather_ms'] * 1e3:7.1f} us")
    print(f"best col_block: {best}")
    if args.cache:
        TileCache(args.cache).put(shape_key(dev, args.n, args.k, args.vec_len, args.ncentroids, args.m, args.lut_dtype), best)
    if args.yaml:
        write_yaml(args.yaml, args.n, args.k, args.vec_len, args.ncentroids, args.m, best,
                   results[best] if best in results else results[0])
    return 0


if __name__ == "__main__":
    sys.exit(main())
