"""Weight converter: calibrated LUT-NN checkpoint -> the inference engine's weight file, LUTs built on the GPU.

Counterpart of the reference's model-calibration/pim_weight_converter.py (argument names :8-18, key handling
:38-57, per-linear shapes :74-85, LUT = bmm(centroids, weight) :86-91, quantisation :21-35, output keys
:93-96).  Input: a safetensors (or .npz) file whose encoder-layer tensors are named
"...layer.{L}.{op}.weight" (the dense weight stored as [in_features][out_features], i.e. Linear.weight^T),
"...layer.{L}.{op}.centroids.weight" ([CB][C*v]), "...layer.{L}.{op}.bias" and the LayerNorm tensors.  Output:
an .npz with, per linear, "{L}.{op}.centroids.weight", "{L}.{op}.lut.tensor" (int8 [CB*C][M], or float32 with
--lut_dtype fp32), "{L}.{op}.lut.scale", "{L}.{op}.lut.bias" (0-d float32), "{L}.{op}.bias", and every other
layer tensor unchanged.  The matrix product and the quantisation run in libpimdl (pimdl_lutgen)."""
import argparse
import os
import re
import sys

import numpy as np


def parse_args(argv=None):
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--weight_input_file", type=str, required=True)
    parser.add_argument("--features", type=int, default=768)
    parser.add_argument("--ncentroids", type=int, default=16)
    parser.add_argument("--vec_len", type=int, default=2)
    parser.add_argument("--nsharecodebook", type=int, default=1)
    parser.add_argument("--weight_output_file", type=str, required=True)
    parser.add_argument("--lut_dtype", choices=("int8", "fp32"), default="int8",
                        help="fp32 keeps the unquantised table (scale 1, bias 0); not in the reference")
    parser.add_argument("--ordered_sum", action="store_true",
                        help="add the products of a table entry in ascending order with separately rounded fp32 "
                             "operations (bit for bit a scalar CPU loop) instead of on the matrix instruction")
    return parser.parse_args(argv)


def read_tensors(path):
    """All tensors of a safetensors or .npz file as numpy arrays (nothing in the file is executed)."""
    if path.endswith(".npz"):
        z = np.load(path, allow_pickle=False)
        return {k: z[k] for k in z.files}
    from safetensors import safe_open
    out = {}
    with safe_open(path, framework="numpy") as f:
        for k in f.keys():
            out[k] = f.get_tensor(k)
    return out


def split_layers(tensors):
    """{layer id: {"{L}.rest.of.key": array}} for every key that names an encoder layer; embeddings and
    anything outside the layers are dropped, as in the reference (:42-55)."""
    layers = {}
    for k, t in tensors.items():
        parts = k.split(".")
        if "embeddings" in parts:
            continue
        m = re.search(r"(?:^|\.)layer\.(\d+)\.(.*)$", k)
        if not m:
            continue
        layers.setdefault(int(m.group(1)), {})[f"{m.group(1)}.{m.group(2)}"] = t
    return layers


def linear_shape(op_name, features):
    """in/out features of a linear from its name (:74-81): attention and intermediate layers read
    `features`, output layers (not attention.output) read 4*features; attention and output layers write
    `features`, intermediate layers 4*features."""
    in_features = features if ("attention" in op_name or "intermediate" in op_name) else features * 4
    out_features = features if ("attention" in op_name or "output" in op_name) else features * 4
    return in_features, out_features


def convert(tensors, ctx, pimdl, features=768, ncentroids=16, vec_len=2, nsharecodebook=1, lut_dtype="int8",
            ordered_sum=False):
    if nsharecodebook != 1:
        # The reference divides the codebook count by it (pim_weight_converter.py:82, LUTLinear_t.py:26) and then views
        # the [in][out] weight and the activations as [ncodebooks][vec_len][...] (pim_weight_converter.py:86,
        # LUTLinear_t.py:68-69), which only has the right number of elements for 1: its own code raises for any other
        # value, and its inference engine has one codebook per sub-vector (index_calc_host.cpp:22).
        raise ValueError("nsharecodebook != 1 is not supported: the reference's own converter and LUTLinear_t.forward fail "
                         "on it (a [in][out] weight cannot be viewed as [in/vec_len/nsharecodebook][vec_len][out])")
    layers = split_layers(tensors)
    out = {}
    for _li, lt in sorted(layers.items()):
        weights = {k[:-len(".weight")]: v for k, v in lt.items()
                   if k.endswith(".weight") and not k.endswith(".centroids.weight") and "LayerNorm" not in k}
        for op, W in weights.items():
            cent = lt.get(op + ".centroids.weight")
            if cent is None:
                raise ValueError(f"{op}: dense weight without centroids")
            in_f, out_f = linear_shape(op, features)
            CB = in_f // vec_len
            W = np.ascontiguousarray(W, np.float32).reshape(in_f, out_f)
            cent3 = np.ascontiguousarray(cent, np.float32).reshape(CB, ncentroids, vec_len)
            if lut_dtype == "int8":
                lut, scales = ctx.lutgen(cent3, W, pimdl.LUT_I8, 0, ordered=ordered_sum)
                scale = np.float32(scales[0])
            else:
                lut, _ = ctx.lutgen(cent3, W, pimdl.LUT_F32, 0, ordered=ordered_sum)
                scale = np.float32(1.0)
            out[op + ".lut.tensor"] = lut.reshape(CB * ncentroids, out_f)
            out[op + ".lut.scale"] = np.asarray(scale, np.float32).reshape(())
            out[op + ".lut.bias"] = np.asarray(0.0, np.float32).reshape(())   # -scale * zero_point, zero_point = 0
        for k, v in lt.items():
            if k.endswith(".weight") and k[:-len(".weight")] in weights:
                continue  # replaced by the LUT
            out[k] = np.asarray(v)
    return out


def main(argv=None):
    args = parse_args(argv)
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.dirname(here))
    from __graft_entry__ import load_package
    pimdl = load_package()
    ctx = pimdl.Context(0)
    try:
        out = convert(read_tensors(args.weight_input_file), ctx, pimdl, args.features, args.ncentroids, args.vec_len,
                      args.nsharecodebook, args.lut_dtype, args.ordered_sum)
    finally:
        ctx.close()
    np.savez(args.weight_output_file, **out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
