"""Stage-by-stage check of one encoder layer on the GPU against the CPU oracle, on a sample of rows.

LUT-AMM is discontinuous, so each stage is compared against the oracle given the GPU's own input to that
stage (op order and residual placement: inference-engine/src/host/transformer_layer.cpp:263-625).
Bars: every LUT-AMM bit-exact; layer normalisation (transformer_layer.cpp:50-90) within 1e-5 relative;
attention and tanh-GELU against their float64 definitions (the reference computes them with ggml, which
none of its tests pins).  Rows of every stage but attention are independent, so a row sample is a full
check of those rows; attention is checked on whole (batch, head) pairs."""
import math

import numpy as np

import oracle

THREADS = 8


def amm_oracle(w, x, bias_mode=1):
    """index_calculation + gather + pim_lut's epilogue (bias * num_codebook) for the rows of x."""
    cent = w["centroids"]
    CB, _, v = cent.shape
    idx = oracle.index_calculation(np.ascontiguousarray(x), cent, v, threads=THREADS)
    acc = oracle.gather_i8(idx, w["lut"], threads=THREADS)
    return oracle.dequant(acc, w["bias"], CB, w["scale"], w.get("lut_bias", 0.0), bias_mode, threads=THREADS)


def gelu_tanh64(f):
    f = f.astype(np.float64)
    return 0.5 * f * (1 + np.tanh(math.sqrt(2 / math.pi) * (f + 0.044715 * f ** 3)))


def check_layer_stages(weights, params, x, keep, rows, attn_pairs, fused_gelu=True):
    """weights: the layer's host weights; x: the layer's input (torch CUDA tensor); keep: the intermediates
    TransformerLayer.forward recorded (torch CUDA tensors); rows: token rows to check; attn_pairs: (batch, head)
    pairs whose attention output is recomputed in float64."""
    rows = np.asarray(rows)
    p = params

    def host(t):
        if t is None:
            return None
        import torch
        return t[torch.as_tensor(rows, device=t.device)].contiguous().cpu().numpy()

    xs = host(x)
    k = {name: host(t) for name, t in keep.items()}
    # the six LUT-AMMs, each from the GPU's own input rows: bit-exact
    for name, src in (("q", xs), ("k", xs), ("v", xs), ("o", k["attn"]), ("ffn1", k["h"]), ("ffn2", k["gelu"])):
        want = amm_oracle(weights[name], src)
        if name == "ffn1" and fused_gelu:
            # the operator's epilogue applies GELU to exactly these values; only its rounding is left
            np.testing.assert_allclose(k["gelu"], gelu_tanh64(want), rtol=2e-6, atol=1e-7, err_msg="gelu(ffn1)")
            continue
        assert np.array_equal(k[name].view(np.uint32), want.view(np.uint32)), \
            f"{name}: {(k[name] != want).sum()} of {want.size} outputs differ from the oracle"
    if not fused_gelu:
        np.testing.assert_allclose(k["gelu"], gelu_tanh64(k["ffn1"]), rtol=1e-4, atol=1e-5)
    # residual + LayerNorm in the reference's placement: h = x + norm(o), out = h + norm(ffn2)
    for res, src, dst, nm in ((xs, "o", "h", "attention_norm"), (k["h"], "ffn2", "out", "ffn_norm")):
        ln = oracle.layer_norm(k[src], weights[nm]["weight"], weights[nm]["bias"])
        np.testing.assert_allclose(k[dst], res + ln, rtol=1e-5, atol=1e-5, err_msg=dst)
    # attention: softmax(q k^T / sqrt(head_dim)) v, unmasked, per (batch, head)
    S, hd = p.seq_len, p.head_dim
    for (b, h) in attn_pairs:
        tok = slice(b * S, (b + 1) * S)
        col = slice(h * hd, (h + 1) * hd)
        q, kk, v = (keep[n][tok, col].double().cpu().numpy() for n in ("q", "k", "v"))
        s = q @ kk.T / math.sqrt(hd)
        s = np.exp(s - s.max(-1, keepdims=True))
        want = (s / s.sum(-1, keepdims=True)) @ v
        np.testing.assert_allclose(keep["attn"][tok, col].cpu().numpy(), want, rtol=1e-4, atol=1e-4,
                                   err_msg=f"attention batch {b} head {h}")
