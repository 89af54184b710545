"""Encoder layer and model forward of a LUT-NN transformer on one MI355X.

Host-side counterpart of the reference's layer/model code (C++ over ggml and the UPMEM SDK):

    pim_lut_transformer_layer   inference-engine/src/host/transformer_layer.cpp:263-625
    transformer_inference       inference-engine/src/host/transformer_model.cpp:13-49
    weight file (.npz)          inference-engine/test/test_transformer.cpp:246-463, written by
                                model-calibration/pim_weight_converter.py:47-52,93-96
    YAML configuration          inference-engine/src/host/parser.cpp:86-330

Every linear layer is a LUT-AMM operator of libpimdl (closest-centroid search + LUT gather on the GPU);
layer normalisation is libpimdl's pimdl_layer_norm (the reference's norm() statement by statement);
attention is libpimdl's pimdl_attention for head_dim 64 (PyTorch-ROCm's fused attention otherwise) and GELU
runs inside the first feed-forward operator's epilogue.  The reference computes those two with ggml (flash
attention, GELU through an fp16 table); no test of the reference pins their outputs, so here they are the
textbook fp32 definitions: softmax(Q K^T / sqrt(head_dim)) V without a mask, and the tanh form of GELU.  The DPU tile re-orderings between the steps of the reference layer disappear:
every buffer here is row-major [tokens][features].

Op order of one layer (transformer_layer.cpp, "step" comments):
    q, k, v = AMM_q(x), AMM_k(x), AMM_v(x)          (or one fused AMM_qkv)
    a       = attention(q, k, v)
    o       = AMM_o(a)
    h       = x + norm(o; attention LayerNorm)       (:474-486)
    f       = AMM_ffn2(gelu(AMM_ffn1(h)))
    y       = h + norm(f; output LayerNorm)          (:599-611)
"""
import math
import os
import sys
import time
from dataclasses import dataclass, field

import numpy as np

# linear layers of one encoder layer: (short name, key prefix in the weight file)
LINEARS = (("q", "attention.self.query"), ("k", "attention.self.key"), ("v", "attention.self.value"),
           ("o", "attention.output.dense"), ("ffn1", "intermediate.dense"), ("ffn2", "output.dense"))
NORMS = (("attention_norm", "attention.output.LayerNorm"), ("ffn_norm", "output.LayerNorm"))


@dataclass
class AmmShape:
    num_codebook: int
    num_centroid: int
    input_feature_len: int
    output_feature_len: int

    @property
    def sub_vec_len(self):
        return self.input_feature_len // self.num_codebook


@dataclass
class TransformerParams:
    """network_params / kernel_params of the reference's YAML (parser.cpp:104-122 and following)."""
    seq_len: int
    batch_size: int
    head_num: int
    head_dim: int
    token_dim: int
    ffn_hidden_dim: int
    layer_num: int
    shapes: dict = field(default_factory=dict)   # "qkv" | "q","k","v" | "o" | "ffn1" | "ffn2" -> AmmShape

    @property
    def n(self):
        return self.seq_len * self.batch_size

    @classmethod
    def from_yaml(cls, path):
        import yaml
        with open(path) as f:
            cfg = yaml.safe_load(f)
        net, ker = cfg["network_params"], cfg["kernel_params"]
        p = cls(int(net["seq_len"]), int(net["batch_size"]), int(net["head_num"]), int(net["head_dim"]),
                int(net["token_dim"]), int(net["ffn_hidden_dim"]), int(net["layer_num"]))
        if p.head_num * p.head_dim != p.token_dim:
            raise ValueError("head_num * head_dim != token_dim")
        dims = {"qkv": (p.token_dim, 3 * p.token_dim), "o": (p.token_dim, p.token_dim),
                "ffn1": (p.token_dim, p.ffn_hidden_dim), "ffn2": (p.ffn_hidden_dim, p.token_dim)}
        for op, (k_in, m_out) in dims.items():
            p.shapes[op] = AmmShape(int(ker[f"{op}_num_codebook"]), int(ker[f"{op}_num_centroid"]), k_in, m_out)
        for op in ("q", "k", "v"):  # the separate projections share the qkv kernel parameters
            p.shapes[op] = AmmShape(p.shapes["qkv"].num_codebook, p.shapes["qkv"].num_centroid, p.token_dim,
                                    p.token_dim)
        return p

    @classmethod
    def bert_base(cls, batch_size=32, seq_len=128, layer_num=12, sub_vec_len=4, num_centroid=16):
        p = cls(seq_len, batch_size, 12, 64, 768, 3072, layer_num)
        for op, (k_in, m_out) in {"q": (768, 768), "k": (768, 768), "v": (768, 768), "o": (768, 768),
                                  "ffn1": (768, 3072), "ffn2": (3072, 768)}.items():
            p.shapes[op] = AmmShape(k_in // sub_vec_len, num_centroid, k_in, m_out)
        return p


# ------------------------------------------------------------------------------------ weight files

def save_npz(path, layers):
    """Write layer weights with the key names and dtypes of pim_weight_converter.py:93-96:
    "{L}.{prefix}.centroids.weight" f32 [CB][C*v], ".lut.tensor" int8 [CB*C][M], ".lut.scale" / ".lut.bias"
    0-d f32, ".bias" f32 [M]; "{L}.{norm}.weight" / ".bias" f32 [D]."""
    out = {}
    for li, layer in enumerate(layers):
        for name, prefix in LINEARS:
            w = layer[name]
            cent = np.asarray(w["centroids"], np.float32)
            CB, C, v = cent.shape
            lut = np.asarray(w["lut"], np.int8)
            out[f"{li}.{prefix}.centroids.weight"] = cent.reshape(CB, C * v)
            out[f"{li}.{prefix}.lut.tensor"] = lut.reshape(CB * C, lut.shape[-1])
            out[f"{li}.{prefix}.lut.scale"] = np.asarray(w["scale"], np.float32).reshape(())
            out[f"{li}.{prefix}.lut.bias"] = np.asarray(w.get("lut_bias", 0.0), np.float32).reshape(())
            out[f"{li}.{prefix}.bias"] = np.asarray(w["bias"], np.float32)
        for name, prefix in NORMS:
            out[f"{li}.{prefix}.weight"] = np.asarray(layer[name]["weight"], np.float32)
            out[f"{li}.{prefix}.bias"] = np.asarray(layer[name]["bias"], np.float32)
    np.savez(path, **out)


def load_npz(path, params):
    """Read a weight file in the format above; `params` supplies num_centroid per linear (the file
    stores centroids as [CB][C*v] and the LUT as [CB*C][M], test_transformer.cpp:283-299)."""
    z = np.load(path, allow_pickle=False)
    layers = []
    for li in range(params.layer_num):
        layer = {}
        for name, prefix in LINEARS:
            shape = params.shapes[name]
            cent = np.asarray(z[f"{li}.{prefix}.centroids.weight"], np.float32)
            CB = cent.shape[0]
            C = shape.num_centroid
            if CB != shape.num_codebook or cent.shape[1] % C:
                raise ValueError(f"layer {li} {name}: centroid block {cent.shape} does not match the configuration")
            lut = np.asarray(z[f"{li}.{prefix}.lut.tensor"])
            if lut.dtype != np.int8 or lut.shape[0] != CB * C:
                raise ValueError(f"layer {li} {name}: LUT {lut.dtype}{lut.shape} does not match the configuration")
            layer[name] = {"centroids": cent.reshape(CB, C, cent.shape[1] // C), "lut": lut.reshape(CB, C, -1),
                           "scale": float(z[f"{li}.{prefix}.lut.scale"]), "lut_bias": float(z[f"{li}.{prefix}.lut.bias"]),
                           "bias": np.asarray(z[f"{li}.{prefix}.bias"], np.float32)}
        for name, prefix in NORMS:
            layer[name] = {"weight": np.asarray(z[f"{li}.{prefix}.weight"], np.float32),
                           "bias": np.asarray(z[f"{li}.{prefix}.bias"], np.float32)}
        layers.append(layer)
    return layers


# --------------------------------------------------------------------------------------- the layer

class TransformerLayer:
    """One encoder layer resident on the GPU: six LUT-AMM operators and two LayerNorms."""

    def __init__(self, ctx, pimdl, weights, params, fused_qkv=False, side=None, fused_gelu=True):
        """fused_gelu: GELU is applied by the first feed-forward operator's own epilogue instead of a pass of
        its own over the [n][ffn_hidden_dim] tensor.
        side: optional ((context, torch stream), (context, torch stream)) for the K and V projections.
        The three projections read the same input and are independent; at small batches each of them
        fills only half of the GPU, so running them on three streams overlaps them."""
        import torch
        self.ctx, self.params, self.torch = ctx, params, torch
        self.fused_qkv = fused_qkv
        self.fused_gelu = fused_gelu
        self.own_attention = True  # head_dim 64: pimdl_attention; other head sizes use PyTorch's fused attention
        self.side = None if fused_qkv else side
        n = params.n
        self.amm = {}
        lin = dict(weights)
        if fused_qkv:  # one operator producing [q | k | v]: LUT columns and biases concatenated
            q, k, v = weights["q"], weights["k"], weights["v"]
            if not (np.array_equal(q["centroids"], k["centroids"]) and np.array_equal(q["centroids"], v["centroids"])
                    and q["scale"] == k["scale"] == v["scale"]):
                raise ValueError("fused QKV needs shared centroids and one LUT scale")
            lin["qkv"] = {"centroids": q["centroids"], "scale": q["scale"], "lut_bias": q.get("lut_bias", 0.0),
                          "lut": np.concatenate([q["lut"], k["lut"], v["lut"]], axis=2),
                          "bias": np.concatenate([q["bias"], k["bias"], v["bias"]])}
        names = (("qkv",) if fused_qkv else ("q", "k", "v")) + ("o", "ffn1", "ffn2")
        for name in names:
            w = lin[name]
            # bias_mode: pim_lut's epilogue adds lut_bias * num_codebook (pim_lut_host.cpp:201)
            owner = ctx
            if self.side and name in ("k", "v"):
                owner = self.side[0 if name == "k" else 1][0]
            self.amm[name] = owner.amm(w["centroids"], w["lut"], np.float32(w["scale"]), w["bias"], max_n=n,
                                       lut_bias=float(w.get("lut_bias", 0.0)), bias_mode=pimdl.BIAS_TIMES_CB,
                                       activation=pimdl.ACT_GELU_TANH if (fused_gelu and name == "ffn1")
                                       else pimdl.ACT_NONE)
        # the three projections search the same rows: one search launch for all of them where the library can
        self.qkv_group = None
        if not fused_qkv and not self.side:
            try:
                self.qkv_group = ctx.amm_group([self.amm[nm] for nm in ("q", "k", "v")])
            except pimdl.PimdlError:
                self.qkv_group = None  # shapes the shared search does not cover: three separate runs
        dev = torch.device("cuda", torch.cuda.current_device())
        self.norm = {name: (torch.from_numpy(np.ascontiguousarray(weights[name]["weight"], np.float32)).to(dev),
                            torch.from_numpy(np.ascontiguousarray(weights[name]["bias"], np.float32)).to(dev))
                     for name, _ in NORMS}

    def close(self):
        if self.qkv_group is not None:
            self.qkv_group.close()
            self.qkv_group = None
        for a in self.amm.values():
            a.close()
        self.amm = {}

    def _run(self, name, x, n):
        torch = self.torch
        y = torch.empty((n, self.amm[name].M), device=x.device, dtype=torch.float32)
        self.amm[name].run_ptr(x.data_ptr(), n, y.data_ptr())
        return y

    def _norm_residual(self, name, x, residual):
        torch = self.torch
        w, b = self.norm[name]
        y = torch.empty_like(x)
        self.ctx.layer_norm((x.data_ptr(), x.shape[0], x.shape[1]), w.data_ptr(), b.data_ptr(),
                            residual.data_ptr(), y.data_ptr(), 1e-6)
        return y

    def forward(self, x, keep=None):
        """x: float32 CUDA tensor [batch*seq][token_dim], row t = (batch t // seq_len, position t % seq_len).
        `keep`: optional dict that receives every intermediate (for stage-by-stage checks)."""
        torch, p = self.torch, self.params
        n = x.shape[0]
        if n % p.seq_len:
            raise ValueError("token count is not a multiple of seq_len")
        B, S, H, hd = n // p.seq_len, p.seq_len, p.head_num, p.head_dim
        x = x.contiguous()
        if self.fused_qkv:
            qkv = self._run("qkv", x, n)
            q, k, v = (qkv[:, i * p.token_dim:(i + 1) * p.token_dim] for i in range(3))
        elif self.qkv_group is not None and self.qkv_group.fused_cols == 3 * p.token_dim:
            # one search launch and one gather launch into [q | k | v]
            qkv = torch.empty((n, 3 * p.token_dim), device=x.device, dtype=torch.float32)
            self.qkv_group.run_fused_ptr(x.data_ptr(), n, qkv.data_ptr())
            q, k, v = (qkv[:, i * p.token_dim:(i + 1) * p.token_dim] for i in range(3))
        elif self.qkv_group is not None:
            q, k, v = (torch.empty((n, p.token_dim), device=x.device, dtype=torch.float32) for _ in range(3))
            self.qkv_group.run_ptr(x.data_ptr(), n, [q.data_ptr(), k.data_ptr(), v.data_ptr()])
        elif self.side:
            main = torch.cuda.current_stream()
            q, k, v = (torch.empty((n, p.token_dim), device=x.device, dtype=torch.float32) for _ in range(3))
            for (_, stream), name, dst in zip(self.side, ("k", "v"), (k, v)):
                stream.wait_stream(main)                                   # fork: x is ready
                self.amm[name].run_ptr(x.data_ptr(), n, dst.data_ptr())    # queued on that context's stream
            self.amm["q"].run_ptr(x.data_ptr(), n, q.data_ptr())
            for _, stream in self.side:
                main.wait_stream(stream)                                   # join
        else:
            q, k, v = self._run("q", x, n), self._run("k", x, n), self._run("v", x, n)
        att_scale = 1.0 / math.sqrt(p.token_dim / p.head_num)
        if hd == 64 and self.own_attention:
            # the library's attention kernel reads q, k, v where they are (also as column ranges of the fused
            # projection's output) and writes [n][token_dim] directly
            a = torch.empty((n, p.token_dim), device=x.device, dtype=torch.float32)
            self.ctx.attention_ptr(q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), B, S, H, hd,
                                   q.stride(0), p.token_dim, att_scale)
        else:
            qh, kh, vh = (t.reshape(B, S, H, hd).permute(0, 2, 1, 3) for t in (q, k, v))
            # unmasked softmax(q k^T / sqrt(head_dim)) v in fp32; PyTorch's fused kernel reads the strided head views
            attn = torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, scale=att_scale)     # [B][H][S][hd]
            a = attn.permute(0, 2, 1, 3).reshape(n, p.token_dim).contiguous()
        o = self._run("o", a, n)
        h = self._norm_residual("attention_norm", o, x)
        if self.fused_gelu:
            f1, g = None, self._run("ffn1", h, n)  # the pre-activation values never reach memory
        else:
            f1 = self._run("ffn1", h, n)
            g = torch.nn.functional.gelu(f1, approximate="tanh")
        f2 = self._run("ffn2", g, n)
        y = self._norm_residual("ffn_norm", f2, h)
        if keep is not None:
            keep.update(q=q, k=k, v=v, attn=a, o=o, h=h, ffn1=f1, gelu=g, ffn2=f2, out=y)
        return y


class Transformer:
    """layer_num encoder layers (transformer_model.cpp:13-49: each layer's output is the next one's input)."""

    def __init__(self, ctx, pimdl, layers, params, fused_qkv=False, parallel_qkv=False, fused_gelu=True):
        """Separate Q/K/V projections run as a group with one search launch (the default, where the shapes
        allow it) or, with parallel_qkv, on three streams; both measured within 1 % of each other."""
        import torch
        self.side = None
        if parallel_qkv and not fused_qkv:
            self.side = []
            for _ in range(2):
                c, st = pimdl.Context(torch.cuda.current_device()), torch.cuda.Stream()
                c.set_stream(st.cuda_stream)
                self.side.append((c, st))
        self.layers = [TransformerLayer(ctx, pimdl, w, params, fused_qkv, self.side, fused_gelu) for w in layers]
        self.params = params

    @classmethod
    def from_layers(cls, layers, params):
        """A model over TransformerLayer objects that already exist (they stay the caller's to close)."""
        self = cls.__new__(cls)
        self.side, self.layers, self.params = None, list(layers), params
        return self

    def close(self):
        for layer in self.layers:
            layer.close()
        for c, _ in self.side or []:
            c.close()
        self.side = None

    def forward(self, x):
        for layer in self.layers:
            x = layer.forward(x)
        return x

    def capture(self, x):
        """Records one forward pass on `x`'s shape into a HIP graph and returns (graph, static_input,
        static_output): copy new features into static_input, graph.replay(), read static_output.
        A layer is ~20 short kernels; launched one by one from Python the GPU waits for the host
        about a third of the time, replayed from a graph it does not.  The library's calls are
        recorded like any other launch (they run on the stream the context is bound to and, for
        device buffers that have been seen before, allocate and synchronise nothing)."""
        torch = self.layers[0].torch
        ctx = self.layers[0].ctx
        side = torch.cuda.Stream()
        static_x = x.clone()
        side.wait_stream(torch.cuda.current_stream())
        ctx.set_stream(side.cuda_stream)
        try:
            with torch.cuda.stream(side):
                for _ in range(2):  # first calls size the context's scratch and set kernel attributes
                    self.forward(static_x)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side, capture_error_mode="thread_local"):
                static_y = self.forward(static_x)
        finally:
            ctx.set_stream(torch.cuda.current_stream().cuda_stream)
        return graph, static_x, static_y


def synth_layers(params, ctx, pimdl, seed=0, shared_qkv_centroids=False):
    """Random-init weights of the right shapes (what the reference's driver falls back to without a
    weight file, test_transformer.cpp:483): centroids N(0,1), dense weights N(0, 0.02) turned into int8
    LUTs on the GPU (pimdl_lutgen), zero bias, unit LayerNorm weight."""
    rng = np.random.default_rng(seed)
    layers = []
    for _ in range(params.layer_num):
        layer = {}
        qkv_cent = None
        for name, _prefix in LINEARS:
            s = params.shapes[name]
            CB, C, v = s.num_codebook, s.num_centroid, s.sub_vec_len
            if shared_qkv_centroids and name in ("q", "k", "v"):
                if qkv_cent is None:
                    qkv_cent = rng.standard_normal((CB, C, v)).astype(np.float32)
                cent = qkv_cent
            else:
                cent = rng.standard_normal((CB, C, v)).astype(np.float32)
            W = (rng.standard_normal((s.input_feature_len, s.output_feature_len)) * 0.02).astype(np.float32)
            lut, scales = ctx.lutgen(cent, W, pimdl.LUT_I8, 0)
            layer[name] = {"centroids": cent, "lut": lut, "scale": float(scales[0]), "lut_bias": 0.0,
                           "bias": np.zeros(s.output_feature_len, np.float32)}
        for name, _prefix in NORMS:
            layer[name] = {"weight": np.ones(params.token_dim, np.float32), "bias": np.zeros(params.token_dim, np.float32)}
        layers.append(layer)
    return layers


def main(argv=None):
    """Counterpart of the reference's drivers (test_transformer.cpp, test_transformer_layer.cpp and the
    run_model.py / run_layer.py scripts that call them):
        python transformer.py config.yaml [weights.npz] [--iters K] [--graph] [--layer]
        python transformer.py --transformer_config_file config.yaml [--model_weight_file weights.npz] ...
    reads the same YAML and weight file, runs the forward on random token features and prints the
    per-iteration and average time in the reference's wording (test_transformer.cpp:356,381).
      --graph           record the forward once into a HIP graph and time its replays
      --layer           one layer only (run_layer.py); --need_breakdown adds the time of each stage of it
    The scripts' other flags are accepted and have nothing to do here: --need_compile (the kernels are in the
    library), --need_measure_energy, --breakdown_type."""
    import argparse
    ap = argparse.ArgumentParser(prog="transformer.py")
    ap.add_argument("config", nargs="?")
    ap.add_argument("weights", nargs="?")
    ap.add_argument("--transformer_config_file")          # run_model.py:8 / run_layer.py:8
    ap.add_argument("--model_weight_file", default=None)  # run_model.py:9
    ap.add_argument("--need_compile", action="store_true")
    ap.add_argument("--need_measure_energy", action="store_true")
    ap.add_argument("--need_breakdown", action="store_true")
    ap.add_argument("--breakdown_type", type=int, default=0)
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--graph", action="store_true")
    ap.add_argument("--layer", action="store_true")
    try:
        args = ap.parse_args(list(sys.argv[1:] if argv is None else argv))
    except SystemExit:
        return 2
    config = args.transformer_config_file or args.config
    weights = args.model_weight_file if args.model_weight_file not in (None, "null") else args.weights
    if not config:
        print("usage: transformer.py config_yaml_path [weight_path] [--iters K] [--graph] [--layer]", file=sys.stderr)
        return 2
    iters, use_graph = args.iters, args.graph
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.dirname(here))
    from __graft_entry__ import load_package
    pimdl = load_package()
    import torch
    params = TransformerParams.from_yaml(config)
    if args.layer:
        params.layer_num = 1
    print("finish parameter parsing")
    ctx = pimdl.Context(0)
    ctx.set_stream(torch.cuda.current_stream().cuda_stream)
    if weights and os.path.exists(weights):
        print("weight file is found, load weights from file.")
        layers = load_npz(weights, params)
    else:
        print("weight file is not found, generate weights randomly.")
        layers = synth_layers(params, ctx, pimdl)
    model = Transformer(ctx, pimdl, layers, params)
    print("finish weight initialization")
    x = torch.randn((params.n, params.token_dim), device="cuda", dtype=torch.float32)
    if use_graph:
        graph, static_x, _static_y = model.capture(x)
    print("inference start")
    total = 0.0
    for i in range(iters):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if use_graph:
            static_x.copy_(x)
            graph.replay()
        else:
            model.forward(x)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        total += dt
        print(f"iteration {i}, inference time {dt:.6f}")
    print("inference end")
    if iters:
        print(f"{iters} rounds' average inference time {total / iters:.6f}")
    if args.need_breakdown:
        # stage times of the first layer (device time between events, each stage launched on its own)
        layer, keep = model.layers[0], {}
        layer.forward(x, keep)
        n = x.shape[0]

        def timed(fn):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            fn()
            e0.record()
            for _ in range(10):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / 10 * 1e-3

        stages = []
        if "qkv" in layer.amm:
            stages.append(("qkv", lambda: layer._run("qkv", x, n)))
        else:
            stages += [(nm, (lambda nm=nm: layer._run(nm, x, n))) for nm in ("q", "k", "v")]
        stages += [("o", lambda: layer._run("o", keep["attn"], n)),
                   ("attention_norm", lambda: layer._norm_residual("attention_norm", keep["o"], x)),
                   ("ffn1", lambda: layer._run("ffn1", keep["h"], n)),
                   ("ffn2", lambda: layer._run("ffn2", keep["gelu"], n)),
                   ("ffn_norm", lambda: layer._norm_residual("ffn_norm", keep["ffn2"], keep["h"]))]
        print("layer 0 breakdown (seconds):")
        for name, fn in stages:
            print(f"  {name:16s} {timed(fn):.6f}")
    model.close()
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
