"""The layer/model wrapper on the GPU, checked stage by stage against the CPU oracle.

LUT-AMM is discontinuous (a centroid index can flip on a 1e-7 change of its input), so a whole layer is not
compared end to end against a CPU layer: each stage is compared against the oracle *given the GPU's own
input to that stage*.  Bars: every AMM bit-exact; layer normalisation within 1e-5 relative (the two
double-precision sums run in a different order than the reference's sequential loop); attention and GELU
(textbook fp32 definitions; the reference's ggml versions are pinned by none of its tests) within 1e-4."""
import math
import os

import numpy as np
import pytest

import oracle
from conftest import kernel_switches
from __graft_entry__ import load_package

pimdl = load_package()
from pim_dl_asplos_amd import transformer as T  # noqa: E402

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
CFG = os.path.join(HERE, "golden", "transformer_small.yaml")


@pytest.fixture(scope="module")
def ctx():
    import torch
    c = pimdl.Context(0)
    c.set_stream(torch.cuda.current_stream().cuda_stream)
    yield c
    c.close()


def amm_oracle(w, x):
    v = w["centroids"].shape[2]
    CB = w["centroids"].shape[0]
    idx = oracle.index_calculation(x, w["centroids"], v, threads=8)
    acc = oracle.gather_i8(idx, w["lut"], threads=8)
    return oracle.dequant(acc, w["bias"], CB, w["scale"], w.get("lut_bias", 0.0), 1, threads=8)


@pytest.mark.parametrize("n,d", [(1, 8), (37, 768), (256, 1024), (5, 100), (3, 4097), (9, 2048), (6, 1540)])
def test_layer_norm_matches_the_reference_statement(ctx, n, d):
    rng = np.random.default_rng(n * 1000 + d)
    x = (rng.standard_normal((n, d)) * 3 + 0.5).astype(np.float32)
    w = rng.standard_normal(d).astype(np.float32)
    b = rng.standard_normal(d).astype(np.float32)
    r = rng.standard_normal((n, d)).astype(np.float32)
    want = oracle.layer_norm(x, w, b)
    got = ctx.layer_norm(x, w, b)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    assert (got == want).mean() > 0.99  # in practice the sums round to the same floats
    got_r = ctx.layer_norm(x, w, b, residual=r)
    np.testing.assert_allclose(got_r, r + want, rtol=1e-5, atol=1e-6)
    # a constant row has zero variance: scale = 1/sqrt(eps), output = bias exactly
    c = np.full((2, d), 1.25, np.float32)
    assert np.array_equal(ctx.layer_norm(c, w, b), np.broadcast_to(b, (2, d)))


def gelu_tanh64(f):
    f = f.astype(np.float64)
    return 0.5 * f * (1 + np.tanh(math.sqrt(2 / math.pi) * (f + 0.044715 * f ** 3)))


@pytest.mark.parametrize("B,S,H,fused", [(2, 16, 3, False), (3, 128, 4, False), (2, 197, 2, True), (1, 300, 1, False),
                                          (2, 64, 2, True), (1, 1, 1, False)])
def test_attention_kernel_against_float64(ctx, B, S, H, fused):
    """pimdl_attention (head_dim 64, fp32 matrix cores, streaming softmax over 128-key chunks) against
    softmax(q k^T / 8) v in float64, and against PyTorch's fused attention; also reading q, k, v as three
    column ranges of one [n][3*token_dim] buffer."""
    import torch
    D, n = H * 64, B * S
    gen = torch.Generator(device="cuda").manual_seed(B * 1000 + S)
    if fused:
        qkv = torch.randn((n, 3 * D), device="cuda", generator=gen) * 2.0
        q, k, v = qkv[:, :D], qkv[:, D:2 * D], qkv[:, 2 * D:]
        in_stride = 3 * D
    else:
        q, k, v = (torch.randn((n, D), device="cuda", generator=gen) * 2.0 for _ in range(3))
        in_stride = D
    out = torch.full((n, D), float("nan"), device="cuda")
    ctx.attention_ptr(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, 64, in_stride, D, 0.125)
    torch.cuda.synchronize()
    q64, k64, v64 = (t.double().reshape(B, S, H, 64).permute(0, 2, 1, 3) for t in (q, k, v))
    p = torch.softmax(q64 @ k64.transpose(-1, -2) * 0.125, dim=-1)
    want = (p @ v64).permute(0, 2, 1, 3).reshape(n, D)
    assert not torch.isnan(out).any()
    torch.testing.assert_close(out.double(), want, rtol=1e-5, atol=1e-5)
    sd = torch.nn.functional.scaled_dot_product_attention(
        *(t.reshape(B, S, H, 64).permute(0, 2, 1, 3) for t in (q, k, v)), scale=0.125).permute(0, 2, 1, 3).reshape(n, D)
    torch.testing.assert_close(out, sd, rtol=1e-4, atol=1e-4)
    with pytest.raises(pimdl.PimdlError):  # other head sizes are not built
        ctx.attention_ptr(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, 32, in_stride, D, 0.125)


def test_qkv_modes_give_the_same_bits(ctx):
    """Q/K/V as a group (one search launch), on three streams, and one by one."""
    import torch
    p = T.TransformerParams(16, 3, 2, 64, 128, 256, 2)  # 32 codebooks per projection: a shared search exists
    for op, (cb, k_in, m_out) in {"q": (32, 128, 128), "k": (32, 128, 128), "v": (32, 128, 128), "o": (32, 128, 128),
                                  "ffn1": (32, 128, 256), "ffn2": (64, 256, 128)}.items():
        p.shapes[op] = T.AmmShape(cb, 16, k_in, m_out)
    layers = T.synth_layers(p, ctx, pimdl, seed=6)
    x = torch.randn((p.n, p.token_dim), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    outs = []
    for parallel in (False, True):
        m = T.Transformer(ctx, pimdl, layers, p, parallel_qkv=parallel)
        assert kernel_switches() or (m.layers[0].qkv_group is None) == parallel
        outs.append(m.forward(x).clone())
        torch.cuda.synchronize()
        m.close()
    one = T.TransformerLayer(ctx, pimdl, layers[0], p)
    if one.qkv_group is not None:
        one.qkv_group.close()
    one.qkv_group = None  # falls back to three runs
    grouped = T.TransformerLayer(ctx, pimdl, layers[0], p)
    assert torch.equal(one.forward(x), grouped.forward(x))
    # head_dim 64: the library's attention kernel inside the layer against PyTorch's on the same q, k, v
    keep_own, keep_torch = {}, {}
    grouped.forward(x, keep_own)
    grouped.own_attention = False
    grouped.forward(x, keep_torch)
    assert torch.equal(keep_own["q"], keep_torch["q"])
    torch.testing.assert_close(keep_own["attn"], keep_torch["attn"], rtol=1e-4, atol=1e-4)
    torch.cuda.synchronize()
    one.close()
    grouped.close()
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("fused_gelu", [True, False])
def test_layer_stage_by_stage(ctx, fused_gelu):
    import torch
    p = T.TransformerParams.from_yaml(CFG)
    layers = T.synth_layers(p, ctx, pimdl, seed=3)
    rng = np.random.default_rng(9)
    for name, _ in T.NORMS:  # non-trivial LayerNorm parameters and biases
        layers[0][name]["weight"] = rng.standard_normal(p.token_dim).astype(np.float32)
        layers[0][name]["bias"] = rng.standard_normal(p.token_dim).astype(np.float32)
    for name, _ in T.LINEARS:
        layers[0][name]["bias"] = rng.standard_normal(layers[0][name]["bias"].shape[0]).astype(np.float32)
    layer = T.TransformerLayer(ctx, pimdl, layers[0], p, fused_gelu=fused_gelu)
    x = rng.standard_normal((p.n, p.token_dim)).astype(np.float32)
    keep = {}
    y = layer.forward(torch.from_numpy(x).cuda(), keep)
    torch.cuda.synchronize()
    k = {name: t.cpu().numpy() for name, t in keep.items() if t is not None}
    w = layers[0]
    # the six AMMs, each from the GPU's own input: bit-exact
    for name, src in (("q", x), ("k", x), ("v", x), ("o", k["attn"]), ("ffn1", k["h"]), ("ffn2", k["gelu"])):
        want = amm_oracle(w[name], np.ascontiguousarray(src))
        if name == "ffn1" and fused_gelu:
            # the operator's epilogue applies GELU to exactly these values; only its rounding is left
            np.testing.assert_allclose(k["gelu"], gelu_tanh64(want), rtol=2e-6, atol=1e-7)
            continue
        assert np.array_equal(k[name].view(np.uint32), want.view(np.uint32)), name
    # attention: softmax(q k^T / sqrt(head_dim)) v per (batch, head), unmasked
    B, S, H, hd = p.batch_size, p.seq_len, p.head_num, p.head_dim
    q, kk, v = (k[n].astype(np.float64).reshape(B, S, H, hd).transpose(0, 2, 1, 3) for n in ("q", "k", "v"))
    s = q @ kk.transpose(0, 1, 3, 2) / math.sqrt(hd)
    s = np.exp(s - s.max(-1, keepdims=True))
    a = (s / s.sum(-1, keepdims=True)) @ v
    np.testing.assert_allclose(k["attn"], a.transpose(0, 2, 1, 3).reshape(p.n, p.token_dim), rtol=1e-4, atol=1e-4)
    # residual + LayerNorm, in the reference's placement: h = x + norm(o), y = h + norm(ffn2)
    np.testing.assert_allclose(k["h"], x + oracle.layer_norm(k["o"], w["attention_norm"]["weight"], w["attention_norm"]["bias"]),
                               rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(k["out"], k["h"] + oracle.layer_norm(k["ffn2"], w["ffn_norm"]["weight"], w["ffn_norm"]["bias"]),
                               rtol=1e-5, atol=1e-5)
    if not fused_gelu:  # tanh GELU as a pass of its own
        np.testing.assert_allclose(k["gelu"], gelu_tanh64(k["ffn1"]), rtol=1e-4, atol=1e-5)
    assert np.array_equal(y.cpu().numpy(), k["out"])
    layer.close()


def test_fused_qkv_equals_separate_projections(ctx):
    import torch
    p = T.TransformerParams.from_yaml(CFG)
    layers = T.synth_layers(p, ctx, pimdl, seed=4, shared_qkv_centroids=True)
    w = layers[0]
    scale = max(w[n]["scale"] for n in "qkv")
    for n in "qkv":
        w[n]["scale"] = scale  # one LUT scale for the fused operator
    x = torch.randn((p.n, p.token_dim), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    sep, fused = T.TransformerLayer(ctx, pimdl, w, p), T.TransformerLayer(ctx, pimdl, w, p, fused_qkv=True)
    ks, kf = {}, {}
    ys, yf = sep.forward(x, ks), fused.forward(x, kf)
    torch.cuda.synchronize()
    for n in ("q", "k", "v", "out"):
        assert torch.equal(ks[n], kf[n]), n
    assert torch.equal(ys, yf)
    sep.close()
    fused.close()


def test_model_is_the_chain_of_its_layers_and_reads_the_weight_file(ctx, tmp_path):
    import torch
    p = T.TransformerParams.from_yaml(CFG)
    layers = T.synth_layers(p, ctx, pimdl, seed=5)
    path = str(tmp_path / "model.npz")
    T.save_npz(path, layers)
    model = T.Transformer(ctx, pimdl, T.load_npz(path, p), p)
    x = torch.randn((p.n, p.token_dim), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    y = model.forward(x)
    z = x
    for w in layers:
        layer = T.TransformerLayer(ctx, pimdl, w, p)
        z = layer.forward(z)
        layer.close()
    torch.cuda.synchronize()
    assert torch.equal(y, z)
    assert torch.isfinite(y).all()
    model.close()


def _params_hd64():
    """head_dim 64 and 32 codebooks per projection: the Q/K/V group with one gather launch, pimdl_attention and
    the GELU epilogue are all on the path (the YAML configuration's head_dim 8 / 8 codebooks use none of them)."""
    p = T.TransformerParams(16, 3, 2, 64, 128, 384, 2)
    for op, (cb, k_in, m_out) in {"q": (32, 128, 128), "k": (32, 128, 128), "v": (32, 128, 128), "o": (32, 128, 128),
                                  "ffn1": (32, 128, 384), "ffn2": (96, 384, 128)}.items():
        p.shapes[op] = T.AmmShape(cb, 16, k_in, m_out)
    return p


@pytest.mark.parametrize("which", ["yaml", "hd64"])
def test_captured_forward_replays_like_the_eager_one(ctx, which):
    """The model forward recorded into a HIP graph: every replay, with eager work and synchronisations
    in between and with new input copied into the static buffer, equals the eager result bit for bit."""
    import torch
    p = T.TransformerParams.from_yaml(CFG) if which == "yaml" else _params_hd64()
    model = T.Transformer(ctx, pimdl, T.synth_layers(p, ctx, pimdl, seed=9), p)
    if which == "hd64":
        assert kernel_switches() or model.layers[0].qkv_group is not None
    gen = torch.Generator(device="cuda").manual_seed(4)
    xs = [torch.randn((p.n, p.token_dim), device="cuda", generator=gen) for _ in range(3)]
    want = [model.forward(x).clone() for x in xs]
    torch.cuda.synchronize()
    graph, static_x, static_y = model.capture(xs[0])
    for rep in range(2):
        for x, w in zip(xs, want):
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, w)
            assert torch.equal(model.forward(xs[1]), want[1])  # eager work between replays, same context
            torch.cuda.synchronize()
    del graph
    model.close()


def test_graph_survives_growth_of_the_context_scratch():
    """A recorded graph holds the addresses of the context's scratch buffers.  Later eager calls that need more
    scratch (a larger operator, a larger batch, host buffers, the debug outputs) must leave those addresses
    valid: the replay after them still equals the eager result."""
    import torch
    c = pimdl.Context(0)
    c.set_stream(torch.cuda.current_stream().cuda_stream)
    p = _params_hd64()
    model = T.Transformer(c, pimdl, T.synth_layers(p, c, pimdl, seed=10), p)
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((p.n, p.token_dim), device="cuda", generator=gen)
    want = model.forward(x).clone()
    graph, static_x, static_y = model.capture(x)
    # everything that makes the scratch grow: 4096 tokens x 768 codebooks against 48 tokens x 96 before
    rng = np.random.default_rng(3)
    N, K, v, C, M = 4096, 3072, 4, 16, 256
    cent = rng.standard_normal((K // v, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (K // v, C, M)).astype(np.int8)
    big = c.amm(cent, lut, np.float32(0.01), None, max_n=N)
    xb = rng.standard_normal((N, K)).astype(np.float32)
    out_host, idx, acc = big.run_debug(xb)                      # host staging, index and accumulator scratch
    xd = torch.from_numpy(xb).cuda()
    od = torch.empty((N, M), device="cuda")
    big.run_ptr(xd.data_ptr(), N, od.data_ptr())                # device buffers
    torch.cuda.synchronize()
    assert np.array_equal(od.cpu().numpy().view(np.uint32), out_host.view(np.uint32))
    for _ in range(2):
        static_x.copy_(x)
        static_y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, want)
    # during a capture the scratch cannot grow: the call is refused, not served from a fresh allocation
    huge = c.amm(cent, lut, np.float32(0.01), None, max_n=N)
    ot = torch.empty((N, M), device="cuda")
    g2 = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    c.set_stream(side.cuda_stream)
    refused = None
    try:
        with torch.cuda.graph(g2, stream=side, capture_error_mode="thread_local"):
            try:  # a tiled run needs a row-major staging buffer that no call has sized yet
                huge.run_tiled_ptr(xd.data_ptr(), N, ot.data_ptr(), n_stile=1024, f_stile=128)
            except pimdl.PimdlError as e:
                refused = e
    finally:
        c.set_stream(torch.cuda.current_stream().cuda_stream)
    assert refused is not None and refused.code == pimdl.ERR_INVALID and "captured" in str(refused)
    # outside the capture the same call is served, and equals the row-major result re-ordered
    huge.run_tiled_ptr(xd.data_ptr(), N, ot.data_ptr(), n_stile=1024, f_stile=128)
    torch.cuda.synchronize()
    tiled = ot.cpu().numpy().reshape(-1)
    for n_, f_ in zip(rng.integers(0, N, 200), rng.integers(0, M, 200)):
        assert tiled[oracle.output_offset(int(n_), int(f_), 1024, 128, 128, M // 128)] == out_host[n_, f_]
    del graph, g2
    big.close()
    huge.close()
    model.close()
    c.close()


def test_driver_prints_the_reference_wording(capsys):
    assert T.main([CFG, "--iters", "2"]) == 0
    out = capsys.readouterr().out
    assert "weight file is not found, generate weights randomly." in out
    assert "iteration 1, inference time" in out and "inference end" in out
    assert T.main([CFG, "--iters", "2", "--graph"]) == 0  # the same through a recorded HIP graph
    assert "iteration 1, inference time" in capsys.readouterr().out
    # the flag names of the reference's run_model.py / run_layer.py
    assert T.main(["--transformer_config_file", CFG, "--model_weight_file", "null", "--need_compile", "--layer",
                   "--need_breakdown", "--iters", "3"]) == 0
    out = capsys.readouterr().out
    assert "3 rounds' average inference time" in out and "ffn_norm" in out
    assert T.main([]) == 2


def test_column_tile_hint_and_measured_tile_search(ctx, tmp_path):
    """Every column-tile width gives the same bits; an unavailable width is rejected; the tuner picks one
    of the widths it measured and caches it."""
    if kernel_switches():
        pytest.skip("the environment keeps one kernel for every shape; this test walks the library's choices")
    from pim_dl_asplos_amd import autotune as AT
    rng = np.random.default_rng(2)
    N, K, v, C, M = 300, 64, 4, 16, 200
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((K // v, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (K // v, C, M)).astype(np.int8)
    outs = []
    for cb in (0, 48, 64, 96):
        amm = ctx.amm(cent, lut, np.float32(0.02), None, max_n=N, col_block=cb)
        assert cb == 0 or amm.geometry()["col_block"] == cb
        outs.append(amm.run(x))
        amm.close()
    for o in outs[1:]:
        assert np.array_equal(o.view(np.uint32), outs[0].view(np.uint32))
    with pytest.raises(pimdl.PimdlError) as e:
        ctx.amm(cent, lut, np.float32(0.02), None, max_n=N, col_block=80)
    assert e.value.code == pimdl.ERR_INVALID
    best, results = AT.tune(ctx, pimdl, 512, 128, 4, 16, 384, iters=3, full=False)
    assert best["gather_ms"] > 0 and best["gather_ms"] <= best["library_gather_ms"] and best["search"] == {}
    assert {"gather:col_block=48", "gather:col_block=64", "gather:col_block=96"} <= set(results)
    cache = AT.TileCache(str(tmp_path / "tiles.json"))
    key = AT.shape_key("dev", 512, 128, 4, 16, 384, "int8")
    cache.put(key, best)
    assert AT.TileCache(str(tmp_path / "tiles.json")).get(key) == best["gather"]
    AT.write_yaml(str(tmp_path / "t.yaml"), 512, 128, 4, 16, 384, best)
    import yaml
    doc = yaml.safe_load(open(str(tmp_path / "t.yaml")))
    assert doc["amm_shape_params"]["num_codebook"] == 32 and doc["kernel_params"]["gather_ms"] > 0


def test_every_tuning_choice_gives_the_same_bits(ctx):
    """The whole space the measured search walks (accumulation kernel, column block, token item, codebook
    slice, XCD dealing, search kernel and its token tile): bit-identical outputs, checked against the oracle
    once; choices a shape has no kernel for are refused with PIMDL_ERR_INVALID."""
    if kernel_switches():
        pytest.skip("the environment keeps one kernel for every shape; this test walks the library's choices")
    import itertools
    rng = np.random.default_rng(3)
    N, K, v, C, M = 700, 256, 4, 16, 384      # CB = 64: 32-codebook slices exist; 8 | column tiles of 48
    CB = K // v
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    bias = rng.standard_normal(M).astype(np.float32)
    want, _, _ = oracle.amm_cpu(x, cent, lut, bias, v, 0.02, 0.0, threads=8)
    seen = 0
    for gk, cb in itertools.product((pimdl.GATHER_ROWS, pimdl.GATHER_ONEHOT, pimdl.GATHER_SPARSE), (48, 64, 96)):
        try:
            amm = ctx.amm(cent, lut, np.float32(0.02), bias, max_n=N, tuning={"gather_kernel": gk, "col_block": cb})
        except pimdl.PimdlError as e:
            assert e.code == pimdl.ERR_INVALID and gk == pimdl.GATHER_ROWS and cb == 96
            continue
        assert amm.tuning()["gather_kernel"] == gk and amm.tuning()["col_block"] == cb
        settings = [{}]
        if gk != pimdl.GATHER_ROWS:
            settings += [{"token_item": t} for t in (128, 256)] + [{"xcd_col_split": s} for s in (1, 2, 4, 8, pimdl.XCD_PLAIN)]
            settings += [{"cb_per_slice": 16}, {"token_item": 128, "cb_per_slice": 16, "xcd_col_split": 2}]
            if cb <= 64:
                settings.append({"cb_per_slice": 32})
            if gk == pimdl.GATHER_SPARSE:  # one workgroup of eight waves per CU: 512-token items
                settings += [{"token_item": 512}, {"token_item": 512, "cb_per_slice": 32, "xcd_col_split": 4}]
                settings.append({"token_item": 512, "cb_per_slice": 64} if cb == 48 else {"token_item": 512, "cb_per_slice": 16})
        settings += [{"search_kernel": k} for k in (1, 2, 3)] + [{"search_kernel": 3, "search_token_tile": t} for t in (64, 128)]
        for st in settings:
            amm.set_tuning(**st)
            got = amm.run(x)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (gk, cb, st)
            seen += 1
        if gk != pimdl.GATHER_ROWS and cb == 96:
            with pytest.raises(pimdl.PimdlError):
                amm.set_tuning(cb_per_slice=32)
            with pytest.raises(pimdl.PimdlError):
                amm.set_tuning(token_item=512, cb_per_slice=64)
        if gk == pimdl.GATHER_ONEHOT:
            with pytest.raises(pimdl.PimdlError):
                amm.set_tuning(token_item=512)
        with pytest.raises(pimdl.PimdlError):
            amm.set_tuning(col_block=48 if cb != 48 else 64)
        with pytest.raises(pimdl.PimdlError):
            amm.set_tuning(token_item=100)
        amm.close()
    assert seen > 100
    # 17..32 centroids: the sparse kernel (every codebook as two of 16) or the byte adder; no dense one-hot
    # kernel, no fp32 matrix-core search, no eight-wave workgroups
    lut32 = rng.integers(-128, 128, (CB, 32, M)).astype(np.int8)
    cent32 = rng.standard_normal((CB, 32, v)).astype(np.float32)
    want32, _, _ = oracle.amm_cpu(x, cent32, lut32, bias, v, 0.02, 0.0, threads=8)
    for bad in ({"gather_kernel": pimdl.GATHER_ONEHOT}, {"search_kernel": 2}, {"token_item": 512},
                {"gather_kernel": pimdl.GATHER_ROWS, "token_item": 128}):
        with pytest.raises(pimdl.PimdlError) as e:
            ctx.amm(cent32, lut32, np.float32(0.02), None, max_n=N, tuning=bad)
        assert e.value.code == pimdl.ERR_INVALID
    for gk, cb in ((pimdl.GATHER_ROWS, 48), (pimdl.GATHER_ROWS, 64), (pimdl.GATHER_SPARSE, 48), (pimdl.GATHER_SPARSE, 64),
                   (pimdl.GATHER_SPARSE, 96)):
        amm = ctx.amm(cent32, lut32, np.float32(0.02), bias, max_n=N, tuning={"gather_kernel": gk, "col_block": cb})
        settings = [{}]
        if gk == pimdl.GATHER_SPARSE:
            settings += [{"token_item": 128}, {"token_item": 256}, {"cb_per_slice": 16}, {"xcd_col_split": 2}]
            if cb <= 64:
                settings.append({"cb_per_slice": 32, "token_item": 128})
        for st in settings:
            amm.set_tuning(**st)
            assert np.array_equal(amm.run(x).view(np.uint32), want32.view(np.uint32)), (gk, cb, st)
        assert amm.last_gather_kernel().startswith("gather_sparse" if gk == pimdl.GATHER_SPARSE else "gather_i8")
        amm.close()
    # up to 8 centroids: the paired dense kernel (48 or 64 columns), the sparse kernel (the table as 16 centroids
    # with empty rows; also 96 columns) or the byte adder; small launches take the paired kernel by themselves
    for C8 in (8, 5, 1):
        lut8 = rng.integers(-128, 128, (CB, C8, M)).astype(np.int8)
        cent8 = rng.standard_normal((CB, C8, v)).astype(np.float32)
        want8, _, _ = oracle.amm_cpu(x, cent8, lut8, bias, v, 0.02, 0.0, threads=8)
        for tn in ({}, {"gather_kernel": pimdl.GATHER_ONEHOT, "col_block": 48}, {"gather_kernel": pimdl.GATHER_ONEHOT, "col_block": 64},
                   {"gather_kernel": pimdl.GATHER_SPARSE}, {"gather_kernel": pimdl.GATHER_SPARSE, "col_block": 48},
                   {"gather_kernel": pimdl.GATHER_SPARSE, "col_block": 64, "token_item": 128},
                   {"gather_kernel": pimdl.GATHER_SPARSE, "col_block": 96}, {"col_block": 96},
                   {"gather_kernel": pimdl.GATHER_SPARSE, "col_block": 48, "token_item": 512, "cb_per_slice": 64},
                   {"gather_kernel": pimdl.GATHER_ROWS}):
            amm = ctx.amm(cent8, lut8, np.float32(0.02), bias, max_n=N, tuning=tn)
            assert np.array_equal(amm.run(x).view(np.uint32), want8.view(np.uint32)), (C8, tn)
            kind = tn.get("gather_kernel", pimdl.GATHER_SPARSE if tn.get("col_block") == 96 else pimdl.GATHER_ONEHOT)
            assert amm.last_gather_kernel().startswith({pimdl.GATHER_ONEHOT: "gather_onehot", pimdl.GATHER_SPARSE: "gather_sparse",
                                                        pimdl.GATHER_ROWS: "gather_i8"}[kind]), (C8, tn)
            amm.close()
        with pytest.raises(pimdl.PimdlError) as e:
            ctx.amm(cent8, lut8, np.float32(0.02), None, max_n=N, tuning={"gather_kernel": pimdl.GATHER_ONEHOT, "col_block": 96})
        assert e.value.code == pimdl.ERR_INVALID
    with pytest.raises(pimdl.PimdlError):   # 33 centroids and more: the byte adder only
        ctx.amm(rng.standard_normal((CB, 40, v)).astype(np.float32), rng.integers(-128, 128, (CB, 40, M)).astype(np.int8),
                np.float32(0.02), None, max_n=N, tuning={"gather_kernel": pimdl.GATHER_SPARSE})


def test_full_measured_search_runs(ctx):
    if kernel_switches():
        pytest.skip("the environment keeps one kernel for every shape; this test walks the library's choices")
    from pim_dl_asplos_amd import autotune as AT
    best, results = AT.tune(ctx, pimdl, 1024, 256, 4, 16, 384, iters=2, full=True)
    assert any(k.startswith("search:") for k in results) and sum(k.startswith("gather:") for k in results) > 20
    assert best["gather_ms"] <= best["library_gather_ms"] and best["ccs_ms"] <= best["library_ccs_ms"]
