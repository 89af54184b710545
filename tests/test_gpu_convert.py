"""LUT construction on the GPU (pimdl_lutgen) and the weight converter built on it, against the oracle's
restatement of model-calibration/pim_weight_converter.py:21-35,86-91.

Bar: the fp32 table within 1e-5 relative of the oracle's (the MFMA accumulates the v products of an entry
in a different order than a sequential CPU sum); the int8 table within one quantisation step with at least
99.9 % of the entries identical, its scale within 1e-6 relative."""
import numpy as np
import pytest

import oracle
from __graft_entry__ import load_package

pimdl = load_package()
from pim_dl_asplos_amd import convert as CV  # noqa: E402
from pim_dl_asplos_amd import transformer as T  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = pimdl.Context(0)
    yield c
    c.close()


@pytest.mark.parametrize("CB,C,v,M", [(192, 16, 4, 3072), (384, 16, 2, 768), (96, 32, 8, 200), (7, 5, 3, 33), (1, 1, 1, 4)])
def test_lutgen_matches_the_converter_formula(ctx, CB, C, v, M):
    rng = np.random.default_rng(CB + C + v + M)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    W = (rng.standard_normal((CB * v, M)) * 0.02).astype(np.float32)
    want_f = oracle.lutgen_f32(cent, W, threads=8)
    got_f, _ = ctx.lutgen(cent, W, pimdl.LUT_F32, 0)
    np.testing.assert_allclose(got_f, want_f, rtol=1e-5, atol=1e-7)
    want_q, want_s = oracle.lut_quant(want_f)
    got_q, got_s = ctx.lutgen(cent, W, pimdl.LUT_I8, 0)
    np.testing.assert_allclose(got_s[0], want_s[0], rtol=1e-6)
    diff = np.abs(got_q.astype(np.int32) - want_q.astype(np.int32))
    assert diff.max() <= 1 and (diff == 0).mean() >= 0.999
    assert np.abs(got_q.astype(np.int32)).max() <= 127 or (got_q == -128).any()
    # the largest entry in magnitude quantises to +-127 exactly (scale = max|lut| / 127)
    assert np.abs(got_q.astype(np.int32)).max() == 127


@pytest.mark.parametrize("CB,C,v,M", [(192, 16, 4, 3072), (384, 16, 2, 768), (96, 32, 8, 200), (7, 5, 3, 33), (1, 1, 1, 4),
                                      (12, 16, 32, 100)])
def test_ordered_lutgen_is_bit_identical_to_the_scalar_loop(ctx, CB, C, v, M):
    """PIMDL_LUTGEN_ORDERED: fp32 table, int8 table and scale(s) equal the oracle's bit for bit."""
    rng = np.random.default_rng(CB * 7 + C + v + M)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    W = (rng.standard_normal((CB * v, M)) * 0.02).astype(np.float32)
    W[0, :2] = [0.0, -0.0]
    want_f = oracle.lutgen_f32(cent, W, threads=8)
    got_f, _ = ctx.lutgen(cent, W, pimdl.LUT_F32, 0, ordered=True)
    assert np.array_equal(got_f.view(np.uint32), want_f.view(np.uint32))
    for group in (0, 1, 5):
        want_q, want_s = oracle.lut_quant(want_f, group)
        got_q, got_s = ctx.lutgen(cent, W, pimdl.LUT_I8, group, ordered=True)
        assert np.array_equal(got_s.view(np.uint32), np.asarray(want_s, np.float32).view(np.uint32))
        assert np.array_equal(got_q, want_q)


def test_converter_writes_the_engine_format_and_the_model_runs_from_it(ctx, tmp_path):
    """A synthetic 'calibrated checkpoint' in the reference's input naming (safetensors, HF BERT encoder keys)
    goes through the converter; the result loads into the model wrapper and runs."""
    import torch
    from safetensors.numpy import save_file
    features, C, v, L = 32, 16, 2, 2
    rng = np.random.default_rng(11)
    src = {"bert.embeddings.word_embeddings.weight": rng.standard_normal((10, features)).astype(np.float32)}
    ops = ("attention.self.query", "attention.self.key", "attention.self.value", "attention.output.dense",
           "intermediate.dense", "output.dense")
    for li in range(L):
        for op in ops:
            in_f, out_f = CV.linear_shape(op, features)
            pre = f"bert.encoder.layer.{li}.{op}"
            src[pre + ".weight"] = (rng.standard_normal((in_f, out_f)) * 0.05).astype(np.float32)
            src[pre + ".centroids.weight"] = rng.standard_normal((in_f // v, C * v)).astype(np.float32)
            src[pre + ".bias"] = rng.standard_normal(out_f).astype(np.float32)
        for ln in ("attention.output.LayerNorm", "output.LayerNorm"):
            src[f"bert.encoder.layer.{li}.{ln}.weight"] = rng.standard_normal(features).astype(np.float32)
            src[f"bert.encoder.layer.{li}.{ln}.bias"] = rng.standard_normal(features).astype(np.float32)
    inp, outp = str(tmp_path / "calibrated.safetensors"), str(tmp_path / "engine.npz")
    save_file(src, inp)
    assert CV.main(["--weight_input_file", inp, "--weight_output_file", outp, "--features", str(features),
                    "--ncentroids", str(C), "--vec_len", str(v)]) == 0
    z = np.load(outp, allow_pickle=False)
    assert not any("embeddings" in k for k in z.files)
    assert "0.attention.self.query.weight" not in z.files           # replaced by the LUT
    assert z["1.output.dense.lut.tensor"].dtype == np.int8 and z["1.output.dense.lut.tensor"].shape == (64 * C, features)
    assert z["0.intermediate.dense.lut.scale"].shape == () and float(z["0.intermediate.dense.lut.bias"]) == 0.0
    assert np.array_equal(z["0.output.LayerNorm.weight"], src["bert.encoder.layer.0.output.LayerNorm.weight"])
    # the LUT is the oracle's, entry for entry up to one quantisation step
    cent = src["bert.encoder.layer.1.output.dense.centroids.weight"].reshape(64, C, v)
    want_q, want_s = oracle.lut_quant(oracle.lutgen_f32(cent, src["bert.encoder.layer.1.output.dense.weight"]))
    got_q = z["1.output.dense.lut.tensor"].reshape(64, C, features)
    assert np.abs(got_q.astype(np.int32) - want_q.astype(np.int32)).max() <= 1
    np.testing.assert_allclose(float(z["1.output.dense.lut.scale"]), want_s[0], rtol=1e-6)
    # and the engine-side wrapper consumes the file
    p = T.TransformerParams(seq_len=8, batch_size=2, head_num=4, head_dim=8, token_dim=features,
                            ffn_hidden_dim=4 * features, layer_num=L)
    for name, (k_in, m_out) in {"q": (32, 32), "k": (32, 32), "v": (32, 32), "o": (32, 32), "ffn1": (32, 128),
                                "ffn2": (128, 32)}.items():
        p.shapes[name] = T.AmmShape(k_in // v, C, k_in, m_out)
    c2 = pimdl.Context(0)
    c2.set_stream(torch.cuda.current_stream().cuda_stream)
    model = T.Transformer(c2, pimdl, T.load_npz(outp, p), p)
    y = model.forward(torch.randn((p.n, features), device="cuda"))
    torch.cuda.synchronize()
    assert y.shape == (p.n, features) and torch.isfinite(y).all()
    model.close()
    c2.close()


def test_fp32_lut_export(ctx):
    rng = np.random.default_rng(3)
    t = {"encoder.layer.0.intermediate.dense.weight": (rng.standard_normal((16, 64)) * 0.1).astype(np.float32),
         "encoder.layer.0.intermediate.dense.centroids.weight": rng.standard_normal((4, 8 * 4)).astype(np.float32),
         "encoder.layer.0.intermediate.dense.bias": np.zeros(64, np.float32)}
    out = CV.convert(t, ctx, pimdl, features=16, ncentroids=8, vec_len=4, lut_dtype="fp32")
    lut = out["0.intermediate.dense.lut.tensor"]
    assert lut.dtype == np.float32 and lut.shape == (32, 64) and float(out["0.intermediate.dense.lut.scale"]) == 1.0
    want = oracle.lutgen_f32(t["encoder.layer.0.intermediate.dense.centroids.weight"].reshape(4, 8, 4),
                             t["encoder.layer.0.intermediate.dense.weight"])
    np.testing.assert_allclose(lut.reshape(4, 8, 64), want, rtol=1e-5, atol=1e-7)
