"""Host logic of the layer/model wrapper that needs no GPU: the reference's YAML keys and weight-file
format (inference-engine/src/host/parser.cpp:86-330, test/test_transformer.cpp:246-463,
model-calibration/pim_weight_converter.py:93-96)."""
import os

import numpy as np
import pytest

from __graft_entry__ import load_package

load_package()
from pim_dl_asplos_amd import transformer as T  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
CFG = os.path.join(HERE, "golden", "transformer_small.yaml")


def fake_layers(params, seed=0):
    rng = np.random.default_rng(seed)
    layers = []
    for _ in range(params.layer_num):
        layer = {}
        for name, _ in T.LINEARS:
            s = params.shapes[name]
            layer[name] = {"centroids": rng.standard_normal((s.num_codebook, s.num_centroid, s.sub_vec_len)).astype(np.float32),
                           "lut": rng.integers(-128, 128, (s.num_codebook, s.num_centroid, s.output_feature_len)).astype(np.int8),
                           "scale": float(rng.uniform(0.01, 0.1)), "lut_bias": 0.0,
                           "bias": rng.standard_normal(s.output_feature_len).astype(np.float32)}
        for name, _ in T.NORMS:
            layer[name] = {"weight": rng.standard_normal(params.token_dim).astype(np.float32),
                           "bias": rng.standard_normal(params.token_dim).astype(np.float32)}
        layers.append(layer)
    return layers


def test_yaml_keys_of_the_reference():
    p = T.TransformerParams.from_yaml(CFG)
    assert (p.seq_len, p.batch_size, p.head_num, p.head_dim, p.token_dim, p.ffn_hidden_dim, p.layer_num) == \
        (16, 3, 4, 8, 32, 96, 2)
    assert p.n == 48
    assert p.shapes["qkv"].output_feature_len == 96 and p.shapes["qkv"].sub_vec_len == 4
    assert p.shapes["q"].output_feature_len == 32 and p.shapes["q"].num_codebook == 8
    assert p.shapes["o"].sub_vec_len == 2
    assert (p.shapes["ffn1"].num_centroid, p.shapes["ffn1"].sub_vec_len) == (8, 4)
    assert (p.shapes["ffn2"].input_feature_len, p.shapes["ffn2"].sub_vec_len) == (96, 4)


def test_weight_file_round_trip_and_key_names(tmp_path):
    p = T.TransformerParams.from_yaml(CFG)
    layers = fake_layers(p)
    path = str(tmp_path / "w.npz")
    T.save_npz(path, layers)
    z = np.load(path, allow_pickle=False)
    # the names and dtypes pim_weight_converter.py writes and test_transformer.cpp reads
    for key, dtype, shape in (("0.attention.self.query.centroids.weight", np.float32, (8, 64)),
                              ("0.attention.self.query.lut.tensor", np.int8, (128, 32)),
                              ("0.attention.self.query.lut.scale", np.float32, ()),
                              ("0.attention.self.query.lut.bias", np.float32, ()),
                              ("0.attention.self.value.bias", np.float32, (32,)),
                              ("1.attention.output.dense.lut.tensor", np.int8, (256, 32)),
                              ("1.intermediate.dense.centroids.weight", np.float32, (8, 32)),
                              ("1.output.dense.lut.tensor", np.int8, (384, 32)),
                              ("0.attention.output.LayerNorm.weight", np.float32, (32,)),
                              ("1.output.LayerNorm.bias", np.float32, (32,))):
        assert z[key].dtype == dtype and z[key].shape == shape, key
    assert len(z.files) == 2 * (6 * 5 + 2 * 2)
    back = T.load_npz(path, p)
    for a, b in zip(layers, back):
        for name, _ in T.LINEARS:
            assert np.array_equal(a[name]["centroids"], b[name]["centroids"])
            assert np.array_equal(a[name]["lut"], b[name]["lut"])
            assert np.float32(a[name]["scale"]) == np.float32(b[name]["scale"])
            assert np.array_equal(a[name]["bias"], b[name]["bias"])
        for name, _ in T.NORMS:
            assert np.array_equal(a[name]["weight"], b[name]["weight"])


def test_weight_file_that_does_not_match_the_configuration_is_rejected(tmp_path):
    p = T.TransformerParams.from_yaml(CFG)
    layers = fake_layers(p)
    layers[1]["o"]["centroids"] = layers[1]["o"]["centroids"][:-1]
    layers[1]["o"]["lut"] = layers[1]["o"]["lut"][:-1]
    path = str(tmp_path / "bad.npz")
    T.save_npz(path, layers)
    with pytest.raises(ValueError):
        T.load_npz(path, p)


def test_converter_key_handling_and_shapes():
    """split_layers / linear_shape follow pim_weight_converter.py:42-55,74-81."""
    from pim_dl_asplos_amd import convert as CV
    t = {"bert.embeddings.word_embeddings.weight": np.zeros(3),
         "bert.encoder.layer.0.attention.self.query.weight": np.zeros(1),
         "bert.encoder.layer.11.output.dense.centroids.weight": np.zeros(2),
         "bert.pooler.dense.weight": np.zeros(4),
         "layer.3.intermediate.dense.bias": np.zeros(5)}
    layers = CV.split_layers(t)
    assert sorted(layers) == [0, 3, 11]
    assert list(layers[0]) == ["0.attention.self.query.weight"]
    assert list(layers[11]) == ["11.output.dense.centroids.weight"]
    assert list(layers[3]) == ["3.intermediate.dense.bias"]
    assert CV.linear_shape("0.attention.self.query", 768) == (768, 768)
    assert CV.linear_shape("0.attention.output.dense", 768) == (768, 768)
    assert CV.linear_shape("0.intermediate.dense", 768) == (768, 3072)
    assert CV.linear_shape("0.output.dense", 768) == (3072, 768)
    with pytest.raises(ValueError):
        CV.convert({}, None, None, nsharecodebook=2)


def test_shipped_bert_base_configuration_parses():
    p = T.TransformerParams.from_yaml(os.path.join(HERE, "..", "pim-dl-asplos_amd", "configs", "bert_base_b32_s128.yaml"))
    assert p.n == 4096 and p.layer_num == 12
    assert p.shapes["ffn2"].num_codebook == 768 and p.shapes["q"].sub_vec_len == 4
