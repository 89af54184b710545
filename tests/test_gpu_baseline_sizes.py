"""Parity at the full sizes of the benchmark configurations.  Rows of a LUT-AMM are independent, so
the GPU runs the whole batch and the oracle checks a random sample of its rows: indices and int32
accumulators bit for bit, fp32 outputs bit for bit (int8 LUT) or to 1e-5 relative (fp32 LUT)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402

pytestmark = pytest.mark.gpu
THREADS = min(16, os.cpu_count() or 1)


@pytest.fixture(scope="module")
def env():
    from __graft_entry__ import load_package
    pimdl = load_package()
    ctx = pimdl.Context(0)
    yield pimdl, ctx
    ctx.close()


def run_and_check_sample(ctx, seed, N, K, v, C, M, lut_kind, sample=192):
    rng = np.random.default_rng(seed)
    CB = K // v
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    bias = rng.standard_normal(M).astype(np.float32)
    rows = np.sort(rng.choice(N, size=min(sample, N), replace=False))
    rows[0], rows[-1] = 0, N - 1  # both ends of the batch, always
    if lut_kind == "i8":
        lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
        amm = ctx.amm(cent, lut, np.float32(0.0123), bias, max_n=N)
        out, idx, acc = amm.run_debug(x)
        w_out, w_idx, w_acc = oracle.amm_cpu(x[rows], cent, lut, bias, v, 0.0123, 0.0, threads=THREADS)
        assert np.array_equal(idx[rows], w_idx)
        assert np.array_equal(acc[rows], w_acc)
        assert np.array_equal(out[rows].view(np.uint32), w_out.view(np.uint32))
    else:
        lut = rng.standard_normal((CB, C, M)).astype(np.float32)
        amm = ctx.amm(cent, lut, None, bias, max_n=N)
        out, idx, _ = amm.run_debug(x)
        w_idx = oracle.index_calculation(x[rows], cent, v, threads=THREADS)
        assert np.array_equal(idx[rows], w_idx)
        want = oracle.gather_f32(w_idx, lut, bias, threads=THREADS)
        np.testing.assert_allclose(out[rows], want, rtol=1e-5, atol=1e-5 * np.sqrt(CB))  # the stated fp32 tolerance
    assert np.isfinite(out).all()
    amm.close()


@pytest.mark.parametrize("K,M", [(768, 3072), (3072, 768)])
def test_bert_base_ffn_pair_full_batch(env, K, M):
    """The benchmark configuration: BERT-base FFN pair, N = 8192, v = 4, C = 16, int8 LUT."""
    run_and_check_sample(env[1], 11, 8192, K, 4, 16, M, "i8")


@pytest.mark.parametrize("K,M", [(1024, 3072), (1024, 1024), (1024, 4096), (4096, 1024)])
def test_bert_large_linears_full_batch(env, K, M):
    """BERT-large: hidden 1024, FFN 4096, N = 8192 (fused QKV, O, FFN1, FFN2), v = 4, C = 16."""
    run_and_check_sample(env[1], 12, 8192, K, 4, 16, M, "i8", sample=128)


@pytest.mark.parametrize("lut_kind", ["i8", "f32"])
@pytest.mark.parametrize("v,C", [(2, 8), (2, 16), (2, 32), (4, 8), (4, 16), (4, 32), (8, 8), (8, 16), (8, 32)])
def test_vit_base_sweep_full_batch(env, v, C, lut_kind):
    """ViT-Base: N = 64 x 197 = 12608, FFN1 of ViT-Base (768 -> 3072), v x C sweep, both LUT types."""
    run_and_check_sample(env[1], 13 + v + C, 12608, 768, v, C, 3072, lut_kind, sample=96)


@pytest.mark.parametrize("v,C", [(2, 16), (4, 16), (8, 32)])
def test_vit_base_ffn2_full_batch(env, v, C):
    run_and_check_sample(env[1], 29 + v, 12608, 3072, v, C, 768, "i8", sample=96)


def test_reference_single_amm_search_space_shape(env):
    """The shape of the reference's 89 single-AMM tuning configs: N = 32768, 1024 -> 4096, 256 codebooks of
    16 centroids (512 MB of fp32 output, 128 token tiles x 64 column tiles)."""
    run_and_check_sample(env[1], 41, 32768, 1024, 4, 16, 4096, "i8", sample=64)
