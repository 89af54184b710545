"""Parity of the HIP path (through the C ABI) against the CPU oracle, on the same seeded inputs.

Bar: bit-exact centroid indices, bit-exact int32 accumulators, bit-exact fp32 output for the int8
path (the epilogue is three separately rounded fp32 operations on both sides); fp32-LUT path within
1e-5 relative (in fact also bit-exact, since both sides add in ascending codebook order)."""
import os

import numpy as np
import pytest

import oracle
from conftest import kernel_switches
from __graft_entry__ import load_package

pimdl = load_package()
pytestmark = pytest.mark.gpu

THREADS = 8


@pytest.fixture(scope="module")
def ctx():
    c = pimdl.Context(0)
    yield c
    c.close()


def make_case(seed, N, K, v, C, M, lut="i8", dist="normal"):
    rng = np.random.default_rng(seed)
    CB = K // v
    if dist == "normal":
        x = rng.standard_normal((N, K)).astype(np.float32)
        cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    else:  # the reference driver's ranges (test_amm.cpp:26-45)
        x = rng.uniform(-5, 5, (N, K)).astype(np.float32)
        cent = rng.uniform(-10, 10, (CB, C, v)).astype(np.float32)
    bias = rng.standard_normal(M).astype(np.float32)
    if lut == "i8":
        table = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    else:
        table = rng.standard_normal((CB, C, M)).astype(np.float32)
    return x, cent, table, bias


def check_i8(ctx, seed, N, K, v, C, M, scale=0.0123, lut_bias=0.0, bias_mode=0, dist="normal", max_n=None):
    x, cent, lut, bias = make_case(seed, N, K, v, C, M, "i8", dist)
    CB = K // v
    amm = ctx.amm(cent, lut, np.float32(scale), bias, max_n=max_n or N, lut_bias=lut_bias, bias_mode=bias_mode)
    out, idx, acc = amm.run_debug(x)
    want_idx = oracle.index_calculation(x, cent, v, threads=THREADS)
    want_acc = oracle.gather_i8(want_idx, lut, threads=THREADS)
    want_out = oracle.dequant(want_acc, bias, CB, scale, lut_bias, bias_mode, threads=THREADS)
    assert np.array_equal(idx, want_idx), f"indices: {(idx != want_idx).sum()} of {idx.size} differ"
    assert np.array_equal(acc, want_acc), f"accumulators: {(acc != want_acc).sum()} of {acc.size} differ"
    assert np.array_equal(out.view(np.uint32), want_out.view(np.uint32)), "fp32 output bits differ"
    # the plain entry point gives the same bytes as the debug one
    assert np.array_equal(amm.run(x).view(np.uint32), out.view(np.uint32))
    amm.close()


def test_config1_single_amm(ctx):
    """N=128, K=768, v=2 (384 codebooks), 16 centroids, M=768, LUT = quantised centroid x W."""
    rng = np.random.default_rng(0)
    N, K, v, C, M = 128, 768, 2, 16, 768
    CB = K // v
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    W = (rng.standard_normal((K, M)) * 0.02).astype(np.float32)
    lut, scales = oracle.lut_quant(oracle.lutgen_f32(cent, W, threads=THREADS))
    bias = np.zeros(M, np.float32)
    want_out, want_idx, want_acc = oracle.amm_cpu(x, cent, lut, bias, v, float(scales[0]), 0.0, threads=THREADS)
    amm = ctx.amm(cent, lut, scales, bias, max_n=N)
    out, idx, acc = amm.run_debug(x)
    assert np.array_equal(idx, want_idx)
    assert np.array_equal(acc, want_acc)
    assert np.array_equal(out.view(np.uint32), want_out.view(np.uint32))
    amm.close()


@pytest.mark.parametrize("v,C", [(2, 8), (2, 16), (2, 32), (4, 8), (4, 16), (4, 32), (8, 8), (8, 16), (8, 32),
                                 (16, 16), (32, 16), (4, 64), (4, 128), (2, 256)])
def test_sweep_sub_vector_length_and_centroids(ctx, v, C):
    check_i8(ctx, 100 + v * 7 + C, N=300, K=64 * v if v < 16 else 96 * v // 2, v=v, C=C, M=200)


@pytest.mark.parametrize("N,K,v,C,M", [
    (1, 8, 4, 16, 4),        # smallest sensible shape
    (17, 24, 4, 16, 20),     # CB=6 (padded to 32), M not a multiple of the column block
    (255, 36, 4, 16, 63),    # M % 4 != 0: scalar stores
    (257, 40, 4, 5, 130),    # C not a power of two
    (513, 12, 3, 7, 33),     # sub_vec_len with no specialised kernel
    (64, 10, 5, 20, 18),     # generic v, 8-bit indices, K % 4 != 0
    (100, 6, 2, 16, 64),     # CB=3 (odd), K % 4 != 0: scalar activation loads
    (300, 44, 4, 20, 40),    # 17..32 centroids on the matrix-core search: ids past C never win
    (129, 18, 2, 17, 24),    # same, v=2, CB=9
    (200, 72, 8, 31, 50),    # same, v=8
    (333, 70, 10, 16, 52),   # sub_vec_len 10 (the reference's token_dim 2560 over 256 codebooks): CB=7, K % 4 != 0
    (130, 170, 10, 12, 37),  # ... CB=17 (two codebook tiles, the second ragged), C not a power of two
    (65, 640, 10, 40, 24),   # ... 8-bit indices, several centroid groups per codebook
    (257, 60, 20, 16, 20),   # sub_vec_len 20 (token_dim 5120): CB=3
    (100, 500, 20, 130, 16), # ... CB=25, more than 128 centroids
])
def test_ragged_shapes(ctx, N, K, v, C, M):
    check_i8(ctx, N + K + M, N, K, v, C, M)


@pytest.mark.parametrize("N,M", [
    (512, 768),     # 8 column tiles x 4 token tiles: one column tile per XCD
    (1000, 380),    # 4 column tiles x 8 token tiles (last one ragged): columns over 4, tokens over 2
    (2048, 192),    # 2 column tiles x 16 token tiles: columns over 2, tokens over 4
    (4096, 96),     # 1 column tile x 32 token tiles: tokens over 8
    (768, 768),     # 6 token tiles: no split divides, plain order
])
def test_every_item_is_computed_once_however_items_are_dealt_to_the_xcds(ctx, N, M):
    """The one-hot gather deals (column tile, token tile) items to the 8 XCDs by a split chosen per shape;
    a dropped or doubled item shows as wrong accumulators."""
    if os.environ.get("PIMDL_GATHER_ROWS") == "1":
        pytest.skip("the matrix-core gather is switched off")
    x, cent, lut, bias = make_case(N + M, N, 128, 4, 16, M)
    amm = ctx.amm(cent, lut, np.float32(0.01), bias, max_n=N, col_block=96)
    out, idx, acc = amm.run_debug(x)
    want_idx = oracle.index_calculation(x, cent, 4, threads=THREADS)
    want_acc = oracle.gather_i8(want_idx, lut, threads=THREADS)
    assert np.array_equal(idx, want_idx)
    assert np.array_equal(acc, want_acc)
    assert np.array_equal(out.view(np.uint32),
                          oracle.dequant(want_acc, bias, 32, 0.01, 0.0, 0, threads=THREADS).view(np.uint32))
    amm.close()


@pytest.mark.parametrize("C,lut,group", [(16, "i8", 0), (32, "i8", 0), (16, "f32", 0), (16, "i8", 4)])
def test_gelu_in_the_epilogue(ctx, C, lut, group):
    """activation=ACT_GELU_TANH: same indices and accumulators, output = tanh-GELU of the plain output
    (each of the gather kernels: matrix-core one-hot, byte adder, fp32 table, grouped scales)."""
    N, K, v, M = 300, 128, 4, 200
    x, cent, table, bias = make_case(C + group, N, K, v, C, M, lut)
    CB = K // v
    scales = None if lut == "f32" else (np.full((CB + group - 1) // group, 0.02, np.float32) if group else np.float32(0.02))
    plain = ctx.amm(cent, table, scales, bias, max_n=N, scale_group=group)
    fused = ctx.amm(cent, table, scales, bias, max_n=N, scale_group=group, activation=pimdl.ACT_GELU_TANH)
    y = plain.run(x).astype(np.float64)
    want = 0.5 * y * (1 + np.tanh(np.sqrt(2 / np.pi) * (y + 0.044715 * y ** 3)))
    got = fused.run(x)
    assert (np.abs(y) > 3).any() and (np.abs(y) < 0.1).any()  # both tails and the middle are exercised
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)
    if lut == "i8" and not group:
        _, idx, acc = fused.run_debug(x)
        _, idx0, acc0 = plain.run_debug(x)
        assert np.array_equal(idx, idx0) and np.array_equal(acc, acc0)
    # extreme inputs: -0 for very negative values (never NaN), identity for very positive ones
    big = ctx.amm(cent, table, scales, np.where(np.arange(M) % 2 == 0, 1e6, -1e6).astype(np.float32), max_n=N,
                  scale_group=group, activation=pimdl.ACT_GELU_TANH)
    raw = ctx.amm(cent, table, scales, np.where(np.arange(M) % 2 == 0, 1e6, -1e6).astype(np.float32), max_n=N,
                  scale_group=group)
    yb, y0 = big.run(x), raw.run(x)
    assert np.array_equal(yb[:, 0::2], y0[:, 0::2]) and not yb[:, 1::2].any() and not np.isnan(yb).any()
    for a in (plain, fused, big, raw):
        a.close()
    with pytest.raises(pimdl.PimdlError):
        ctx.amm(cent, table, scales, bias, max_n=N, scale_group=group, activation=7)


def test_reference_driver_value_ranges_and_bias_modes(ctx):
    # uniform(-5,5) activations, uniform(-10,10) centroids, scale 0.1, bias 0.2 as in the shipped YAML
    check_i8(ctx, 7, 256, 128, 4, 16, 96, scale=0.1, lut_bias=0.2, bias_mode=0, dist="uniform")
    check_i8(ctx, 8, 256, 128, 4, 16, 96, scale=0.1, lut_bias=0.2, bias_mode=1, dist="uniform")


def test_golden_reference_vectors_on_gpu(ctx, golden_index):
    """The fixtures produced by the reference's own compiled index_calculation."""
    for i in range(int(golden_index["ncases"])):
        x, cent, want = golden_index[f"c{i}_x"], golden_index[f"c{i}_cent"], golden_index[f"c{i}_idx"]
        CB, C, v = cent.shape
        lut = np.zeros((CB, C, 4), np.int8)
        amm = ctx.amm(cent, lut, np.float32(1.0), None, max_n=x.shape[0])
        got = amm.index_calculation(x)
        assert np.array_equal(got, want), f"golden case {i} ({golden_index[f'c{i}_kind']})"
        for key in golden_index.files:
            if key.startswith(f"c{i}_tiled_"):
                _, _, ns, cm = key.split("_")
                assert np.array_equal(amm.index_calculation(x, int(ns), int(cm)), golden_index[key]), key
        amm.close()


def test_near_ties_follow_the_scan_not_the_true_argmin(ctx):
    """Inputs midway between two centroids: many distance pairs differ by ~1e-6."""
    rng = np.random.default_rng(5)
    N, CB, C, v = 2048, 32, 16, 4
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    a = rng.integers(0, C, (N, CB))
    b = (a + 1 + rng.integers(0, C - 1, (N, CB))) % C
    cb = np.arange(CB)[None, :]
    mid = (cent[cb, a] + cent[cb, b]) * np.float32(0.5)
    x = (mid + rng.standard_normal((N, CB, v)).astype(np.float32) * np.float32(2e-7)).reshape(N, CB * v)
    want = oracle.index_calculation(x, cent, v, threads=THREADS)
    true_argmin = oracle.np_distances(x, cent).argmin(-1)
    assert (want != true_argmin).sum() > 100  # the case really separates the two rules
    amm = ctx.amm(cent, np.zeros((CB, C, 4), np.int8), np.float32(1.0), None, max_n=N)
    assert np.array_equal(amm.index_calculation(x), want)
    amm.close()


@pytest.mark.parametrize("C", [16, 8, 5, 32, 20, 64])
def test_gather_from_given_indices_and_invariants(ctx, C):
    """C <= 8 runs the paired form of the matrix-core gather (two codebooks per index byte, odd CB), 17..32 the
    sparse form with every codebook as two of 16 (byte indices), more than 32 the byte adder."""
    rng = np.random.default_rng(21)
    N, CB, M, v = 300, 41 if C < 16 else 40, 192, 4
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    idx = rng.integers(0, C, (N, CB)).astype(np.uint16)
    amm = ctx.amm(cent, lut, np.float32(1.0), None, max_n=N)
    out = amm.lut_gather(idx)
    want = oracle.gather_i8(idx, lut, threads=THREADS)
    assert np.array_equal(out, want.astype(np.float32))
    amm.close()
    # extremes: every entry -128 / +127, CB = 768 (the largest of the BERT shapes)
    CB = 768
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    idx = rng.integers(0, C, (64, CB)).astype(np.uint16)
    for val in (-128, 127):
        amm = ctx.amm(cent, np.full((CB, C, 64), val, np.int8), np.float32(1.0), None, max_n=64)
        assert (amm.lut_gather(idx) == float(val * CB)).all()
        amm.close()


@pytest.mark.parametrize("C,v", [(16, 4), (8, 2), (32, 8)])
def test_fp32_lut_path(ctx, C, v):
    N, K, M = 300, 48 * v, 100
    x, cent, lut, bias = make_case(31 + C, N, K, v, C, M, "f32")
    amm = ctx.amm(cent, lut, None, bias, max_n=N)
    out, idx, _ = amm.run_debug(x)
    want_idx = oracle.index_calculation(x, cent, v, threads=THREADS)
    assert np.array_equal(idx, want_idx)
    want = oracle.gather_f32(want_idx, lut, bias, threads=THREADS)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-6)  # the stated tolerance for fp32 paths
    amm.close()


@pytest.mark.parametrize("group,C,v,CB,M", [(1, 16, 4, 48, 100), (3, 16, 4, 48, 100), (5, 16, 2, 48, 64),
                                            (16, 16, 4, 192, 96), (64, 8, 8, 48, 33), (7, 32, 4, 40, 100),
                                            (4, 64, 4, 20, 72), (2, 256, 2, 6, 40)])
def test_scale_per_codebook_group(ctx, group, C, v, CB, M):
    """int8 LUT with one scale per `group` codebooks (an extension the reference does not have, so the
    only pin is the oracle's definition: int32 inside a group, then fp32 `tot += (float)acc_g * scale[g]`
    over groups ascending, then + bias).  Bit-exact against it, including ragged last groups, a group
    larger than CB, 4- and 8-bit index rows; group 1 is one scale per codebook."""
    N, K = 300, CB * v
    x, cent, lut, bias = make_case(500 + group + C, N, K, v, C, M)
    ng = (CB + group - 1) // group
    scales = np.random.default_rng(group).uniform(1e-3, 0.1, ng).astype(np.float32)
    amm = ctx.amm(cent, lut, scales, bias, max_n=N, scale_group=group)
    out = amm.run(x)
    want_idx = oracle.index_calculation(x, cent, v, threads=THREADS)
    want = oracle.gather_i8_grouped(want_idx, lut, scales, bias, group, threads=THREADS)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32)), \
        f"{(out.view(np.uint32) != want.view(np.uint32)).sum()} of {out.size} outputs differ"
    amm.close()


@pytest.mark.parametrize("kind", ["f32", "grouped"])
def test_two_tokens_per_lane_in_the_fp32_table_gather(ctx, kind):
    """Wide outputs make the fp32-table gather give each lane two tokens (rows t and t + 256 of a 512-token
    block); the last block is ragged in both halves' sense: 1100 = 2 * 512 + 76."""
    N, v, CB, C, M = 1100, 4, 8, 16, 2752
    x, cent, lut, bias = make_case(77, N, CB * v, v, C, M, "f32" if kind == "f32" else "i8")
    want_idx = oracle.index_calculation(x, cent, v, threads=THREADS)
    if kind == "f32":
        amm = ctx.amm(cent, lut, None, bias, max_n=N)
        np.testing.assert_allclose(amm.run(x), oracle.gather_f32(want_idx, lut, bias, threads=THREADS), rtol=1e-5, atol=1e-6)
    else:
        scales = np.random.default_rng(3).uniform(1e-3, 0.1, 3).astype(np.float32)
        amm = ctx.amm(cent, lut, scales, bias, max_n=N, scale_group=3)
        want = oracle.gather_i8_grouped(want_idx, lut, scales, bias, 3, threads=THREADS)
        assert np.array_equal(amm.run(x).view(np.uint32), want.view(np.uint32))
    amm.close()


@pytest.mark.parametrize("N,K,v,C,Ms,lut", [
    (300, 256, 4, 16, (96, 200, 64), "i8"),     # tiled index rows (matrix-core gather), three outputs of different widths
    (1000, 128, 4, 8, (128, 128), "i8"),        # paired gather
    (1300, 128, 4, 8, (192, 192, 192), "i8"),   # paired gather, three members in one gather launch
    (700, 256, 4, 16, (96, 96), "i8"),          # one gather launch, 96-column tiles
    (2100, 128, 4, 16, (768, 768, 768), "i8"),  # the Q/K/V shape
    (257, 256, 2, 32, (100, 60), "i8"),         # 32 centroids: byte indices, tiled index rows (sparse gather, two tables)
    (900, 256, 4, 32, (96, 96, 96), "i8"),      # 32 centroids, three members in one gather launch
    (300, 256, 8, 16, (48, 80, 48), "f32"),     # fp32 tables
    (8192, 768, 4, 8, (768, 3072), "i8"),       # 8 centroids at a size where the wide member takes the sparse kernel, the narrow one the paired
    (8192, 256, 8, 8, (1536, 1536), "i8"),      # 8 centroids, both members on the sparse kernel, one gather launch
])
def test_operators_sharing_an_input_are_searched_by_one_launch(ctx, N, K, v, C, Ms, lut):
    """AmmGroup (separate Q/K/V projections): every output bit for bit that of the operator run alone."""
    if kernel_switches():
        pytest.skip("a kernel this test is about is switched off by the environment")
    rng = np.random.default_rng(N + K)
    x = rng.standard_normal((N, K)).astype(np.float32)
    amms = []
    for i, M in enumerate(Ms):
        _, cent, table, bias = make_case(900 + i, 1, K, v, C, M, lut)
        amms.append(ctx.amm(cent, table, None if lut == "f32" else np.float32(0.01 * (i + 1)), bias, max_n=N))
    group = ctx.amm_group(amms)
    outs = group.run(x)
    for a, o in zip(amms, outs):
        assert np.array_equal(o.view(np.uint32), a.run(x).view(np.uint32))
    if C == 8 and N == 8192:  # which kernel each member's launch rule took
        want_kernels = {(768, 3072): ("gather_onehot", "gather_sparse"), (1536, 1536): ("gather_sparse", "gather_sparse")}[Ms]
        for a, k in zip(amms, want_kernels):
            assert a.last_gather_kernel().startswith(k), (a.last_gather_kernel(), k)
    outs2 = group.run(x[:77])  # a smaller batch through the same group
    for o, o2 in zip(outs, outs2):
        assert np.array_equal(o[:77], o2)
    # one gather launch for all members where they are matrix-core gathers of one shape
    same_shape = lut == "i8" and C <= 32 and len(set(Ms)) == 1 and Ms[0] % amms[0].geometry()["col_block"] == 0
    assert (group.fused_cols > 0) == same_shape
    if same_shape:
        fused = group.run_fused(x)
        assert np.array_equal(fused.view(np.uint32), np.concatenate(outs, axis=1).view(np.uint32))
    else:
        with pytest.raises(pimdl.PimdlError):
            group.run_fused(x)
    group.close()
    for a in amms:
        a.close()


def test_group_conditions(ctx):
    if kernel_switches():
        pytest.skip("a kernel this test is about is switched off by the environment")
    rng = np.random.default_rng(5)
    mk = lambda K, v, C, M, kind="i8": ctx.amm(*(lambda c: (c[1], c[2]))(make_case(1, 1, K, v, C, M, kind)),
                                               None if kind == "f32" else np.float32(0.01), None, max_n=64)
    a, b = mk(128, 4, 16, 32), mk(128, 4, 16, 48)
    for bad in (mk(256, 4, 16, 32), mk(128, 2, 16, 32), mk(128, 4, 8, 32), mk(128, 4, 16, 32, "f32")):
        with pytest.raises(pimdl.PimdlError):
            ctx.amm_group([a, bad])
        bad.close()
    with pytest.raises(pimdl.PimdlError):
        ctx.amm_group([a])                       # fewer than two operators
    c40a, c40b = mk(160, 4, 16, 32), mk(160, 4, 16, 32)  # 40 codebooks: not a multiple of 32
    with pytest.raises(pimdl.PimdlError):
        ctx.amm_group([c40a, c40b])
    g = ctx.amm_group([a, b])
    with pytest.raises(pimdl.PimdlError):
        g.run(rng.standard_normal((65, 128)).astype(np.float32))  # beyond max_n
    g.close()
    for m in (a, b, c40a, c40b):
        m.close()


def test_scale_groups_from_lutgen(ctx):
    """lutgen with per-group quantisation -> operator with the same grouping: closer to the fp32 product
    than the per-tensor quantisation of the same table, and equal to the oracle on the generated table."""
    rng = np.random.default_rng(77)
    CB, C, v, M, N = 64, 16, 4, 128, 256
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    cent[::4] *= 8.0                                     # codebooks of very different magnitude
    W = (rng.standard_normal((CB * v, M)) * 0.02).astype(np.float32)
    x = rng.standard_normal((N, CB * v)).astype(np.float32)
    lut_f, _ = ctx.lutgen(cent, W, lut_dtype=pimdl.LUT_F32)
    lut_t, s_t = ctx.lutgen(cent, W)
    lut_g, s_g = ctx.lutgen(cent, W, scale_group=1)
    assert s_g.shape == (CB,)
    idx = oracle.index_calculation(x, cent, v, threads=THREADS)
    exact = oracle.gather_f32(idx, lut_f, np.zeros(M, np.float32), threads=THREADS)
    a_t = ctx.amm(cent, lut_t, s_t, None, max_n=N)
    a_g = ctx.amm(cent, lut_g, s_g, None, max_n=N, scale_group=1)
    out_t, out_g = a_t.run(x), a_g.run(x)
    want_g = oracle.gather_i8_grouped(idx, lut_g, s_g, np.zeros(M, np.float32), 1, threads=THREADS)
    assert np.array_equal(out_g.view(np.uint32), want_g.view(np.uint32))
    err_t, err_g = np.abs(out_t - exact).mean(), np.abs(out_g - exact).mean()
    assert err_g < 0.7 * err_t, (err_g, err_t)
    a_t.close()
    a_g.close()


def test_device_pointers_and_partial_batches(ctx):
    """Inputs already resident in HBM (torch tensors), n smaller than max_n, output rows past n untouched."""
    import torch

    N, K, v, C, M = 700, 256, 4, 16, 320
    x, cent, lut, bias = make_case(41, N, K, v, C, M)
    amm = ctx.amm(cent, lut, np.float32(0.05), bias, max_n=1024)
    want = oracle.amm_cpu(x, cent, lut, bias, v, 0.05, 0.0, threads=THREADS)[0]
    xd = torch.from_numpy(x).cuda()
    od = torch.full((1024, M), -7.0, device="cuda")
    torch.cuda.synchronize()
    amm.run_ptr(xd.data_ptr(), N, od.data_ptr())
    ctx.synchronize()
    got = od.cpu().numpy()
    assert np.array_equal(got[:N].view(np.uint32), want.view(np.uint32))
    assert (got[N:] == -7.0).all()
    # a second, smaller batch through the same operator
    amm.run_ptr(xd.data_ptr(), 33, od.data_ptr())
    ctx.synchronize()
    assert np.array_equal(od.cpu().numpy()[:33].view(np.uint32), want[:33].view(np.uint32))
    amm.close()


def test_error_paths(ctx):
    cent = np.zeros((4, 16, 4), np.float32)
    lut = np.zeros((4, 16, 8), np.int8)
    with pytest.raises(pimdl.PimdlError) as e:
        ctx.amm(cent, lut, None, None)           # int8 LUT without scales
    assert e.value.code == -1
    with pytest.raises(pimdl.PimdlError) as e:           # grouped scales have no zero point
        ctx.amm(cent, lut, np.ones(2, np.float32), None, scale_group=3, lut_bias=0.5)
    assert e.value.code == -1
    amm = ctx.amm(cent, lut, np.ones(2, np.float32), None, scale_group=3, max_n=8)
    with pytest.raises(pimdl.PimdlError) as e:           # no single int32 accumulator to return
        amm.run_debug(np.zeros((4, 16), np.float32))
    assert e.value.code == -1
    amm.close()
    amm = ctx.amm(cent, lut, np.float32(1), None, max_n=8)
    with pytest.raises(pimdl.PimdlError) as e:
        amm.run(np.zeros((9, 16), np.float32))   # n > max_n
    assert e.value.code == -1
    assert amm.run(np.zeros((0, 16), np.float32)).shape == (0, 8)  # empty batch is a no-op
    amm.close()


# ---- the two-speed search: fast scores + margin test, exact replay on near ties -----------------

@pytest.mark.parametrize("v,C", [(2, 16), (4, 16), (8, 16), (4, 7), (16, 16), (4, 32), (2, 64)])
def test_search_with_exact_ties_and_degenerate_inputs(ctx, v, C):
    """Duplicate centroids (margin 0), all-zero rows, inputs equal to a centroid, tiny and huge
    magnitudes: every pair must come out as the reference's scan says, whichever path took it."""
    rng = np.random.default_rng(1000 + 10 * v + C)
    N, CB = 389, 37
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    cent[::3, C // 2] = cent[::3, 0]                   # exact duplicates: first index must win
    cent[1::5] *= np.float32(1e-3)                     # a codebook of tiny centroids
    cent[2::7] *= np.float32(1e4)                      # and one of huge ones
    x = rng.standard_normal((N, CB, v)).astype(np.float32)
    x[::4] = 0.0
    pick = rng.integers(0, C, (N, CB))
    on = rng.random((N, CB)) < 0.3
    x[on] = cent[np.nonzero(on)[1], pick[on]]          # exactly on a centroid
    x[5::11] *= np.float32(1e5)
    x = x.reshape(N, CB * v)
    want = oracle.index_calculation(x, cent, v, threads=THREADS)
    amm = ctx.amm(cent, np.zeros((CB, C, 4), np.int8), np.float32(1.0), None, max_n=N)
    got = amm.index_calculation(x)
    assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} differ"
    amm.close()


@pytest.mark.parametrize("v,C", [(8, 16), (4, 16), (8, 32), (4, 32), (4, 20), (8, 12), (4, 5), (8, 8), (2, 16)])
def test_search_with_a_few_near_ties_per_wave(ctx, v, C):
    """One (token, codebook) pair in about 400 sits midway between two centroids, the others are ordinary: a wave
    then has one or two lanes to replay exactly, which it does lane by lane with all its lanes (many at once take
    another path, covered by the dense cases above).  Both token tiles of the search, a ragged batch, a codebook
    count that leaves the last codebook tile partly empty; every index against the reference's scan."""
    rng = np.random.default_rng(3000 + 10 * v + C)
    N, CB = 1500, 37
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    x = rng.standard_normal((N, CB, v)).astype(np.float32)
    on = rng.random((N, CB)) < 1.0 / 400
    a = rng.integers(0, C, (N, CB))
    b = (a + 1 + rng.integers(0, C - 1, (N, CB))) % C
    cbi = np.nonzero(on)[1]
    mid = (cent[cbi, a[on]] + cent[cbi, b[on]]) * np.float32(0.5)
    x[on] = mid + rng.standard_normal(mid.shape).astype(np.float32) * np.float32(2e-7)
    x = x.reshape(N, CB * v)
    want = oracle.index_calculation(x, cent, v, threads=THREADS)
    assert (want != oracle.np_distances(x, cent).argmin(-1)).sum() > 0  # some pairs separate the scan from the true argmin
    amm = ctx.amm(cent, np.zeros((CB, C, 4), np.int8), np.float32(1.0), None, max_n=N)
    for tile in (0, 64, 128):
        amm.set_tuning(search_token_tile=tile)
        got = amm.index_calculation(x)
        assert np.array_equal(got, want), f"tile {tile}: {(got != want).sum()} of {got.size} differ"
    amm.close()


@pytest.mark.parametrize("v,C", [(4, 16), (2, 16), (8, 16), (4, 32)])
def test_search_with_non_finite_values(ctx, v, C):
    """NaN / Inf / near-overflow values in activations and centroids take the exact path and match
    the reference's compare semantics (a NaN distance never replaces the running best)."""
    rng = np.random.default_rng(2000 + 10 * v + C)
    N, CB = 300, 40
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    cent[3, 2, 0] = np.nan
    cent[5, 0, 1] = np.nan          # NaN in centroid 0: the scan keeps index 0
    cent[7, 4, 0] = np.inf
    cent[9, 1, :] = 3e19            # |c|^2 overflows fp32
    cent[11, 6, 0] = -np.inf
    x = rng.standard_normal((N, CB * v)).astype(np.float32)
    x[1, :] = np.nan
    x[2, 5] = np.inf
    x[3, 7] = -np.inf
    x[4, :] = 2e19
    x[6, 3] = 3e38
    with np.errstate(all="ignore"):
        want = oracle.index_calculation(x, cent, v, threads=THREADS)
    amm = ctx.amm(cent, np.zeros((CB, C, 4), np.int8), np.float32(1.0), None, max_n=N)
    got = amm.index_calculation(x)
    assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} differ"
    amm.close()


def test_matrix_core_rounding_stays_inside_the_search_margin(ctx):
    """The bf16-split search accepts a winner only outside an error margin that assumes every addition of
    the matrix core's chain (48 products + the initial accumulator) is within 2^-24 of the partial sum:
    51 units of 2^-24 * sum|terms| for v = 4.  Measured on this device over 10^6 outputs with operand pieces
    of mixed magnitude, the chain stays an order of magnitude inside that."""
    worst = ctx.diag_mfma_error(1024)
    assert 0.0 < worst < 12.0, worst


def test_matrix_core_rounding_on_crafted_worst_cases(ctx):
    """Random operands are not the worst case for an accumulator.  The crafted chains add 48 equal products just
    below / above 1/2, 1 and 2 units in the last place of an accumulator of 1.0 (either sign), and products
    falling by a factor of four per slot: a sequential round-to-nearest adder loses 24 units on them, a
    truncating one up to 96.  The search margin allows 51; the device must stay below half of that."""
    worst = ctx.diag_mfma_error_crafted()
    print("crafted mfma error (units of 2^-24 * sum|terms|):", worst)
    assert 0.0 <= worst < 25.5, worst


def test_search_at_full_ffn2_shape(ctx):
    """N=8192, K=3072, v=4, 16 centroids: every index of the headline shape against the oracle,
    once with N(0,1) data and once with the reference driver's ranges."""
    for dist in ("normal", "ref"):
        x, cent, _, _ = make_case(77, 8192, 3072, 4, 16, 4, "i8", dist)
        want = oracle.index_calculation(x, cent, 4, threads=THREADS)
        amm = ctx.amm(cent, np.zeros((768, 16, 4), np.int8), np.float32(1.0), None, max_n=8192)
        got = amm.index_calculation(x)
        assert np.array_equal(got, want), f"{dist}: {(got != want).sum()} of {got.size} differ"
        amm.close()


def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        v = int(rng.choice([2, 4, 8, 2, 4, 8, 3, 16]))
        C = int(rng.choice([rng.integers(2, 9), rng.integers(9, 17), rng.integers(17, 33), 16, 16, 32, 8, 64]))
        CB = int(rng.choice([rng.integers(1, 12), rng.integers(12, 80), 32, 64, 96]))
        M = int(rng.choice([rng.integers(1, 64), rng.integers(64, 420), 96, 192, 768]))
        N = int(rng.choice([rng.integers(1, 70), rng.integers(70, 700), rng.integers(700, 2600), 256, 1024]))
        kind = str(rng.choice(["i8", "i8", "i8", "f32", "grouped"]))
        cases.append((i, N, CB * v, v, C, M, kind))
    return cases


@pytest.mark.parametrize("case", _random_cases(48, 2024), ids=lambda c: "n%d_k%d_v%d_c%d_m%d_%s" % c[1:])
def test_random_shapes_against_the_oracle(ctx, case):
    """Seeded random shapes across every kernel variant (search: bf16 narrow / wide, exact, generic; gather:
    one-hot, paired, byte adder, fp32 one and two tokens per lane, grouped), with a non-zero LUT bias in both
    bias modes for the int8 table."""
    i, N, K, v, C, M, kind = case
    x, cent, lut, bias = make_case(7000 + i, N, K, v, C, M, "f32" if kind == "f32" else "i8")
    CB = K // v
    want_idx = oracle.index_calculation(x, cent, v, threads=THREADS)
    if kind == "i8":
        mode = i % 2
        amm = ctx.amm(cent, lut, np.float32(0.0371), bias, max_n=N, lut_bias=0.25, bias_mode=mode)
        out, idx, acc = amm.run_debug(x)
        want_acc = oracle.gather_i8(want_idx, lut, threads=THREADS)
        assert np.array_equal(idx, want_idx)
        assert np.array_equal(acc, want_acc)
        want = oracle.dequant(want_acc, bias, CB, 0.0371, 0.25, mode, threads=THREADS)
        assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    elif kind == "f32":
        amm = ctx.amm(cent, lut, None, bias, max_n=N)
        out, idx, _ = amm.run_debug(x)
        assert np.array_equal(idx, want_idx)
        np.testing.assert_allclose(out, oracle.gather_f32(want_idx, lut, bias, threads=THREADS), rtol=1e-5,
                                   atol=1e-5 * np.sqrt(CB))
    else:
        group = 1 + i % 5
        scales = np.random.default_rng(i).uniform(1e-3, 0.1, (CB + group - 1) // group).astype(np.float32)
        amm = ctx.amm(cent, lut, scales, bias, max_n=N, scale_group=group)
        want = oracle.gather_i8_grouped(want_idx, lut, scales, bias, group, threads=THREADS)
        assert np.array_equal(amm.run(x).view(np.uint32), want.view(np.uint32))
    amm.close()
