"""Pins the CPU oracle (oracle/pimdl_oracle.c) before anything is compared against it.

Each oracle function is checked against something it was not derived from: the reference's own
compiled index_calculation (fixtures, and live where oracle/_ref exists), closed forms that
separate the reference's hysteresis scan from a true argmin, library routines (integer matmul,
einsum), and invariants.
"""
import numpy as np
import pytest

import oracle


def _cases(golden):
    for i in range(int(golden["ncases"])):
        yield i, str(golden[f"c{i}_kind"]), golden[f"c{i}_x"], golden[f"c{i}_cent"], golden[f"c{i}_idx"]


# ------------------------------------------------------------------ A1 closest-centroid search


def test_index_matches_reference_golden(golden_index):
    n = 0
    for i, kind, x, cent, idx in _cases(golden_index):
        v = cent.shape[2]
        got = oracle.index_calculation(x, cent, v)
        assert np.array_equal(got, idx), f"case {i} ({kind})"
        assert np.array_equal(oracle.np_index_calculation(x, cent), idx), f"numpy, case {i} ({kind})"
        n += 1
    assert n == 21


def test_index_tiled_layout_matches_reference_golden(golden_index):
    for key in golden_index.files:
        if "_tiled_" not in key:
            continue
        cid, _, n_stile, cb_mtile = key.split("_")
        x, cent = golden_index[f"{cid}_x"], golden_index[f"{cid}_cent"]
        got = oracle.index_calculation(x, cent, cent.shape[2], int(n_stile), int(cb_mtile))
        assert np.array_equal(got, golden_index[key]), key


def test_golden_contains_cases_where_scan_differs_from_true_argmin(golden_index):
    """The fixtures must be able to catch an implementation that uses a plain argmin."""
    differing = 0
    for i, kind, x, cent, idx in _cases(golden_index):
        d = oracle.np_distances(x, cent)
        differing += int((d.argmin(-1) != idx).sum())
    assert differing > 20


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (needs the reference tree)")
@pytest.mark.parametrize("v,C", [(2, 16), (4, 16), (8, 8), (4, 32), (16, 16), (32, 64), (4, 128)])
def test_index_matches_reference_live(v, C):
    rng = np.random.default_rng(v * 1000 + C)
    N, CB = 64, 24
    x = rng.standard_normal((N, CB * v)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    want = oracle.ref_index_calculation(x, cent, v, threads=2)
    assert np.array_equal(oracle.index_calculation(x, cent, v, threads=2), want)
    # non-identity tiling
    want_t = oracle.ref_index_calculation(x, cent, v, 16, 8)
    assert np.array_equal(oracle.index_calculation(x, cent, v, 16, 8), want_t)


def _one_subvector(dists):
    """Build (x, cent) with v=1 whose distances to x=0 are exactly `dists` when they are squares
    of fp32 numbers: cent_c = sqrt(d_c) must square back exactly, so callers pass roots."""
    roots = np.asarray(dists, dtype=np.float32)
    cent = roots.reshape(1, -1, 1)
    x = np.zeros((1, 1), dtype=np.float32)
    return x, cent, (roots * roots).astype(np.float32)


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (needs the reference tree)")
def test_index_matches_reference_live_on_non_finite_values():
    """NaN / Inf / overflowing values: the restatement must keep the reference's compare semantics
    (`best - d > 1e-6` is false for NaN, so a NaN never replaces the running best)."""
    rng = np.random.default_rng(7)
    N, CB, C, v = 64, 24, 16, 4
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    cent[3, 2, 0] = np.nan
    cent[5, 0, 1] = np.nan
    cent[7, 4, 0] = np.inf
    cent[9, 1, :] = 3e19
    x = rng.standard_normal((N, CB * v)).astype(np.float32)
    x[1, :] = np.nan
    x[2, 5] = np.inf
    x[4, :] = 2e19
    with np.errstate(all="ignore"):
        got = oracle.index_calculation(x, cent, v, threads=2)
        want = oracle.ref_index_calculation(x, cent, v, threads=2)
    assert np.array_equal(got, want)
    assert (got[:, 5] == 0).all()  # NaN in centroid 0 pins the scan at index 0


def test_scan_hysteresis_closed_forms():
    # equal to centroid j => j
    rng = np.random.default_rng(1)
    cent = rng.standard_normal((5, 16, 4)).astype(np.float32)
    x = np.concatenate([cent[cb, (3 * cb + 1) % 16] for cb in range(5)])[None, :]
    assert oracle.index_calculation(x, cent, 4)[0].tolist() == [(3 * cb + 1) % 16 for cb in range(5)]
    # all centroids identical => 0
    cent0 = np.repeat(cent[:, :1], 16, axis=1)
    assert not oracle.index_calculation(rng.standard_normal((7, 20)).astype(np.float32), cent0, 4).any()

    # chains on explicit distances (through np_scan_argmin, and through the C code with v=1)
    one = np.float32(1.0)
    d_chain = np.array([one, one - np.float32(0.8e-6), one - np.float32(1.6e-6)], dtype=np.float32)
    assert oracle.np_scan_argmin(d_chain[None, :])[0] == 2      # 1 - d[2] = 1.6e-6 > 1e-6
    d_stall = np.array([one, one - np.float32(0.8e-6), one - np.float32(0.9e-6)], dtype=np.float32)
    assert oracle.np_scan_argmin(d_stall[None, :])[0] == 0      # true argmin would say 2
    assert int(np.argmin(d_stall)) == 2

    # the same through the C path: v=1, x=0, centroids = roots
    roots = np.sqrt(np.array([1.0, 1.0 - 0.8e-6, 1.0 - 0.9e-6], dtype=np.float64)).astype(np.float32)
    x, cent1, d = _one_subvector(roots)
    want = oracle.np_scan_argmin(d[None, :])[0]
    assert oracle.index_calculation(x, cent1, 1)[0, 0] == want
    # a later, clearly smaller distance is taken
    x, cent1, d = _one_subvector(np.array([2.0, 1.5, 1.5, 1.0, 3.0], dtype=np.float32))
    assert oracle.index_calculation(x, cent1, 1)[0, 0] == 3
    # exact tie keeps the earlier index
    x, cent1, d = _one_subvector(np.array([2.0, 1.0, 1.0, 1.0], dtype=np.float32))
    assert oracle.index_calculation(x, cent1, 1)[0, 0] == 1


def test_threshold_is_the_double_literal():
    """(float)1e-6 < 1e-6 < nextafter((float)1e-6): a difference of exactly (float)1e-6 must NOT
    switch, the next float up must."""
    t = np.float32(1e-6)
    assert float(t) < 1e-6 < float(np.nextafter(t, np.float32(1)))
    for diff, expect in ((t, 0), (np.nextafter(t, np.float32(1)), 1)):
        d = np.array([diff, np.float32(0.0)], dtype=np.float32)  # best - d[1] = diff exactly
        assert oracle.np_scan_argmin(d[None, :])[0] == expect


def test_distances_are_unfused_and_in_dimension_order():
    """The C distances equal the numpy chain of separately rounded fp32 ops, and differ from a
    float64 evaluation in at least one place (so the test can see a fused/reordered version)."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((32, 64)).astype(np.float32)
    cent = rng.standard_normal((8, 16, 8)).astype(np.float32)
    d_c = oracle.distances(x, cent, 8)
    d_np = oracle.np_distances(x, cent)
    assert np.array_equal(d_c.view(np.uint32), d_np.view(np.uint32))
    d64 = ((x.reshape(32, 8, 1, 8).astype(np.float64) - cent[None].astype(np.float64)) ** 2).sum(-1)
    assert (d64.astype(np.float32) != d_c).any()
    # reversed dimension order gives different bits somewhere
    d_rev = oracle.np_distances(x.reshape(32, 8, 8)[:, :, ::-1].reshape(32, 64), cent[:, :, ::-1])
    assert (d_rev.view(np.uint32) != d_c.view(np.uint32)).any()


def test_index_brute_force_tiny():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 6)).astype(np.float32)
    cent = rng.standard_normal((3, 4, 2)).astype(np.float32)
    got = oracle.index_calculation(x, cent, 2)
    for n in range(5):
        for cb in range(3):
            dist = []
            for c in range(4):
                d = np.float32(0)
                for t in range(2):
                    diff = np.float32(x[n, cb * 2 + t] - cent[cb, c, t])
                    d = np.float32(d + np.float32(diff * diff))
                dist.append(d)
            best, bi = dist[0], 0
            for c in range(1, 4):
                if float(np.float32(best - dist[c])) > 1e-6:
                    best, bi = dist[c], c
            assert got[n, cb] == bi


# ------------------------------------------------------------------ A3 gather, A4 epilogue


def _rand_amm(rng, N, CB, C, M):
    idx = rng.integers(0, C, (N, CB)).astype(np.uint16)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    return idx, lut


def test_gather_equals_integer_onehot_matmul():
    rng = np.random.default_rng(11)
    idx, lut = _rand_amm(rng, 37, 29, 16, 50)
    acc = oracle.gather_i8(idx, lut, threads=2)
    assert np.array_equal(acc, oracle.np_gather_onehot(idx, lut))


def test_gather_invariants():
    rng = np.random.default_rng(12)
    idx, lut = _rand_amm(rng, 16, 24, 8, 40)
    acc = oracle.gather_i8(idx, lut)
    perm = rng.permutation(24)
    assert np.array_equal(oracle.gather_i8(idx[:, perm], lut[perm]), acc)
    ones = np.ones_like(lut)
    assert (oracle.gather_i8(idx, ones) == 24).all()
    # extremes: all -128 with CB codebooks
    assert (oracle.gather_i8(idx, np.full_like(lut, -128)) == -128 * 24).all()
    # row-constant LUT: entry (cb, c, :) = c - 3 => acc = sum_cb idx - 3*CB
    rc = np.broadcast_to((np.arange(8) - 3).astype(np.int8)[None, :, None], lut.shape)
    want = idx.astype(np.int32).sum(1, keepdims=True) - 3 * 24
    assert np.array_equal(oracle.gather_i8(idx, rc), np.broadcast_to(want, (16, 40)))


def test_dequant_closed_form():
    rng = np.random.default_rng(13)
    acc = rng.integers(-50000, 50000, (9, 21)).astype(np.int32)
    bias_t = rng.standard_normal(21).astype(np.float32)
    scale, lb = np.float32(0.0123), np.float32(0.2)
    want0 = (acc.astype(np.float32) * scale + lb) + bias_t[None, :]
    want1 = (acc.astype(np.float32) * scale + np.float32(lb * np.float32(7))) + bias_t[None, :]
    assert np.array_equal(oracle.dequant(acc, bias_t, 7, scale, lb, 0), want0.astype(np.float32))
    assert np.array_equal(oracle.dequant(acc, bias_t, 7, scale, lb, 1), want1.astype(np.float32))
    # the two reference epilogues agree when lut_bias == 0
    assert np.array_equal(oracle.dequant(acc, bias_t, 7, scale, 0.0, 0), oracle.dequant(acc, bias_t, 7, scale, 0.0, 1))


def test_amm_cpu_is_the_composition():
    rng = np.random.default_rng(14)
    N, CB, v, C, M = 20, 12, 4, 16, 24
    x = rng.standard_normal((N, CB * v)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    bias_t = rng.standard_normal(M).astype(np.float32)
    out, idx, acc = oracle.amm_cpu(x, cent, lut, bias_t, v, 0.05, 0.0, threads=2)
    assert np.array_equal(idx, oracle.np_index_calculation(x, cent))
    assert np.array_equal(acc, oracle.np_gather_onehot(idx, lut))
    assert np.array_equal(out, (acc.astype(np.float32) * np.float32(0.05) + np.float32(0)) + bias_t)


def test_gather_f32_against_float64():
    rng = np.random.default_rng(15)
    N, CB, C, M = 10, 48, 16, 33
    idx = rng.integers(0, C, (N, CB)).astype(np.uint16)
    lut = rng.standard_normal((CB, C, M)).astype(np.float32)
    bias_t = rng.standard_normal(M).astype(np.float32)
    got = oracle.gather_f32(idx, lut, bias_t)
    want = lut.astype(np.float64)[np.arange(CB)[None, :], idx.astype(np.int64)].sum(1) + bias_t
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # exact statement of the fixed order
    acc = np.zeros((N, M), np.float32)
    for cb in range(CB):
        acc = (acc + lut[cb, idx[:, cb].astype(np.int64)]).astype(np.float32)
    assert np.array_equal(got, (acc + bias_t).astype(np.float32))


def test_gather_grouped_reduces_to_per_tensor_and_matches_numpy():
    rng = np.random.default_rng(16)
    N, CB, C, M = 9, 24, 16, 20
    idx, lut = _rand_amm(rng, N, CB, C, M)
    bias_t = rng.standard_normal(M).astype(np.float32)
    one = np.array([0.01], np.float32)
    per_tensor = oracle.dequant(oracle.gather_i8(idx, lut), bias_t, CB, 0.01, 0.0, 0)
    assert np.array_equal(oracle.gather_i8_grouped(idx, lut, one, bias_t, CB), per_tensor)
    for group in (1, 4, 5, 24):
        ng = (CB + group - 1) // group
        scales = rng.uniform(0.001, 0.02, ng).astype(np.float32)
        got = oracle.gather_i8_grouped(idx, lut, scales, bias_t, group)
        acc = np.zeros((N, M), np.float32)
        for g in range(ng):
            sl = slice(g * group, min(CB, (g + 1) * group))
            part = oracle.np_gather_onehot(idx[:, sl], lut[sl])
            acc = (acc + (part.astype(np.float32) * scales[g]).astype(np.float32)).astype(np.float32)
        assert np.array_equal(got, (acc + bias_t).astype(np.float32)), group


# ------------------------------------------------------------------ A5 LUT construction


def test_lutgen_against_einsum_and_degenerate_case():
    rng = np.random.default_rng(17)
    CB, C, v, M = 12, 16, 4, 40
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    W = (rng.standard_normal((CB * v, M)) * 0.02).astype(np.float32)
    lut = oracle.lutgen_f32(cent, W, threads=2)
    want = np.einsum("bcv,bvm->bcm", cent.astype(np.float64), W.reshape(CB, v, M).astype(np.float64))
    assert np.allclose(lut, want, rtol=1e-5, atol=1e-7)
    # a weight operand read as [M][K] instead of [K][M] is caught
    bad = np.einsum("bcv,bvm->bcm", cent, W.reshape(M, CB * v).T.reshape(CB, v, M))
    assert not np.allclose(lut, bad, rtol=1e-3, atol=1e-4)
    # v=1, C=1: the LUT is W scaled row-wise by the single centroid coordinate
    cent1 = rng.standard_normal((6, 1, 1)).astype(np.float32)
    W1 = rng.standard_normal((6, 10)).astype(np.float32)
    assert np.array_equal(oracle.lutgen_f32(cent1, W1)[:, 0, :], (cent1[:, 0, :] * W1).astype(np.float32))


def test_lut_quant_matches_published_formula_and_invariants():
    rng = np.random.default_rng(18)
    lut = (rng.standard_normal((10, 16, 30)) * 0.3).astype(np.float32)
    q, scales = oracle.lut_quant(lut)
    q_np, scale_np = oracle.np_lut_quant(lut)
    assert scales.shape == (1,) and scales[0] == scale_np
    assert np.array_equal(q, q_np)
    assert np.abs(q.astype(np.int32)).max() == 127          # the extreme value maps to +-127
    assert (np.abs(q.astype(np.float32) * scales[0] - lut) <= scales[0] * 0.5 * (1 + 1e-6)).all()
    # ties go to even: values exactly k+0.5 scale units
    scale = np.float32(1.0)
    t = np.array([[[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5]]], dtype=np.float32)
    q2, s2 = oracle.lut_quant(t)
    assert s2[0] == scale
    assert q2.reshape(-1).tolist() == [127, 0, 2, 2, 0, -2, -2, 126]
    # per-codebook groups (extension): each block is quantised on its own
    qg, sg = oracle.lut_quant(lut, group_codebooks=2)
    assert sg.shape == (5,)
    for g in range(5):
        qq, ss = oracle.np_lut_quant(lut[2 * g:2 * g + 2])
        assert ss == sg[g] and np.array_equal(qq, qg[2 * g:2 * g + 2])


# ------------------------------------------------------------------ DPU layouts (compat shim)


def test_layout_helpers():
    rng = np.random.default_rng(19)
    CB, C, M = 4, 8, 24
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    # identity tile => unchanged; otherwise a permutation with the documented formula
    assert np.array_equal(oracle.reorder_pim_lut(lut, M), lut.reshape(-1))
    r = oracle.reorder_pim_lut(lut, 8)
    assert sorted(r.tolist()) == sorted(lut.reshape(-1).tolist())
    assert np.array_equal(r.reshape(M // 8, CB, C, 8), lut.reshape(CB, C, M // 8, 8).transpose(2, 0, 1, 3))
    # output offsets: bijection, and row-major under the identity tiling
    N = 12
    offs = {oracle.output_offset(n, f, 4, 12, 6, 2) for n in range(N) for f in range(M)}
    assert offs == set(range(N * M))
    assert all(oracle.output_offset(n, f, N, M, M, 1) == n * M + f for n in range(N) for f in range(M))
    # index pre-scaling (pim_lut_host.cpp:59,80,96-104) on an identity-tiled buffer
    idx = rng.integers(0, C, (N, CB)).astype(np.uint16)
    assert np.array_equal(oracle.prepare_input_index(idx, N, CB, C, N, CB, 0, 24, 8, 2).reshape(N, CB), idx * 24)
    assert np.array_equal(oracle.prepare_input_index(idx, N, CB, C, N, CB, 1, 24, 8, 2).reshape(N, CB), idx * 8)
    want = (np.arange(CB)[None, :] % 2) * C * 8 + idx * 8
    assert np.array_equal(oracle.prepare_input_index(idx, N, CB, C, N, CB, 2, 24, 8, 2).reshape(N, CB), want)


@pytest.mark.parametrize("N,CB,C,ns,cm,fs,flt,cblt", [(12, 8, 16, 4, 4, 24, 8, 2), (6, 12, 5, 3, 6, 10, 5, 3),
                                                      (8, 8, 32, 2, 8, 4096, 4096, 4)])
def test_prepare_input_index_under_a_dpu_tiling(N, CB, C, ns, cm, fs, flt, cblt):
    """pim_lut_host.cpp:40-104 on a buffer in the search's tiled order (index_calc_host.cpp:41-49), stated without
    the offset formula: that order is the row-major [N][CB] array cut into (N/ns, ns, CB/cm, cm) with the two middle
    axes swapped, and the rewrite depends on an entry's value and on its position inside its cb_mtile only.  The
    last case overflows 16 bits, which the reference's uint16 buffer truncates."""
    rng = np.random.default_rng(N * 131 + CB)
    idx = rng.integers(0, C, (N, CB)).astype(np.uint16)
    tiled = np.ascontiguousarray(idx.reshape(N // ns, ns, CB // cm, cm).transpose(0, 2, 1, 3))   # [n_tile][cb_tile][n_in][cb_in]
    wide = tiled.astype(np.uint32)
    cb_in = np.arange(cm, dtype=np.uint32)[None, None, None, :]
    want = {0: wide * fs, 1: wide * flt, 2: (cb_in % cblt) * C * flt + wide * flt}
    for load_type in (0, 1, 2):
        got = oracle.prepare_input_index(tiled.reshape(-1), N, CB, C, ns, cm, load_type, fs, flt, cblt)
        assert np.array_equal(got.reshape(tiled.shape), (want[load_type] & 0xFFFF).astype(np.uint16)), load_type
    # the search's own tiled output is that same array view (ties the two layout statements together)
    x = rng.standard_normal((N, CB * 2)).astype(np.float32)
    cent = rng.standard_normal((CB, C, 2)).astype(np.float32)
    rm = oracle.index_calculation(x, cent, 2)
    til = oracle.index_calculation(x, cent, 2, n_stile=ns, cb_mtile=cm)
    assert np.array_equal(np.asarray(til).reshape(N // ns, CB // cm, ns, cm), rm.reshape(N // ns, ns, CB // cm, cm).transpose(0, 2, 1, 3))


def test_layer_norm_closed_form():
    rng = np.random.default_rng(20)
    x = rng.standard_normal((6, 64)).astype(np.float32) * 3 + 1
    g = rng.standard_normal(64).astype(np.float32)
    b = rng.standard_normal(64).astype(np.float32)
    y = oracle.layer_norm(x, g, b)
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-6) * g + b
    assert np.allclose(y, want, rtol=1e-5, atol=1e-5)
