"""The reference-compatible C++ host layer (include/pimdl/amm_host.h) and its CLI driver, checked
against the oracle, including the reference's DPU tile orders for indices, LUT and output."""
import os
import struct
import subprocess

import numpy as np
import pytest

import oracle
from __graft_entry__ import ROOT, load_package

pimdl = load_package()
pytestmark = pytest.mark.gpu

CLI = os.path.join(ROOT, "pim-dl-asplos_amd", "bin", "test_amm")
THREADS = 8


@pytest.fixture(scope="module")
def ctx():
    c = pimdl.Context(0)
    yield c
    c.close()


def tiled_view(rowmajor, n_stile, f_stile, f_mtile):
    """Row-major [N][M] -> flat array in the order the reference's amm_host returns (test_amm.cpp:193-202)."""
    N, M = rowmajor.shape
    out = np.empty(N * M, rowmajor.dtype)
    lut_par = M // f_stile
    for n in range(N):
        for f in range(M):
            out[oracle.output_offset(n, f, n_stile, f_stile, f_mtile, lut_par)] = rowmajor[n, f]
    return out


def read_dump(path):
    raw = open(path, "rb").read()
    hdr = struct.unpack_from("<12I", raw, 0)
    N, K, v, C, M, ns, cm, fs, fm, load_type, fl, cl = hdr
    scale, lut_bias = struct.unpack_from("<2f", raw, 48)
    off = 56
    CB = K // v

    def take(count, dtype):
        nonlocal off
        a = np.frombuffer(raw, dtype=dtype, count=count, offset=off)
        off += a.nbytes
        return a

    x = take(N * K, np.float32).reshape(N, K)
    cent = take(CB * C * v, np.float32).reshape(CB, C, v)
    lut = take(CB * C * M, np.int8).reshape(CB, C, M)
    bias = take(M, np.float32)
    out = take(N * M, np.float32)
    assert off == len(raw)
    return dict(N=N, K=K, v=v, C=C, M=M, ns=ns, cm=cm, fs=fs, fm=fm, scale=scale, lut_bias=lut_bias, x=x, cent=cent,
                lut=lut, bias=bias, out=out)


def test_cli_driver_with_reference_yaml_and_dpu_tiling(tmp_path):
    """`test_amm config.yaml` as run_amm.py would launch it; the output buffer is in DPU order."""
    assert os.path.exists(CLI), "CLI not built (run __graft_entry__.build())"
    dump = str(tmp_path / "dump.bin")
    cfg = os.path.join(ROOT, "tests", "golden", "amm_small_tiled.yaml")
    res = subprocess.run([CLI, cfg, "ignored_dpu_binary", "--dump", dump, "--rounds", "1", "2"], capture_output=True,
                         text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "PIM AVG AMM time" in res.stdout and res.stdout.count("PIM AMM time") == 3
    d = read_dump(dump)
    CB = d["K"] // d["v"]
    idx = oracle.index_calculation(d["x"], d["cent"], d["v"], threads=THREADS)
    acc = oracle.gather_i8(idx, d["lut"], threads=THREADS)
    # the host layer follows pim_lut's epilogue (bias * num_codebook, pim_lut_host.cpp:201)
    want = oracle.dequant(acc, d["bias"], CB, d["scale"], d["lut_bias"], 1, threads=THREADS)
    want_tiled = tiled_view(want, d["ns"], d["fs"], d["fm"])
    assert np.array_equal(d["out"].view(np.uint32), want_tiled.view(np.uint32))


def test_tiled_entry_points_through_the_c_abi(ctx):
    rng = np.random.default_rng(77)
    N, K, v, C, M = 96, 64, 4, 16, 96
    CB = K // v
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    bias = rng.standard_normal(M).astype(np.float32)
    amm = ctx.amm(cent, lut, np.float32(0.02), bias, max_n=N)
    ns, cm, fs, fm = 32, 8, 48, 16
    want_idx = oracle.index_calculation(x, cent, v)
    want = oracle.dequant(oracle.gather_i8(want_idx, lut), bias, CB, 0.02, 0.0, 0)
    got = amm.run_tiled(x, ns, cm, fs, fm)
    assert np.array_equal(got.view(np.uint32), tiled_view(want, ns, fs, fm).view(np.uint32))
    # identity tiling == row-major
    assert np.array_equal(amm.run_tiled(x).reshape(N, M).view(np.uint32), want.view(np.uint32))
    # pim_lut's half: tiled index buffer in, tiled output out
    idx_tiled = oracle.index_calculation(x, cent, v, ns, cm)
    got2 = amm.lut_gather_tiled(idx_tiled, N, ns, cm, fs, fm)
    assert np.array_equal(got2.view(np.uint32), tiled_view(want, ns, fs, fm).view(np.uint32))
    # context-level index_calculation (centroids passed per call, as in the reference)
    assert np.array_equal(ctx.index_calculation(x, cent), want_idx)
    assert np.array_equal(ctx.index_calculation(x, cent, ns, cm), idx_tiled)
    with pytest.raises(pimdl.PimdlError):
        amm.run_tiled(x, 7, 0, 0, 0)  # does not divide n
    amm.close()
