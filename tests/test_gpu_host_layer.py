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
    idx = take(N * CB, np.uint16) if off < len(raw) else None  # --split: the index buffer as pim_lut left it
    assert off == len(raw)
    return dict(N=N, K=K, v=v, C=C, M=M, ns=ns, cm=cm, fs=fs, fm=fm, scale=scale, lut_bias=lut_bias, x=x, cent=cent,
                lut=lut, bias=bias, out=out, idx=idx, load_type=load_type, fl=fl, cl=cl)


def run_cli(tmp_path, *flags):
    assert os.path.exists(CLI), "CLI not built (run __graft_entry__.build())"
    dump = str(tmp_path / "dump.bin")
    cfg = os.path.join(ROOT, "tests", "golden", "amm_small_tiled.yaml")
    res = subprocess.run([CLI, cfg, "ignored_dpu_binary", "--dump", dump, *flags], capture_output=True, text=True,
                         timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    return res.stdout, read_dump(dump)


def expected_tiled_output(d):
    CB = d["K"] // d["v"]
    idx = oracle.index_calculation(d["x"], d["cent"], d["v"], threads=THREADS)
    acc = oracle.gather_i8(idx, d["lut"], threads=THREADS)
    # the host layer follows pim_lut's epilogue (bias * num_codebook, pim_lut_host.cpp:201)
    want = oracle.dequant(acc, d["bias"], CB, d["scale"], d["lut_bias"], 1, threads=THREADS)
    return tiled_view(want, d["ns"], d["fs"], d["fm"])


def test_cli_driver_with_reference_yaml_and_dpu_tiling(tmp_path):
    """`test_amm config.yaml` as run_amm.py would launch it; the output buffer is in DPU order."""
    stdout, d = run_cli(tmp_path, "--rounds", "1", "2")
    assert "PIM AVG AMM time" in stdout and stdout.count("PIM AMM time") == 3
    assert np.array_equal(d["out"].view(np.uint32), expected_tiled_output(d).view(np.uint32))


@pytest.mark.parametrize("load_type", [0, 1, 2])
def test_index_calculation_then_pim_lut(tmp_path, load_type):
    """The two halves of amm_host called one after the other through their C++ signatures
    (index_calc_host.h:5, pim_lut_host.h:13-14) with a non-identity DPU tiling, for the static, fine-grain and
    coarse-grain LUT orders: the output, and the index buffer as pim_lut leaves it (pim_lut_host.cpp:40-104)."""
    stdout, d = run_cli(tmp_path, "--split", "--load-type", str(load_type), "--rounds", "1", "1")
    assert d["load_type"] == load_type and d["idx"] is not None
    assert np.array_equal(d["out"].view(np.uint32), expected_tiled_output(d).view(np.uint32))
    CB = d["K"] // d["v"]
    ids = oracle.index_calculation(d["x"], d["cent"], d["v"], d["ns"], d["cm"], threads=THREADS)
    want_idx = oracle.prepare_input_index(ids, d["N"], CB, d["C"], d["ns"], d["cm"], load_type, d["fs"], d["fl"], d["cl"])
    assert np.array_equal(d["idx"], want_idx)
    assert not np.array_equal(want_idx, np.asarray(ids).reshape(-1))  # the rewrite changed something


@pytest.mark.parametrize("flags", [(), ("--split",)])
def test_inputs_changed_in_place_between_calls(tmp_path, flags):
    """bias, LUT entries and a centroid change behind the same pointers before the last call; the reference reads
    all of them anew on every call (pim_lut_host.cpp:143,201), so the last output must follow the new values."""
    stdout, d = run_cli(tmp_path, "--refill", "--rounds", "1", "2", *flags)
    assert "inputs changed in place" in stdout
    assert np.array_equal(d["out"].view(np.uint32), expected_tiled_output(d).view(np.uint32))


def test_assume_unchanged_skips_the_change_detection(tmp_path):
    """PimdlHostOptions::assume_unchanged: LUT and centroids are not read again once uploaded, so their in-place
    changes before the last call go unnoticed (the dump then holds them as uploaded), while the bias tensor, which
    is compared on every call, is followed.  Without changes the option changes nothing."""
    stdout, d = run_cli(tmp_path, "--assume-unchanged", "--rounds", "1", "2")
    assert np.array_equal(d["out"].view(np.uint32), expected_tiled_output(d).view(np.uint32))
    stdout, d = run_cli(tmp_path, "--assume-unchanged", "--refill", "--rounds", "1", "2")
    assert "inputs changed in place" in stdout
    assert np.array_equal(d["out"].view(np.uint32), expected_tiled_output(d).view(np.uint32))
    # the same run without the option sees the new tables: another output
    _, d2 = run_cli(tmp_path, "--refill", "--rounds", "1", "2")
    assert np.array_equal(d2["bias"], d["bias"]) and not np.array_equal(d2["lut"], d["lut"])
    assert not np.array_equal(d2["out"], d["out"])


def test_breakdown_lines_of_the_reference(tmp_path):
    """--breakdown: the two lines the reference's AMM_BREAKDOWN build prints per call (amm_host.cpp:24,
    pim_lut_host.cpp:211), cumulative seconds that only grow, and the same output bits."""
    import re
    stdout, d = run_cli(tmp_path, "--breakdown", "--rounds", "1", "3")
    assert np.array_equal(d["out"].view(np.uint32), expected_tiled_output(d).view(np.uint32))
    ic = [float(m) for m in re.findall(r"^index calculation time (\d+\.\d{6})$", stdout, re.M)]
    rest = re.findall(r"^other latency (\d+\.\d{6}), data transfer latency (\d+\.\d{6}), pim kernel latency (\d+\.\d{6})$", stdout, re.M)
    assert len(ic) == 4 and len(rest) == 4
    cols = np.array([[float(v) for v in r] for r in rest])
    assert all(np.diff(ic) > 0) and (np.diff(cols, axis=0) >= 0).all() and (cols[-1] > 0).all()


def test_host_buffers_in_chunks(ctx, monkeypatch):
    """Host pointers go through the pinned staging ring in chunks of tokens; with 512-token chunks a batch of 3000
    tokens is six chunks, the last one ragged, on four slots.  Every combination of host and device buffers gives
    the bits of one launch over the whole batch on device buffers (and those are the oracle's)."""
    import torch
    monkeypatch.setenv("PIMDL_HOST_CHUNK_TOKENS", "512")
    rng = np.random.default_rng(31)
    N, K, v, C, M = 3000, 256, 4, 16, 320
    CB = K // v
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    bias = rng.standard_normal(M).astype(np.float32)
    amm = ctx.amm(cent, lut, np.float32(0.05), bias, max_n=N)
    want, _, _ = oracle.amm_cpu(x, cent, lut, bias, v, 0.05, 0.0, threads=THREADS)
    xd = torch.from_numpy(x).cuda()
    yd = torch.zeros((N, M), device="cuda")
    amm.run_ptr(xd.data_ptr(), N, yd.data_ptr())
    ctx.synchronize()
    assert np.array_equal(yd.cpu().numpy().view(np.uint32), want.view(np.uint32))
    for n in (N, 512, 513, 1):
        # host -> host
        out = np.full((n, M), -7.0, np.float32)
        amm.run_ptr(x.ctypes.data, n, out.ctypes.data)
        assert np.array_equal(out.view(np.uint32), want[:n].view(np.uint32)), n
        # host -> device (returns once the input is copied; the rest is stream-ordered)
        yd.fill_(-7.0)
        torch.cuda.synchronize()
        xcopy = x[:n].copy()
        amm.run_ptr(xcopy.ctypes.data, n, yd.data_ptr())
        xcopy[:] = 0.0   # the caller may reuse its input
        ctx.synchronize()
        assert np.array_equal(yd[:n].cpu().numpy().view(np.uint32), want[:n].view(np.uint32)), n
        # device -> host
        out = np.full((n, M), -7.0, np.float32)
        amm.run_ptr(xd.data_ptr(), n, out.ctypes.data)
        assert np.array_equal(out.view(np.uint32), want[:n].view(np.uint32)), n
    # a second operator with wider rows makes the ring's buffers grow
    M2 = 1024
    lut2 = rng.integers(-128, 128, (CB, C, M2)).astype(np.int8)
    amm2 = ctx.amm(cent, lut2, np.float32(0.05), None, max_n=N)
    want2, _, _ = oracle.amm_cpu(x, cent, lut2, np.zeros(M2, np.float32), v, 0.05, 0.0, threads=THREADS)
    out2 = np.empty((N, M2), np.float32)
    amm2.run_ptr(x.ctypes.data, N, out2.ctypes.data)
    assert np.array_equal(out2.view(np.uint32), want2.view(np.uint32))
    out = np.empty((N, M), np.float32)
    amm.run_ptr(x.ctypes.data, N, out.ctypes.data)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    amm.close()
    amm2.close()


def test_scratch_of_a_creeping_batch_stays_bounded():
    """A caller whose batch grows call by call: the context's grow-only scratch is replaced by geometrically larger
    buffers (old ones are kept for HIP graphs that may hold them), so what it holds in the end is a small multiple
    of what the largest call needs, not the sum over all calls."""
    import torch
    c = pimdl.Context(0)
    rng = np.random.default_rng(32)
    K, v, C, M = 64, 4, 16, 512
    CB = K // v
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    x = rng.standard_normal((2000, K)).astype(np.float32)
    amm = c.amm(cent, lut, np.float32(1.0), None, max_n=2000)
    amm.run_debug(x[:1])           # the debug path stages through the grow-only scratch (output, accumulators, ids)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for n in range(2, 2001, 3):
        amm.run_debug(x[:n])
    torch.cuda.synchronize()
    grown = free0 - torch.cuda.mem_get_info()[0]
    # the last call needs 2000 x (512 x 4 out + 512 x 4 acc + 16 x 2 ids + 64 x 4 in) = 8.8 MB; exact-size growth with
    # the old buffers kept would hold the sum over 667 calls, about 3 GB (the bound leaves room for the allocator's
    # own granularity on some eighty small buffers)
    assert grown < 256 << 20, grown
    amm.close()
    c.close()


def test_index_ids_out_of_range_are_refused(ctx):
    rng = np.random.default_rng(5)
    N, CB, C, M = 40, 6, 12, 32
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    amm = ctx.amm(np.zeros((CB, C, 2), np.float32), lut, np.float32(1.0), None, max_n=N)
    idx = rng.integers(0, C, (N, CB)).astype(np.uint16)
    want = oracle.dequant(oracle.gather_i8(idx, lut), np.zeros(M, np.float32), CB, 1.0, 0.0, 0)
    assert np.array_equal(amm.lut_gather(idx), want)
    bad = idx.copy()
    bad[17, 4] = C  # the first id that is not a centroid
    with pytest.raises(pimdl.PimdlError, match=r"token 17, codebook 4"):
        amm.lut_gather(bad)
    # a buffer already rewritten into table offsets, handed in again
    with pytest.raises(pimdl.PimdlError, match="not a centroid id"):
        amm.lut_gather(idx * np.uint16(M))
    amm.close()


def test_set_bias(ctx):
    rng = np.random.default_rng(6)
    N, K, v, C, M = 70, 32, 4, 16, 50
    CB = K // v
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    b1, b2 = rng.standard_normal(M).astype(np.float32), rng.standard_normal(M).astype(np.float32)
    amm = ctx.amm(cent, lut, np.float32(0.3), b1, max_n=N)
    for step, b in enumerate((b1, b2, None, b1)):
        if step:
            amm.set_bias(b)
        want, _, _ = oracle.amm_cpu(x, cent, lut, np.zeros(M, np.float32) if b is None else b, v, 0.3, 0.0)
        assert np.array_equal(amm.run(x).view(np.uint32), want.view(np.uint32))
    amm.close()


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
