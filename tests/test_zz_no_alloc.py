"""The allocation-free entry point, pimdl_amm_run_noalloc, against pimdl_amm_run (through the C ABI).

Bar: the output bits of the existing entry point (which the other GPU tests hold bit-exact against
the oracle).  Two calls in a row share the library's fixed scratch array, the second with a smaller
input; a third operator with 8-bit indices follows on the same array.  Sizes beyond the array and
host pointers are refused."""
import numpy as np
import pytest

import oracle
from __graft_entry__ import load_package

pimdl = load_package()
pytestmark = pytest.mark.gpu

THREADS = 8


@pytest.fixture(scope="module")
def ctx():
    c = pimdl.Context(0)
    yield c
    c.close()


def _case(seed, N, K, v, C, M):
    rng = np.random.default_rng(seed)
    CB = K // v
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (CB, C, M)).astype(np.int8)
    bias = rng.standard_normal(M).astype(np.float32)
    return x, cent, lut, bias


def _both(amm, xd, n, M):
    """(existing entry point, allocation-free entry point) on the same device input, as numpy arrays."""
    import torch

    ref = torch.full((n, M), -3.0, device="cuda")
    got = torch.full((n, M), -5.0, device="cuda")
    torch.cuda.synchronize()
    amm.run_ptr(xd.data_ptr(), n, ref.data_ptr())
    amm.run_noalloc_ptr(xd.data_ptr(), n, got.data_ptr())
    amm.ctx.synchronize()
    return ref.cpu().numpy(), got.cpu().numpy()


def test_noalloc_matches_run_on_two_calls_in_a_row(ctx):
    import torch

    # first call: 1000 tokens (ragged: not a multiple of the 64-token index blocks), 4-bit indices
    N1, K, v, C, M = 1000, 768, 4, 16, 768
    x, cent, lut, bias = _case(11, N1, K, v, C, M)
    amm = ctx.amm(cent, lut, np.float32(0.0123), bias, max_n=N1)
    xd = torch.from_numpy(x).cuda()
    ref1, got1 = _both(amm, xd, N1, M)
    assert np.array_equal(ref1.view(np.uint32), got1.view(np.uint32))
    # ... and against the oracle, on a row sample
    rows = np.arange(0, N1, 37)
    idx = oracle.index_calculation(x[rows], cent, v, threads=THREADS)
    want = oracle.dequant(oracle.gather_i8(idx, lut, threads=THREADS), bias, K // v, 0.0123, 0.0, 0, threads=THREADS)
    assert np.array_equal(got1[rows].view(np.uint32), want.view(np.uint32))

    # second call, smaller input: the scratch still holds the first call's indices beyond these rows
    N2 = 130
    x2 = np.ascontiguousarray(x[::-1][:N2])
    xd2 = torch.from_numpy(x2).cuda()
    ref2, got2 = _both(amm, xd2, N2, M)
    assert np.array_equal(ref2.view(np.uint32), got2.view(np.uint32))
    idx2 = oracle.index_calculation(x2, cent, v, threads=THREADS)
    want2 = oracle.dequant(oracle.gather_i8(idx2, lut, threads=THREADS), bias, K // v, 0.0123, 0.0, 0, threads=THREADS)
    assert np.array_equal(got2.view(np.uint32), want2.view(np.uint32))
    amm.close()

    # another operator on the same array: 8-bit indices (32 centroids: one byte per codebook in the tiled order
    # of the matrix-core gather), fewer codebooks
    N3, K3, v3, C3, M3 = 77, 96, 8, 32, 100
    x3, cent3, lut3, bias3 = _case(12, N3, K3, v3, C3, M3)
    amm3 = ctx.amm(cent3, lut3, np.float32(0.5), bias3, max_n=N3)
    ref3, got3 = _both(amm3, torch.from_numpy(x3).cuda(), N3, M3)
    assert np.array_equal(ref3.view(np.uint32), got3.view(np.uint32))
    idx3 = oracle.index_calculation(x3, cent3, v3, threads=THREADS)
    want3 = oracle.dequant(oracle.gather_i8(idx3, lut3, threads=THREADS), bias3, K3 // v3, 0.5, 0.0, 0, threads=THREADS)
    assert np.array_equal(got3.view(np.uint32), want3.view(np.uint32))
    amm3.close()


def test_noalloc_first_call_on_a_fresh_context_allocates_nothing():
    """The entry point on a context and operator that have never seen pimdl_amm_run (nothing has sized the
    context's scratch buffers for it), with 64 centroids: row-major index rows of one byte per codebook and the
    byte-adder gather go through the fixed array.  Device memory in use must not change across the calls."""
    import torch

    N, K, v, C, M = 500, 256, 4, 64, 128
    x, cent, lut, bias = _case(15, N, K, v, C, M)
    idx = oracle.index_calculation(x, cent, v, threads=THREADS)
    want = oracle.dequant(oracle.gather_i8(idx, lut, threads=THREADS), bias, K // v, 0.25, 0.0, 0, threads=THREADS)
    xd = torch.from_numpy(x).cuda()
    got1 = torch.full((N, M), -5.0, device="cuda")
    got2 = torch.full((200, M), -5.0, device="cuda")
    # the kernels' code objects reach the device at their first launch: take that out of the measurement with
    # the same entry point on another context
    warm = pimdl.Context(0)
    wamm = warm.amm(cent, lut, np.float32(0.25), bias, max_n=N)
    wamm.run_noalloc_ptr(xd.data_ptr(), N, got1.data_ptr())
    warm.synchronize()
    got1.fill_(-5.0)

    fresh = pimdl.Context(0)
    amm = fresh.amm(cent, lut, np.float32(0.25), bias, max_n=N)
    assert amm.last_gather_kernel() == ""   # never launched
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    amm.run_noalloc_ptr(xd.data_ptr(), N, got1.data_ptr())
    fresh.synchronize()
    free1 = torch.cuda.mem_get_info()[0]
    amm.run_noalloc_ptr(xd.data_ptr(), 200, got2.data_ptr())   # second call, smaller input
    fresh.synchronize()
    free2 = torch.cuda.mem_get_info()[0]
    assert free0 == free1 == free2, (free0, free1, free2)
    assert amm.last_gather_kernel().startswith("gather_i8_kernel<64,")
    assert np.array_equal(got1.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got2.cpu().numpy().view(np.uint32), want[:200].view(np.uint32))
    # and the existing entry point gives the same bits
    ref = torch.empty((N, M), device="cuda")
    amm.run_ptr(xd.data_ptr(), N, ref.data_ptr())
    fresh.synchronize()
    assert np.array_equal(ref.cpu().numpy().view(np.uint32), want.view(np.uint32))
    amm.close()
    wamm.close()
    fresh.close()
    warm.close()


def test_noalloc_fp32_table(ctx):
    import torch

    N, K, v, C, M = 300, 256, 4, 16, 200
    rng = np.random.default_rng(13)
    x = rng.standard_normal((N, K)).astype(np.float32)
    cent = rng.standard_normal((K // v, C, v)).astype(np.float32)
    lut = rng.standard_normal((K // v, C, M)).astype(np.float32)
    amm = ctx.amm(cent, lut, None, None, max_n=N)
    ref, got = _both(amm, torch.from_numpy(x).cuda(), N, M)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))
    amm.close()


def test_noalloc_refuses_what_it_cannot_hold(ctx):
    import torch

    # 8192 tokens x 1536 codebooks x 1 byte = 12 MiB of packed indices: more than the fixed array
    N, K, v, C, M = 8192, 3072, 2, 32, 16
    rng = np.random.default_rng(14)
    cent = rng.standard_normal((K // v, C, v)).astype(np.float32)
    lut = rng.integers(-128, 128, (K // v, C, M)).astype(np.int8)
    amm = ctx.amm(cent, lut, np.float32(1.0), None, max_n=N)
    xd = torch.zeros((N, K), device="cuda")
    od = torch.zeros((N, M), device="cuda")
    with pytest.raises(pimdl.PimdlError) as e:
        amm.run_noalloc_ptr(xd.data_ptr(), N, od.data_ptr())
    assert e.value.code == pimdl.ERR_INVALID and "exceed the fixed scratch" in str(e.value)
    # what fits is served: 5000 tokens need 7.3 MiB
    n_ok = pimdl.NOALLOC_SCRATCH_BYTES // (K // v) // 64 * 64
    assert 0 < n_ok < N
    ref, got = _both(amm, xd, n_ok, M)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))
    # host pointers would need staging buffers: refused
    xh = np.zeros((4, K), np.float32)
    with pytest.raises(pimdl.PimdlError) as e:
        amm.run_noalloc_ptr(xh.ctypes.data, 4, od.data_ptr())
    assert e.value.code == pimdl.ERR_INVALID and "device pointers" in str(e.value)
    amm.close()
