"""The allocation-free entry point, cuvdia_spmm_offsets_noalloc_f32, against
cuvdia_spmm_offsets_f32 on the same operands: the two run the same kernels, so
the results must agree bit for bit (and both agree with the oracle within the
fp32 bar of the other GPU tests).  Every case makes two calls in a row, the
second on a smaller matrix with a shorter table, so that a table left over
from the first call would show.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

IP = ctypes.POINTER(ctypes.c_int)


def _rand_dia(o, rng, h, w, offsets):
    d = o.Dia(h, w, offsets, None, 1)
    d.vals[:] = np.nan                       # padding must never be read
    m = o.valid_mask(d)
    d.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    return d


def _both(L, D, torch, A, B, dst0, trans, alpha, beta):
    """Runs both entry points on copies of the same operands; returns the two results (host, Fortran order)."""
    vals = torch.from_numpy(A.vals).cuda()
    Bd = D.to_device_colmajor(B)
    batch = Bd.shape[0]
    n_in, n_out = (A.h, A.w) if trans == "t" else (A.w, A.h)
    outs = []
    for fn in (L.cuvdia_spmm_offsets_f32, L.cuvdia_spmm_offsets_noalloc_f32):
        out = D.to_device_colmajor(dst0)
        rc = fn(vals.data_ptr(), A.offsets.ctypes.data_as(IP), A.nd, A.stride, A.h, A.w, 1,
                Bd.data_ptr(), n_in, out.data_ptr(), n_out, batch, trans.encode(), alpha, beta, None)
        assert rc == 0, L.cuvdia_strerror(rc)
        outs.append((out, L.cuvdia_last_path()))
    torch.cuda.synchronize()
    return [(D.to_host_colmajor(o), p) for o, p in outs]


def _window(px, k):
    r = k // 2
    return [dy * px + dx for dy in range(-r, r + 1) for dx in range(-r, r + 1)]


# (h, w, offsets, batch) of the first call, then of the second, smaller one
CASES = [
    # tiled kernels: a 2-d window, then a narrower band on a smaller matrix
    ((1024, 1024, _window(32, 5), 96), (320, 320, [-9, -8, -7, 0, 1, 2, 40], 40)),
    # rectangular, unsorted table, 300 single-diagonal chunks (generic kernels), then a tiled call with 3 chunks
    ((700, 900, [7 * i - 1000 for i in range(300)][::-1], 64), (256, 192, [-3, -2, 5, 6, 7, 100], 32)),
    # narrow batch (generic kernels), then narrower still
    ((512, 512, [-64, -1, 0, 1, 64], 8), (200, 260, [0, 3], 1)),
]


@pytest.mark.parametrize("trans", ["n", "t"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_noalloc_matches_the_allocating_entry_point(oracle, case, trans):
    import torch
    from cuv_amd import _lib, dia as D
    import _gpu_util as gu
    L = _lib.lib()
    rng = np.random.default_rng(4200 + case)
    alpha, beta = 0.75, 0.5
    for h, w, offsets, batch in CASES[case]:
        A = _rand_dia(oracle, rng, h, w, offsets)
        n_in, n_out = (h, w) if trans == "t" else (w, h)
        B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
        dst0 = np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
        (ref, ref_path), (got, got_path) = _both(L, D, torch, A, B, dst0, trans, alpha, beta)
        assert got_path == ref_path
        assert np.array_equal(got, ref), "results of the two entry points differ (%dx%d, nd %d)" % (h, w, len(offsets))
        gu.assert_close_mag(got, oracle.prod(A, B, dst0, trans, alpha, beta),
                            oracle.prod_mag(A, B, dst0, trans, alpha, beta), "noalloc vs oracle")
    assert L.cuvdia_cache_clear() == 0


def test_noalloc_rejects_tables_beyond_its_capacity():
    import torch
    from cuv_amd import _lib
    L = _lib.lib()
    nd = 1025
    offs = np.arange(nd, dtype=np.int32)
    n = 2048
    vals = torch.zeros(nd * n, device="cuda:0")
    B = torch.zeros(32 * n, device="cuda:0")
    out = torch.full((32 * n,), 3.0, device="cuda:0")
    rc = L.cuvdia_spmm_offsets_noalloc_f32(vals.data_ptr(), offs.ctypes.data_as(IP), nd, n, n, n, 1,
                                           B.data_ptr(), n, out.data_ptr(), n, 32, b"n", 1.0, 0.0, None)
    assert rc == _lib.ETOOLARGE
    assert b"capacity" in L.cuvdia_strerror(rc)
    torch.cuda.synchronize()
    assert bool((out == 3.0).all()), "a rejected call must not touch dst"
    # the limit itself is served
    rc = L.cuvdia_spmm_offsets_noalloc_f32(vals.data_ptr(), offs.ctypes.data_as(IP), 1024, n, n, n, 1,
                                           B.data_ptr(), n, out.data_ptr(), n, 32, b"n", 1.0, 0.0, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert bool((out == 0.0).all())


def test_noalloc_leaves_free_device_memory_unchanged(oracle):
    """Free device memory as the driver reports it is the same before and after a series of calls with
    tables of different sizes (the operands are allocated beforehand; the first call on the device, which
    resolves the static array, is made before the first reading)."""
    import torch
    from cuv_amd import _lib
    L = _lib.lib()
    n, batch = 2048, 64
    vals = torch.rand(64 * n, device="cuda:0")
    B = torch.rand(batch * n, device="cuda:0")
    out = torch.zeros(batch * n, device="cuda:0")

    def call(offs):
        offs = np.asarray(offs, np.int32)
        rc = L.cuvdia_spmm_offsets_noalloc_f32(vals.data_ptr(), offs.ctypes.data_as(IP), len(offs), n, n, n, 1,
                                               B.data_ptr(), n, out.data_ptr(), n, batch, b"n", 1.0, 0.0, None)
        assert rc == 0, L.cuvdia_strerror(rc)

    call([0, 1])
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for offs in (_window(32, 5), [-5, 0, 9], list(range(-30, 30)), [7 * i - 200 for i in range(64)]):
        call(offs)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, "free device memory changed by %d bytes" % (free0 - free1)


@pytest.mark.parametrize("trans", ["n", "t"])
def test_noalloc_under_graph_capture(oracle, trans):
    """A call recorded into a graph (after one eager call on the device) replays correctly: three replays with
    the dense operand rewritten and eager work between them, each against the allocating entry point run
    eagerly on the same operands."""
    import torch
    from cuv_amd import _lib, dia as D
    L = _lib.lib()
    rng = np.random.default_rng(977)
    h, w, batch = 1024, 1024, 64
    A = _rand_dia(oracle, rng, h, w, _window(32, 5))
    n_in, n_out = (h, w) if trans == "t" else (w, h)
    vals = torch.from_numpy(A.vals).cuda()
    Bd = torch.empty(batch, n_in, device="cuda:0")
    dst0 = torch.from_numpy(rng.uniform(-1, 1, (batch, n_out)).astype(np.float32)).cuda()
    out = torch.empty(batch, n_out, device="cuda:0")
    ref = torch.empty(batch, n_out, device="cuda:0")
    offs = A.offsets

    def run(fn, dst, stream):
        rc = fn(vals.data_ptr(), offs.ctypes.data_as(IP), A.nd, A.stride, h, w, 1, Bd.data_ptr(), n_in,
                dst.data_ptr(), n_out, batch, trans.encode(), 0.75, 0.5, stream)
        assert rc == 0, L.cuvdia_strerror(rc)

    Bd.copy_(torch.from_numpy(rng.uniform(-1, 1, (batch, n_in)).astype(np.float32)))
    out.copy_(dst0)
    run(L.cuvdia_spmm_offsets_noalloc_f32, out, None)          # the first call on the device: outside capture
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph.capture_begin()
        run(L.cuvdia_spmm_offsets_noalloc_f32, out, ctypes.c_void_p(side.cuda_stream))
        graph.capture_end()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    for replay in range(3):
        Bd.copy_(torch.from_numpy(rng.uniform(-1, 1, (batch, n_in)).astype(np.float32)))
        out.copy_(dst0)
        ref.copy_(dst0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        run(L.cuvdia_spmm_offsets_f32, ref, None)
        torch.cuda.synchronize()
        assert torch.equal(out, ref), "replay %d differs from the eager result" % replay
        assert float(out.abs().sum()) > 0
    assert L.cuvdia_cache_clear() == 0
