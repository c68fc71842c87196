"""The projection on a batch whose operands exceed the 2 GiB that the tiled kernel's 32-bit byte offsets reach:
the library walks the batch in slabs of columns (first slab with the caller's beta, every later one adding to what
is there).  131072 rows (7x7 window on a 512x256 map), batch 4160: 2.18 GB per operand, slabs of 4064 and 96
columns.  Checked without a CPU pass over 50 GFLOP:
  * the call runs the tiled kernels (not the generic fallback);
  * the whole result against the same sum built from two calls on halves of the batch, each small enough for one
    launch, within 1e-5 of the summed term magnitudes (proj(|P| |Q|^T), itself from the library);
  * sampled slots against an fp64 evaluation of the defining sum on the device;
  * padding slots (NaN) are neither read nor written."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_projection_walks_a_batch_beyond_2_gib_in_slabs():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from cuv_amd import dia as D, _lib, workloads as W
    L = _lib.lib()
    dev = "cuda:0"
    px, py, batch = 512, 256, 4160
    n = px * py
    offs = [dy * px + dx for dy in range(-3, 4) for dx in range(-3, 4)]
    nd = len(offs)
    assert n * batch * 4 > 2 ** 31
    g = torch.Generator(device=dev)
    g.manual_seed(0xBA7C4)
    off = torch.tensor(np.asarray(offs, np.int64), device=dev)
    rows = torch.arange(n, device=dev)
    valid = ((rows[None, :] + off[:, None]) >= 0) & ((rows[None, :] + off[:, None]) < n)       # (nd, n)
    nan = torch.full((), float("nan"), device=dev)

    def new_dia(fill):
        m = D.dev_dia_matrix_f(n, n, nd, n, 1, device=dev)
        m.set_offsets(offs)
        m.vec.copy_(torch.where(valid, fill.view(nd, n), nan).view(-1))
        return m

    P = torch.rand(batch, n, generator=g, device=dev) * 2 - 1
    Q = torch.rand(batch, n, generator=g, device=dev) * 2 - 1
    c0 = torch.rand(nd * n, generator=g, device=dev)
    alpha, beta = 1.0 / batch, 0.75

    C = new_dia(c0)
    bd = D.dev_block_descriptor_f(C)
    D.densedense_to_dia(C, bd, P, Q, alpha, beta)
    assert L.cuvdia_last_path() in (_lib.PATH_TILED, _lib.PATH_WINDOW), "the large batch must not fall back to the generic kernel"
    got = C.vec.view(nd, n)
    assert bool(torch.isnan(got[~valid]).all()), "padding slots were written"
    assert bool(torch.isfinite(got[valid]).all()), "padding slots were read"

    # the same sum from two launches on halves of the batch
    half = 2080
    R = new_dia(c0)
    D.densedense_to_dia(R, bd, P[:half], Q[:half], alpha, beta)
    D.densedense_to_dia(R, bd, P[half:], Q[half:], alpha, 1.0)
    M = new_dia(c0.abs() * 0)
    D.densedense_to_dia(M, bd, P[:half].abs(), Q[:half].abs(), alpha, 0.0)
    D.densedense_to_dia(M, bd, P[half:].abs(), Q[half:].abs(), alpha, 1.0)
    mag = torch.nan_to_num(M.vec.view(nd, n)) + beta * c0.view(nd, n).abs()
    err = (torch.nan_to_num(got) - torch.nan_to_num(R.vec.view(nd, n))).abs()
    assert bool((err <= 2e-5 * mag + 1e-30).all()), "slabs vs halves: worst err/mag %.3g" % float((err / (mag + 1e-30)).max())

    # sampled slots in fp64: C[d, i] = beta * c0[d, i] + alpha * sum_c P[c, i] * Q[c, i + off_d]
    rng = np.random.default_rng(7)
    ds = torch.tensor(rng.integers(0, nd, 300), device=dev)
    is_ = torch.tensor(np.concatenate([rng.integers(0, n, 290), [0, 1, 2, 3, n - 4, n - 3, n - 2, n - 1, 1539, n - 1540]]),
                       device=dev)
    js = is_ + off[ds]
    ok = (js >= 0) & (js < n)
    ds, is_, js = ds[ok], is_[ok], js[ok]
    pv, qv = P[:, is_].double(), Q[:, js].double()
    ref = beta * c0.view(nd, n)[ds, is_].double() + alpha * (pv * qv).sum(0)
    m = beta * c0.view(nd, n)[ds, is_].double().abs() + alpha * (pv.abs() * qv.abs()).sum(0)
    e = (got[ds, is_].double() - ref).abs()
    assert bool((e <= 1e-5 * m + 1e-30).all()), "sampled slots: worst err/mag %.3g" % float((e / (m + 1e-30)).max())
