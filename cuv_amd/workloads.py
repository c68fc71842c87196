"""Seeded synthetic inputs for the five measured DIA workloads.

Each workload is a diagonal pattern plus host-side numpy operands; the same
generator feeds the parity tests, the smoke check and the benchmark, so a
timed result and its check always see identical bytes.

  cfg0  4096x4096, 33 diagonals -16..16, values U[-1,1]; x in R^4096
  cfg1  128x128 map, 7x7 window (49 diagonals dy*128+dx), values N(0,0.01);
        V 16384x128 Bernoulli(0.5); H = A*V
  cfg2  same A; H = sigmoid(N(0,1)); V' = 0.5*V' + A^T*H, V' prefilled U[0,1]
  cfg3  A Bernoulli(0.5), B sigmoid(N(0,1)), both 16384x128;
        dst = 0.9*dst + (1/128)*proj_diag(A*B^T)
  cfg4  256x256 map x 4 channels, 13x13 window per channel shift
        (676 diagonals c*65536+dy*256+dx), batch 256, operands U[0,1]

Work per call (fp32, each operand touched once, only valid diagonal slots):
  bytes_spmm   = 4*(nnz + n_in*b + n_out*b*(1 + [beta != 0])) + 4*nd
  bytes_dd2dia = 4*(n_out*b + n_in*b + nnz*(1 + [beta != 0])) + 4*nd
  flops        = 2*nnz*b
"""
from dataclasses import dataclass, field

import numpy as np

SEED0 = 0xC0FFEE


@dataclass
class Pattern:
    """A diagonal pattern: shape, offset table (in table order), padding."""
    h: int
    w: int
    offsets: np.ndarray
    stride: int
    rf: int = 1

    @property
    def nd(self):
        return int(self.offsets.size)

    def valid_counts(self):
        k = self.offsets.astype(np.int64)
        i0 = self.rf * np.maximum(0, -k)
        j0 = np.maximum(0, k)
        return np.maximum(0, np.minimum(self.h - i0, self.rf * (self.w - j0)))

    @property
    def nnz(self):
        return int(self.valid_counts().sum())

    def valid_mask(self):
        m = np.zeros((self.nd, self.stride), bool)
        k = self.offsets.astype(np.int64)
        i0 = self.rf * np.maximum(0, -k)
        n = self.valid_counts()
        for d in range(self.nd):
            if n[d] > 0:
                m[d, i0[d]:i0[d] + n[d]] = True
        return m.reshape(-1)


def window_offsets(px, fs, channels=1, map_elems=None):
    """Offsets c*map + dy*px + dx for dy, dx in [-(fs//2), fs//2], channel-major
    then dy-major: the pattern a locally connected layer with an fs x fs window
    on a px-wide map produces."""
    r = fs // 2
    map_elems = px * px if map_elems is None else map_elems
    offs = [c * map_elems + dy * px + dx
            for c in range(channels)
            for dy in range(-r, r + 1)
            for dx in range(-r, r + 1)]
    return np.asarray(offs, np.int32)


def spmm_bytes(p, batch, trans, beta):
    n_out, n_in = (p.w, p.h) if trans == "t" else (p.h, p.w)
    return 4 * (p.nnz + n_in * batch + n_out * batch * (2 if beta != 0 else 1)) + 4 * p.nd


def dd2dia_bytes(p, batch, beta):
    return 4 * (p.h * batch + p.w * batch + p.nnz * (2 if beta != 0 else 1)) + 4 * p.nd


def flops(p, batch):
    return 2 * p.nnz * batch


def _sigmoid32(x):
    x = x.astype(np.float32)
    return (np.float32(1) / (np.float32(1) + np.exp(-x))).astype(np.float32)


def _colmajor(a):
    return np.asfortranarray(a.astype(np.float32, copy=False))


def _rng(idx):
    return np.random.Generator(np.random.MT19937(SEED0 + idx))


@dataclass
class Workload:
    name: str
    op: str                 # "spmm" or "dd2dia"
    pattern: Pattern
    batch: int
    trans: str = "n"
    alpha: float = 1.0
    beta: float = 0.0
    vals: np.ndarray = None        # nd*stride fp32 (spmm: A; dd2dia: dst)
    X: np.ndarray = None           # spmm: dense input (n_in x b)
    dst: np.ndarray = None         # spmm: prefilled destination (n_out x b) or None
    A: np.ndarray = None           # dd2dia: left dense operand (h x b)
    B: np.ndarray = None           # dd2dia: right dense operand (w x b)
    extra: dict = field(default_factory=dict)

    @property
    def bytes(self):
        if self.op == "spmm":
            return spmm_bytes(self.pattern, self.batch, self.trans, self.beta)
        return dd2dia_bytes(self.pattern, self.batch, self.beta)

    @property
    def flops(self):
        return flops(self.pattern, self.batch)


def pattern_cfg0():
    return Pattern(4096, 4096, np.arange(-16, 17, dtype=np.int32), 4096)


def pattern_lc7():
    return Pattern(16384, 16384, window_offsets(128, 7), 16384)


def pattern_large(px=256, channels=4, fs=13):
    n = px * px * channels
    return Pattern(n, n, window_offsets(px, fs, channels), n)


def _vals_normal(rng, p, std=0.01):
    return (rng.standard_normal(p.nd * p.stride, dtype=np.float32) * np.float32(std))


def cfg0(trans="n"):
    rng = _rng(0)
    p = pattern_cfg0()
    vals = rng.uniform(-1, 1, p.nd * p.stride).astype(np.float32)
    x = _colmajor(rng.uniform(-1, 1, (4096, 1)))
    return Workload("cfg0_spmv_%s" % trans, "spmm", p, 1, trans, 1.0, 0.0, vals=vals, X=x)


def cfg1():
    rng = _rng(1)
    p = pattern_lc7()
    vals = _vals_normal(rng, p)
    V = _colmajor((rng.random((p.w, 128)) < 0.5))
    return Workload("cfg1_up_pass", "spmm", p, 128, "n", 1.0, 0.0, vals=vals, X=V)


def cfg2():
    p = pattern_lc7()
    vals = _vals_normal(_rng(1), p)                 # the 49-diagonal A of cfg1
    rng = _rng(2)
    H = _colmajor(_sigmoid32(rng.standard_normal((p.h, 128), dtype=np.float32)))
    dst = _colmajor(rng.random((p.w, 128), dtype=np.float32))
    return Workload("cfg2_down_pass", "spmm", p, 128, "t", 1.0, 0.5, vals=vals, X=H, dst=dst)


def cfg3():
    p = pattern_lc7()
    vals = _vals_normal(_rng(1), p)                 # dst starts as cfg1's A
    rng = _rng(3)
    A = _colmajor((rng.random((p.h, 128)) < 0.5))
    B = _colmajor(_sigmoid32(rng.standard_normal((p.w, 128), dtype=np.float32)))
    return Workload("cfg3_weight_gradient", "dd2dia", p, 128, "n", 1.0 / 128, 0.9,
                    vals=vals, A=A, B=B)


def cfg4(op="spmm", trans="n", px=256, channels=4, fs=13, batch=256, beta=0.0):
    """The large layer.  px/channels/fs/batch can be reduced for CPU-sized
    variants that keep the multi-channel offset structure."""
    rng = _rng(4)
    p = pattern_large(px, channels, fs)
    vals = _vals_normal(rng, p)
    n = p.h
    if op == "spmm":
        X = _colmajor(rng.random((n, batch), dtype=np.float32))
        dst = _colmajor(rng.random((n, batch), dtype=np.float32)) if beta != 0 else None
        return Workload("cfg4_large_%s" % ("trans" if trans == "t" else "fwd"), "spmm", p,
                        batch, trans, 1.0, beta, vals=vals, X=X, dst=dst)
    A = _colmajor(rng.random((n, batch), dtype=np.float32))
    B = _colmajor(rng.random((n, batch), dtype=np.float32))
    return Workload("cfg4_large_dd2dia", "dd2dia", p, batch, "n", 1.0, beta,
                    vals=vals, A=A, B=B)


BENCH_WORKLOADS = {
    "cfg1": cfg1, "cfg2": cfg2, "cfg3": cfg3,
}
