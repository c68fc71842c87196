"""Writes the known-answer fixtures of tests/golden/.

The reference's DIA tests fill every operand with sequence() (0, 1, 2, ... in
memory order), so each expectation is an exact integer closed form.  This
script evaluates those closed forms in Python integers -- it does not call the
oracle or any product code -- and stores inputs and expected outputs as JSON.

Fixtures and the reference test each one restates:
  spmv_fixture.json      src/tests/spmv.cpp:49-143
                         (32x16, offsets -3..3, stride 32, rf 1, batch 6)
  dd2dia_fixture.json    src/tests/densedense_to_dia.cpp:50-137
                         (36x19, offsets -3..3, stride 36, rf 4, batch 16)
  dia_dense_fixture.json src/tests/dia_mat.cpp:48-119 (32x16) and
                         src/tests/convert.cpp:110-129 (32x32), offsets {0,1,-1}

Run:  python tests/golden/make_fixtures.py
"""
import json
import os
from fractions import Fraction

HERE = os.path.dirname(os.path.abspath(__file__))


def spmv_fixture():
    n, m, k, nd, stride = 32, 16, 6, 7, 32
    offs = list(range(-(nd // 2), nd // 2 + 1))
    a = lambda d, i: stride * d + i          # sequence(A.vec())
    B = lambda r, c: m * c + r               # sequence(B), column-major m x k
    C = lambda r, c: n * c + r               # sequence(C), column-major n x k
    # y = A*B, exact integers
    AB = [[sum(a(d, i) * B(i + off, c) for d, off in enumerate(offs)
               if 0 <= i + off < m) for c in range(k)] for i in range(n)]
    # y = A'*C, exact integers
    AtC = [[sum(a(d, j - off) * C(j - off, c) for d, off in enumerate(offs)
                if 0 <= j - off < n) for c in range(k)] for j in range(m)]
    # factAv=2, factC=1.3f on top of the sequence()-filled destination
    # (spmv.cpp:116-143); 1.3f is the fp32 value, the rest exact rationals
    f13 = Fraction(10905190, 8388608)        # float32(1.3) = 0x3FA66666
    n_scaled = [[float(f13 * C(i, c) + 2 * AB[i][c]) for c in range(k)] for i in range(n)]
    t_scaled = [[float(f13 * B(j, c) + 2 * AtC[j][c]) for c in range(k)] for j in range(m)]
    return dict(h=n, w=m, batch=k, nd=nd, stride=stride, rf=1, offsets=offs,
                note="vals[d*stride+i]=stride*d+i; B(r,c)=w*c+r; C(r,c)=h*c+r",
                AB=AB, AtC=AtC, n_alpha2_beta1p3=n_scaled, t_alpha2_beta1p3=t_scaled)


def dd2dia_fixture():
    n, m, k, nd, stride, rf = 36, 19, 16, 7, 36, 4
    offs = list(range(-(nd // 2), nd // 2 + 1))
    A = lambda i, c: n * c + i
    B = lambda j, c: m * c + j
    # expected[d][i] for valid slots, None for padding
    exp = []
    for off in offs:
        row = []
        for i in range(stride):
            j = off + i // rf
            ok = i < n and 0 <= j < m
            row.append(sum(A(i, c) * B(j, c) for c in range(k)) if ok else None)
        exp.append(row)
    return dict(h=n, w=m, batch=k, nd=nd, stride=stride, rf=rf, offsets=offs,
                note="A(i,c)=h*c+i; B(j,c)=w*c+j; C.vec() starts at 0", expected=exp)


def dia_dense_fixture():
    out = []
    for (h, w) in ((32, 16), (32, 32)):
        stride, offs = 32, [0, 1, -1]
        dense = [[0] * w for _ in range(h)]
        for d, off in enumerate(offs):
            for i in range(h):
                j = i + off
                if 0 <= j < w:
                    dense[i][j] = stride * d + i
        out.append(dict(h=h, w=w, nd=3, stride=stride, rf=1, offsets=offs,
                        note="vals[d*stride+i]=stride*d+i", dense=dense))
    return out


if __name__ == "__main__":
    for name, obj in (("spmv_fixture.json", spmv_fixture()),
                      ("dd2dia_fixture.json", dd2dia_fixture()),
                      ("dia_dense_fixture.json", dia_dense_fixture())):
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(obj, f, separators=(",", ":"))
        print("wrote", name)
