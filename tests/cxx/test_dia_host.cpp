// CPU-only checks of the C++ mirror: containers, conversions, error behaviour
// and the product's host twins of the operations (cuv/matrix_ops/host_ops.hpp)
// against the reference fixtures' closed forms and, element for element,
// against the oracle (namespace cuv_oracle).  Runs without a GPU.
//
// Re-expresses the host-side cases of the reference's tests:
//   src/tests/dia_mat.cpp:111-119 (dia -> dense), src/tests/convert.cpp:110-129,
//   src/tests/spmv.cpp:130-143 (host DIA product vs dense product),
//   src/tests/densedense_to_dia.cpp:139-164 (host dd2dia vs dense product, rf 4).
#include <cuv.hpp>
#include <cuv_host_ops.hpp>

#include "check.hpp"

using namespace cuv;

TEST_CASE(tensor_basics)
{
    tensor<float, host_memory_space, column_major> a(extents[4][3]);
    sequence(a);
    CHECK(a.ndim() == 2 && a.shape()[0] == 4 && a.shape()[1] == 3 && a.size() == 12);
    CHECK((float)a(1, 2) == 9.f);              // column-major: 2*4 + 1
    tensor<float, host_memory_space, row_major> r(extents[4][3]);
    sequence(r);
    CHECK((float)r(1, 2) == 5.f);
    tensor<float, host_memory_space, column_major> b = a;      // shares memory
    b(0, 0) = 42.f;
    CHECK((float)a(0, 0) == 42.f);
    tensor<float, host_memory_space> v(indices[index_range(0, 4)], a.ptr() + 4);   // view of column 1
    CHECK(v.size() == 4 && (float)v[2] == 6.f);
    fill(a, -1);
    CHECK((float)a(3, 2) == -1.f);
    a.dealloc();
    CHECK(a.ptr() == NULL);
}

TEST_CASE(dia_container)
{
    dia_matrix<float, host_memory_space> w(32, 16, 3, 32, 1);
    std::vector<int> off;
    off.push_back(0); off.push_back(1); off.push_back(-1);
    w.set_offsets(off);
    sequence(w.vec());
    CHECK(w.h() == 32 && w.w() == 16 && w.num_dia() == 3 && w.stride() == 32 && w.row_fact() == 1);
    CHECK(w.get_offset(2) == -1);
    CHECK(w.has(5, 6) && w.has(5, 4) && !w.has(5, 7));
    CHECK(w(5, 5) == 5.f && w(5, 6) == 32.f + 5 && w(5, 4) == 64.f + 5 && w(5, 8) == 0.f);
    w.set(5, 6, -3.f);
    CHECK(w(5, 6) == -3.f);
    w.set(5, 9, 1.f);                           // off the pattern: ignored
    CHECK(w(5, 9) == 0.f);
    // assignment takes the value vector away from its source
    dia_matrix<float, host_memory_space> w2;
    w2 = w;
    CHECK(w.vec_ptr() == NULL && w2.vec_ptr() != NULL && w2(5, 6) == -3.f);
    // constructor preconditions
    CHECK_THROWS((dia_matrix<float, host_memory_space>(32, 16, 3, 8, 1)));
    CHECK_THROWS((dia_matrix<float, host_memory_space>(32, 16, 3, 32, 0)));
}

TEST_CASE(dia2dense)
{
    for (int wdt = 16; wdt <= 32; wdt += 16) {
        dia_matrix<float, host_memory_space> w(32, wdt, 3, 32, 1);
        std::vector<int> off;
        off.push_back(0); off.push_back(1); off.push_back(-1);
        w.set_offsets(off);
        sequence(w.vec());
        tensor<float, host_memory_space, column_major> w2(extents[32][wdt]);
        fill(w2, -1);
        convert(w2, w);
        MAT_CMP(w, w2, 0.1f);
        for (int i = 0; i < 32; i++)
            for (int j = 0; j < wdt; j++) {
                const int d = j - i;
                const float exp = d == 0 ? i : d == 1 ? 32 + i : d == -1 ? 64 + i : 0;
                CHECK((float)w2(i, j) == exp);
            }
    }
}

struct SpmvFix {
    static const int n = 32, m = 16, k = 6;
    dia_matrix<float, host_memory_space> A;
    tensor<float, host_memory_space, column_major> A_, B, B_, C, C_;
    SpmvFix() : A(n, m, 7, 32, 1), A_(n, m), B(m, k), B_(m, k), C(n, k), C_(n, k)
    {
        std::vector<int> off;
        for (int i = -3; i <= 3; i++) off.push_back(i);
        A.set_offsets(off);
        sequence(A.vec()); sequence(C); sequence(C_); sequence(B); sequence(B_);
        convert(A_, A);
    }
};

TEST_CASE(spmv_host_correctness)
{
    SpmvFix f;
    prod(f.C, f.A, f.B, 'n', 'n', 2.f, 1.3f);
    cuv_oracle::prod(f.C_, f.A_, f.B, 'n', 'n', 2.f, 1.3f);
    MAT_CMP(f.C, f.C_, 0.1f);
}

TEST_CASE(spmv_host_correctness_trans)
{
    SpmvFix f;
    prod(f.B, f.A, f.C, 't', 'n', 2.f, 1.3f);
    cuv_oracle::prod(f.B_, f.A_, f.C, 't', 'n', 2.f, 1.3f);
    MAT_CMP(f.B, f.B_, 0.5f);
}

TEST_CASE(spmv_host_closed_form)
{
    SpmvFix f;
    tensor<float, host_memory_space, column_major> out(SpmvFix::n, SpmvFix::k);
    fill(out, 0);
    prod(out, f.A, f.B);
    for (int i = 0; i < SpmvFix::n; i++)
        for (int c = 0; c < SpmvFix::k; c++) {
            long s = 0;
            for (int d = 0; d < 7; d++) {
                const int j = i + d - 3;
                if (j >= 0 && j < SpmvFix::m) s += (long)(32 * d + i) * (16 * c + j);
            }
            CHECK((float)out(i, c) == (float)s);
        }
}

TEST_CASE(dd2s_correctness_host)
{
    const int n = 36, m = 19, k = 16, rf = 4;
    dia_matrix<float, host_memory_space> C(n, m, 7, 36, rf);
    std::vector<int> off;
    for (int i = -3; i <= 3; i++) off.push_back(i);
    C.set_offsets(off);
    fill(C.vec(), 0);
    tensor<float, host_memory_space, column_major> A(n, k), B(m, k), dense(n, m);
    sequence(A); sequence(B);
    host_block_descriptor<float> bdh(C);
    densedense_to_dia(C, bdh, A, B);
    fill(dense, 0);
    cuv_oracle::prod(dense, A, B, 'n', 't');
    int seen = 0;
    for (int i = 0; i < n; i++)
        for (int j = 0; j < m; j++)
            if (C(i, j) != 0) {
                CHECK(close_pct(C(i, j), (float)dense(i, j), 0.01f));
                ++seen;
            }
    CHECK(seen > 200);
    // the literal host loop gives the same on a zeroed destination
    dia_matrix<float, host_memory_space> C2(n, m, 7, 36, rf);
    C2.set_offsets(off);
    fill(C2.vec(), 0);
    cuv_oracle::densedense_to_dia_literal(C2, A, B);
    MAT_CMP(C, C2, 0.0001f);
}

// The product's host twins against the oracle on the same pseudo-random operands: both restate the
// reference's host loops in the reference's element order, so every element must agree exactly -- for
// steep matrices, both transposes, factors that are not the defaults, unsorted and out-of-range offsets.
TEST_CASE(host_twins_equal_the_oracle)
{
    unsigned state = 12345u;
    auto rnd = [&]() { state = state * 1664525u + 1013904223u; return (float)((state >> 8) & 0xffff) / 32768.f - 1.f; };
    const int shapes[4][3] = {{40, 40, 1}, {36, 19, 4}, {24, 50, 2}, {130, 64, 1}};
    for (const auto &sh : shapes) {
        const int h = sh[0], w = sh[1], rf = sh[2], batch = 5;
        std::vector<int> off;
        const int cand[9] = {3, -2, 0, 1, -7, w - 1, -(h / rf) + 1, w + 5, -h - 3};
        for (int o : cand) off.push_back(o);
        dia_matrix<float, host_memory_space> A(h, w, (int)off.size(), std::max(h, w), rf), C1(h, w, (int)off.size(), std::max(h, w), rf),
            C2(h, w, (int)off.size(), std::max(h, w), rf);
        A.set_offsets(off); C1.set_offsets(off); C2.set_offsets(off);
        for (unsigned i = 0; i < A.vec().size(); i++) { A.vec()[i] = rnd(); C1.vec()[i] = C2.vec()[i] = rnd(); }
        for (int t = 0; t < 2; t++) {
            const char trans = t ? 't' : 'n';
            const int n_in = t ? h : w, n_out = t ? w : h;
            tensor<float, host_memory_space, column_major> B(n_in, batch), D1(n_out, batch), D2(n_out, batch);
            for (int i = 0; i < n_in * batch; i++) B[i] = rnd();
            for (int i = 0; i < n_out * batch; i++) D1[i] = D2[i] = rnd();
            prod(D1, A, B, trans, 'n', 0.75f, -1.5f);
            cuv_oracle::prod(D2, A, B, trans, 'n', 0.75f, -1.5f);
            for (int i = 0; i < n_out * batch; i++) CHECK((float)D1[i] == (float)D2[i]);
            prod(D1, A, B, trans);                                   // factC == 0 overwrites
            cuv_oracle::prod(D2, A, B, trans);
            for (int i = 0; i < n_out * batch; i++) CHECK((float)D1[i] == (float)D2[i]);
            tensor<float, host_memory_space> x(indices[index_range(0, n_in)], B.ptr()), y1(n_out), y2(n_out);
            spmv(y1, A, x, trans, 2.f, 0.f);
            cuv_oracle::spmv(y2, A, x, trans, 2.f, 0.f);
            for (int i = 0; i < n_out; i++) CHECK((float)y1[i] == (float)y2[i]);
        }
        tensor<float, host_memory_space, column_major> P(h, batch), Q(w, batch);
        for (int i = 0; i < h * batch; i++) P[i] = rnd();
        for (int i = 0; i < w * batch; i++) Q[i] = rnd();
        host_block_descriptor<float> bd(C1);
        densedense_to_dia(C1, bd, P, Q, 0.25f, 0.9f);
        cuv_oracle::densedense_to_dia(C2, bd, P, Q, 0.25f, 0.9f);
        for (unsigned i = 0; i < C1.vec().size(); i++) CHECK((float)C1.vec()[i] == (float)C2.vec()[i]);
        if (rf == 1) {
            tensor<float, host_memory_space> m1((int)off.size()), m2((int)off.size());
            avg_diagonals(m1, A);
            cuv_oracle::avg_diagonals(m2, A);
            for (size_t d = 0; d < off.size(); d++) {
                const long long k = off[d], cnt = std::min<long long>(h - std::max(0LL, -k), w - std::max(0LL, k));
                if (cnt > 0) CHECK((float)m1[d] == (float)m2[d]);
                else CHECK((float)m1[d] == 0.f);
            }
        }
    }
}

TEST_CASE(host_preconditions_throw)
{
    SpmvFix f;
    CHECK_THROWS(prod(f.C, f.A, f.B, 'n', 't'));            // transB must be 'n'
    CHECK_THROWS(prod(f.C, f.A, f.C, 'n', 'n'));            // B has the wrong number of rows
    tensor<float, host_memory_space, column_major> narrow(SpmvFix::n, 2);
    CHECK_THROWS(prod(narrow, f.A, f.B));                   // batch mismatch
}

TEST_CASE(filter_factory_offsets)
{
    filter_factory<float, host_memory_space> ff(128, 128, 7, 1, 1);
    const std::vector<int> off = ff.offsets();
    CHECK(off.size() == 49);
    size_t q = 0;
    for (int dy = -3; dy <= 3; dy++)
        for (int dx = -3; dx <= 3; dx++) CHECK(off[q++] == dy * 128 + dx);
    filter_factory<float, host_memory_space> f2(8, 8, 3, 2, 3);
    dia_matrix<float, host_memory_space> *d = f2.get_dia();
    CHECK(d->h() == 128 && d->w() == 192 && d->num_dia() == 36 && d->stride() == 192);
    CHECK(d->get_offset(0) == -64 - 9 && d->get_offset(35) == 2 * 64 + 9);
    delete d;
}

TEST_CASE(filter_factory_extract_filter)
{
    // 6 x 6 map, 3 x 3 window, two input maps -> one output map: column 14 is map
    // position (2, 2), whose window lies fully inside both input maps
    filter_factory<float, host_memory_space> ff(6, 6, 3, 2, 1);
    dia_matrix<float, host_memory_space> *d = ff.get_dia();
    CHECK(d->h() == 72 && d->w() == 36 && d->num_dia() == 18);
    for (unsigned int i = 0; i < 72; i++)
        for (unsigned int j = 0; j < 36; j++) d->set(i, j, 1000.f * i + j);
    tensor<float, host_memory_space, row_major> *f = ff.extract_filter(*d, 14);
    CHECK(f->shape(0) == 9 && f->shape(1) == 2);
    for (unsigned int m = 0; m < 2; m++) {
        unsigned int k = 0;
        for (unsigned int i = m * 36; i < (m + 1) * 36; i++)
            if (d->has(i, 14)) {
                CHECK((float)(*f)[m * 9 + k] == 1000.f * i + 14);
                k++;
            }
        CHECK(k == 9);
    }
    delete f;
    delete d;
}

int main(int argc, char **argv) { return run_all(argc, argv); }
