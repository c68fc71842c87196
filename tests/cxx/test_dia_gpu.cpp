// The reference's device-side DIA tests, re-expressed against the C++ mirror.
// Needs a GPU: every case runs the device path (the HIP kernels behind the
// C ABI) and compares with the host twin or a dense product.
//
//   src/tests/spmv.cpp:103-129            spmv_dev_correctness{,_trans}
//   src/tests/densedense_to_dia.cpp:109-197  dd2s_correctness_dev, dd2s_cmp_dev_host (row_fact 4)
//   src/tests/dia_mat.cpp:103-132         spmv_uninit, spmv_host2dev
#include <string>
#include <cuv.hpp>
#include <cuv_host_ops.hpp>

#include "check.hpp"

using namespace cuv;

static const int n = 32, m = 16, k = 6;

struct Fix {
    dia_matrix<float, host_memory_space> A;
    tensor<float, host_memory_space, column_major> B, C;
    Fix() : A(n, m, 7, 32, 1), B(m, k), C(n, k)
    {
        std::vector<int> off;
        for (int i = -3; i <= 3; i++) off.push_back(i);
        A.set_offsets(off);
        sequence(A.vec()); sequence(C); sequence(B);
    }
};

TEST_CASE(spmv_dev_correctness_trans)
{
    Fix f;
    dia_matrix<float, dev_memory_space> A2(n, m, f.A.num_dia(), f.A.stride(), 1);
    convert(A2, f.A);
    tensor<float, dev_memory_space, column_major> C2(f.C.shape());
    convert(C2, f.C);
    tensor<float, dev_memory_space, column_major> B2(f.B.shape());
    convert(B2, f.B);
    cuv_oracle::prod(f.B, f.A, f.C, 't', 'n');
    prod(B2, A2, C2, 't', 'n');
    MAT_CMP(f.B, B2, 0.1f);
}

TEST_CASE(spmv_dev_correctness)
{
    Fix f;
    dia_matrix<float, dev_memory_space> A2(n, m, f.A.num_dia(), f.A.stride(), 1);
    convert(A2, f.A);
    tensor<float, dev_memory_space, column_major> C2(f.C.shape());
    convert(C2, f.C);
    tensor<float, dev_memory_space, column_major> B2(f.B.shape());
    convert(B2, f.B);
    const float factAv = 2.f, factC = 1.3f;
    cuv_oracle::prod(f.C, f.A, f.B, 'n', 'n', factAv, factC);
    prod(C2, A2, B2, 'n', 'n', factAv, factC);
    MAT_CMP(f.C, C2, 0.1f);
}

TEST_CASE(spmv_dev_flat_vectors)
{
    // cuv::spmv on flat tensors holding several columns (spmv.cu:243-245)
    Fix f;
    dia_matrix<float, dev_memory_space> A2(n, m, f.A.num_dia(), f.A.stride(), 1);
    convert(A2, f.A);
    tensor<float, dev_memory_space> x(m * k), y(n * k);
    tensor<float, host_memory_space> xh(m * k), yh(n * k), yd(n * k);
    sequence(xh); fill(yh, 0);
    convert(x, xh);
    spmv(y, A2, x, 'n', 1.f, 0.f);
    convert(yd, y);
    for (int c = 0; c < k; c++) {
        tensor<float, host_memory_space> xv(indices[index_range(0, m)], xh.ptr() + c * m);
        tensor<float, host_memory_space> yv(indices[index_range(0, n)], yh.ptr() + c * n);
        cuv_oracle::spmv(yv, f.A, xv, 'n', 1.f, 0.f);
    }
    for (int i = 0; i < n * k; i++) CHECK((float)yd[i] == (float)yh[i]);
}

struct DdFix {
    static const int n = 36, m = 19, k = 16, rf = 4;
    dia_matrix<float, dev_memory_space> C;
    tensor<float, dev_memory_space, column_major> C_, A, B;
    DdFix() : C(n, m, 7, 36, rf), C_(n, m), A(n, k), B(m, k)
    {
        std::vector<int> off;
        for (int i = -3; i <= 3; i++) off.push_back(i);
        C.set_offsets(off);
        sequence(A); sequence(B);
        fill(C.vec(), 0);
    }
};

TEST_CASE(dd2s_correctness_dev)
{
    DdFix f;
    dev_block_descriptor<float> bd(f.C);
    densedense_to_dia(f.C, bd, f.A, f.B);
    tensor<float, host_memory_space, column_major> Ah(f.A.shape()), Bh(f.B.shape()), dense(DdFix::n, DdFix::m);
    convert(Ah, f.A); convert(Bh, f.B);
    fill(dense, 0);
    cuv_oracle::prod(dense, Ah, Bh, 'n', 't');
    int seen = 0;
    for (int i = 0; i < DdFix::n; i++)
        for (int j = 0; j < DdFix::m; j++)
            if (f.C(i, j) != 0) {
                CHECK(close_pct(f.C(i, j), (float)dense(i, j), 0.01f));
                ++seen;
            }
    CHECK(seen > 200);
}

TEST_CASE(dd2s_cmp_dev_host)
{
    DdFix f;
    dia_matrix<float, host_memory_space> C2(DdFix::n, DdFix::m, f.C.num_dia(), f.C.stride(), DdFix::rf);
    tensor<float, host_memory_space, column_major> A2(f.A.shape()), B2(f.B.shape());
    convert(C2, f.C); convert(A2, f.A); convert(B2, f.B);
    dev_block_descriptor<float> bd(f.C);
    host_block_descriptor<float> bdh(C2);
    densedense_to_dia(f.C, bd, f.A, f.B);
    cuv_oracle::densedense_to_dia(C2, bdh, A2, B2);
    MAT_CMP(f.C, C2, 0.01f);
    // documented factors, and the descriptor-free overload
    densedense_to_dia(f.C, f.A, f.B, 0.5f, 0.25f);
    cuv_oracle::densedense_to_dia(C2, bdh, A2, B2, 0.5f, 0.25f);
    MAT_CMP(f.C, C2, 0.01f);
}

// src/tests/dia_mat.cpp:130-140 sets this fixture up (the call itself is
// commented out there); sequence() data makes every mean a closed form.
TEST_CASE(avg_diagonals_dev)
{
    dia_matrix<float, host_memory_space> w(32, 16, 7, 32, 1);
    std::vector<int> off;
    for (int i = -3; i <= 3; ++i) off.push_back(i);
    w.set_offsets(off);
    sequence(w.vec());
    dia_matrix<float, dev_memory_space> wd(32, 16, 7, 32, 1);
    convert(wd, w);
    tensor<float, dev_memory_space> avg(7);
    tensor<float, host_memory_space> avg_h(7), avg_ref(7);
    avg_diagonals(avg, wd);
    cuv_oracle::avg_diagonals(avg_ref, w);
    convert(avg_h, avg);
    for (int d = 0; d < 7; ++d) {
        const int k = off[d], i0 = std::max(0, -k), j0 = std::max(0, k);
        const int n = std::min(32 - i0, 16 - j0);
        const float exact = 32.f * d + i0 + 0.5f * (n - 1);      // mean of 32 d + i, i = i0 .. i0 + n - 1
        CHECK(close_pct(avg_h[d], exact, 0.001f));
        CHECK(close_pct(avg_h[d], avg_ref[d], 0.001f));
    }
    dia_matrix<float, dev_memory_space> steep(36, 19, 7, 36, 4);
    steep.set_offsets(off);
    CHECK_THROWS(avg_diagonals(avg, steep));
    tensor<float, dev_memory_space> wrong(5);
    CHECK_THROWS(avg_diagonals(wrong, wd));
}

// The weight update of examples/rbm/base.py:71 on a DIA layer's value vector:
// with learnrate 0.5, decay 0.25 and sequence() data (W = i, dW = i) every
// product is exact: W' = -0.5 i + 0.875 i = 0.375 i.
TEST_CASE(learn_step_weight_decay_dev)
{
    dia_matrix<float, host_memory_space> w(32, 16, 7, 32, 1), dw(32, 16, 7, 32, 1);
    std::vector<int> off;
    for (int i = -3; i <= 3; ++i) off.push_back(i);
    w.set_offsets(off);
    dw.set_offsets(off);
    sequence(w.vec());
    sequence(dw.vec());
    dia_matrix<float, dev_memory_space> wd(32, 16, 7, 32, 1), dwd(32, 16, 7, 32, 1);
    convert(wd, w);
    convert(dwd, dw);
    learn_step_weight_decay(wd.vec(), dwd.vec(), 0.5f, 0.25f);
    cuv_oracle::learn_step_weight_decay(w.vec(), dw.vec(), 0.5f, 0.25f);
    dia_matrix<float, host_memory_space> back(32, 16, 7, 32, 1);
    convert(back, wd);
    for (unsigned i = 0; i < w.vec().size(); ++i) {
        CHECK(back.vec()[i] == 0.375f * i);
        CHECK(back.vec()[i] == w.vec()[i]);
    }
    tensor<float, dev_memory_space> shorter(5);
    CHECK_THROWS(learn_step_weight_decay(wd.vec(), shorter, 0.5f));
}

// With learnrate 0.5, momentum weight 0.5, decay 0.25 and W = 8 i, m = 4 i,
// dW = 0 every product is exact: m' = 2 i - 0.5*(2 i) = i, W' = 9 i.
TEST_CASE(learn_step_weight_decay_momentum_dev)
{
    const unsigned n = 1000;
    tensor<float, host_memory_space> w(n), m(n), dw(n);
    for (unsigned i = 0; i < n; ++i) {
        w[i] = 8.f * i;
        m[i] = 4.f * i;
        dw[i] = 0.f;
    }
    tensor<float, dev_memory_space> wd(n), md(n), dwd(n);
    convert(wd, w);
    convert(md, m);
    convert(dwd, dw);
    learn_step_weight_decay_momentum(wd, md, dwd, 0.5f, 0.5f, 0.25f);
    cuv_oracle::learn_step_weight_decay_momentum(w, m, dw, 0.5f, 0.5f, 0.25f);
    tensor<float, host_memory_space> wb(n), mb(n);
    convert(wb, wd);
    convert(mb, md);
    for (unsigned i = 0; i < n; ++i) {
        CHECK(wb[i] == 9.f * i);
        CHECK(mb[i] == 1.f * i);
        CHECK(wb[i] == w[i]);
        CHECK(mb[i] == m[i]);
    }
    tensor<float, dev_memory_space> shorter(5);
    CHECK_THROWS(learn_step_weight_decay_momentum(wd, shorter, dwd, 0.5f));
}

TEST_CASE(spmv_uninit)
{
    dia_matrix<float, host_memory_space> w(32, 16, 3, 32, 1);
    std::vector<int> off;
    off.push_back(0); off.push_back(1); off.push_back(-1);
    w.set_offsets(off);
    sequence(w.vec());
    dia_matrix<float, dev_memory_space> wdev(32, 16, 3, 16, 1);
    wdev.dealloc();
    convert(wdev, w);
    CHECK(wdev.vec_ptr() != NULL && wdev.stride() == 32);
    MAT_CMP(w, wdev, 0.1f);
}

TEST_CASE(spmv_host2dev)
{
    dia_matrix<float, host_memory_space> w(32, 16, 3, 32, 1);
    std::vector<int> off;
    off.push_back(0); off.push_back(1); off.push_back(-1);
    w.set_offsets(off);
    sequence(w.vec());
    dia_matrix<float, dev_memory_space> w2(32, 16, w.num_dia(), w.stride(), 1);
    convert(w2, w);
    MAT_CMP(w, w2, 0.1f);
    fill(w.vec(), 0);
    convert(w, w2);
    MAT_CMP(w, w2, 0.1f);
    CHECK(w(5, 6) == 32.f + 5);
}

TEST_CASE(dev_preconditions_throw)
{
    Fix f;
    dia_matrix<float, dev_memory_space> A2(n, m, f.A.num_dia(), f.A.stride(), 1);
    convert(A2, f.A);
    tensor<float, dev_memory_space, column_major> B2(f.B.shape()), C2(f.C.shape()), narrow(n, 2);
    CHECK_THROWS(prod(C2, A2, B2, 'n', 't'));       // transB == 'n'
    CHECK_THROWS(prod(C2, A2, B2, 'x', 'n'));       // transA is 'n' or 't'
    CHECK_THROWS(prod(C2, A2, C2, 'n', 'n'));       // rows of B
    CHECK_THROWS(prod(B2, A2, B2, 't', 'n'));       // transposed product needs h rows in B
    CHECK_THROWS(prod(narrow, A2, B2));             // batch mismatch
    DdFix d;
    tensor<float, dev_memory_space, column_major> wrongA(DdFix::n + 1, DdFix::k);
    dev_block_descriptor<float> bd(d.C);
    CHECK_THROWS(densedense_to_dia(d.C, bd, wrongA, d.B));
    // a descriptor built for another pattern is rejected
    dia_matrix<float, dev_memory_space> other(DdFix::n, DdFix::m, 7, 36, DdFix::rf);
    std::vector<int> off;
    for (int i = -2; i <= 4; i++) off.push_back(i);
    other.set_offsets(off);
    dev_block_descriptor<float> bd2(other);
    CHECK_THROWS(densedense_to_dia(d.C, bd2, d.A, d.B));
}

TEST_CASE(locally_connected_layer)
{
    // a filter_factory pattern driven through all three operations, device vs host
    filter_factory<float, host_memory_space> ff(16, 16, 5, 1, 1);
    dia_matrix<float, host_memory_space> *W = ff.get_dia();
    const int N = W->h(), batch = 40;
    for (int i = 0; i < (int)W->vec().size(); i++) W->vec()[i] = 0.01f * (float)((i * 37) % 101 + 1);   // positive: no cancellation under the percent tolerance
    tensor<float, host_memory_space, column_major> V(N, batch), H(N, batch), Hh(N, batch), Vh(N, batch);
    for (int i = 0; i < N * batch; i++) { V[i] = (float)((i * 13) % 7) / 7.f; H[i] = (float)((i * 29) % 11) / 11.f; }
    dia_matrix<float, dev_memory_space> Wd(N, N, W->num_dia(), W->stride(), 1);
    convert(Wd, *W);
    tensor<float, dev_memory_space, column_major> Vd(V.shape()), Hd(H.shape()), outd(N, batch);
    convert(Vd, V); convert(Hd, H);
    prod(outd, Wd, Vd, 'n', 'n');
    cuv_oracle::prod(Hh, *W, V, 'n', 'n');
    MAT_CMP(Hh, outd, 0.01f);
    prod(outd, Wd, Hd, 't', 'n');
    cuv_oracle::prod(Vh, *W, H, 't', 'n');
    MAT_CMP(Vh, outd, 0.01f);
    densedense_to_dia(Wd, Hd, Vd, 1.f / batch, 0.9f);
    host_block_descriptor<float> bdh(*W);
    cuv_oracle::densedense_to_dia(*W, bdh, H, V, 1.f / batch, 0.9f);
    MAT_CMP(*W, Wd, 0.01f);
    delete W;
}

TEST_CASE(locally_connected_layer_window_projection)
{
    // the same on a 64 x 128 map with a 7 x 7 window, the projection through its kernel tiled in the window's plane
    // (taken by itself from 192 tiles of 4 x 64 positions on; forced here on 32)
    filter_factory<float, host_memory_space> ff(64, 128, 7, 1, 1);
    dia_matrix<float, host_memory_space> *W = ff.get_dia();
    const int N = W->h(), batch = 32;
    for (int i = 0; i < (int)W->vec().size(); i++) W->vec()[i] = 0.01f * (float)((i * 37) % 101 + 1);
    tensor<float, host_memory_space, column_major> V(N, batch), H(N, batch);
    for (int i = 0; i < N * batch; i++) { V[i] = (float)((i * 13) % 7) / 7.f; H[i] = (float)((i * 29) % 11) / 11.f; }
    dia_matrix<float, dev_memory_space> Wd(N, N, W->num_dia(), W->stride(), 1);
    convert(Wd, *W);
    tensor<float, dev_memory_space, column_major> Vd(V.shape()), Hd(H.shape());
    convert(Vd, V); convert(Hd, H);
    CHECK(cuvdia_set_path(CUVDIA_PATH_WINDOW) == CUVDIA_OK);
    densedense_to_dia(Wd, Hd, Vd, 1.f / batch, 0.9f);
    const int ran = cuvdia_last_path();
    CHECK(cuvdia_set_path(CUVDIA_PATH_AUTO) == CUVDIA_OK);
    CHECK(ran == CUVDIA_PATH_WINDOW);
    host_block_descriptor<float> bdh(*W);
    cuv_oracle::densedense_to_dia(*W, bdh, H, V, 1.f / batch, 0.9f);
    MAT_CMP(*W, Wd, 0.01f);
    delete W;
}

TEST_CASE(locally_connected_layer_wide_window_projection)
{
    // a 13 x 13 window on a 64 x 64 map: window rows of 13 diagonals, the kernel with a wave per window row
    filter_factory<float, host_memory_space> ff(64, 64, 13, 1, 1);
    dia_matrix<float, host_memory_space> *W = ff.get_dia();
    const int N = W->h(), batch = 12;
    for (int i = 0; i < (int)W->vec().size(); i++) W->vec()[i] = 0.01f * (float)((i * 37) % 101 + 1);
    tensor<float, host_memory_space, column_major> V(N, batch), H(N, batch);
    for (int i = 0; i < N * batch; i++) { V[i] = (float)((i * 13) % 7) / 7.f; H[i] = (float)((i * 29) % 11) / 11.f; }
    dia_matrix<float, dev_memory_space> Wd(N, N, W->num_dia(), W->stride(), 1);
    convert(Wd, *W);
    tensor<float, dev_memory_space, column_major> Vd(V.shape()), Hd(H.shape());
    convert(Vd, V); convert(Hd, H);
    CHECK(cuvdia_set_path(CUVDIA_PATH_WINDOW) == CUVDIA_OK);
    densedense_to_dia(Wd, Hd, Vd, 1.f / batch, 0.9f);
    const int ran = cuvdia_last_path();
    const std::string kernel = cuvdia_last_kernel();
    CHECK(cuvdia_set_path(CUVDIA_PATH_AUTO) == CUVDIA_OK);
    CHECK(ran == CUVDIA_PATH_WINDOW);
    CHECK(kernel.rfind("dd2dia_window_long_kernel<13,", 0) == 0);
    host_block_descriptor<float> bdh(*W);
    cuv_oracle::densedense_to_dia(*W, bdh, H, V, 1.f / batch, 0.9f);
    MAT_CMP(*W, Wd, 0.01f);
    delete W;
}

int main(int argc, char **argv)
{
    initCUDA(CUDA_TEST_DEVICE);
    const int rc = run_all(argc, argv);
    exitCUDA();
    return rc;
}
