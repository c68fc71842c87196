// C ABI of libcuvdia (declared in include/cuvdia.h): argument validation,
// descriptors, the offsets-keyed descriptor cache and kernel-family selection.
#include "cuvdia.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <list>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "kernels.hpp"
#include "plan.hpp"

using namespace cuvdia;

struct cuvdia_desc {
    int h, w, nd, stride, rf;
    int device;
    std::vector<int> offsets;        // host copy, table order
    long long nnz;
    int n_chunks_n, n_chunks_t;
    void *dev_block;                 // one allocation: offsets | chunks_n | chunks_t
    DiaView view;
};

namespace {

std::atomic_int g_path{CUVDIA_PATH_AUTO};
thread_local int t_last_path = 0;
thread_local char t_last_kernel[96] = "";
thread_local std::string t_hip_error;

// Batches narrower than this go to the generic kernel: the tiled SpMM puts
// one batch column on each of 64 lanes.
constexpr int SPMM_TILED_MIN_BATCH = 24;
// The rows-along-lanes kernel is the automatic choice from this many of its tiles (workgroups) and this batch.
// Largest h, w and |offset| the kernels' 32-bit row arithmetic allows.
constexpr long long DIM_LIMIT = 1LL << 30;

int hip_fail(hipError_t e, const char *what)
{
    t_hip_error = std::string(what) + ": " + hipGetErrorString(e);
    return CUVDIA_EHIP;
}

// A descriptor's tables live on the device that was current when it was
// created; launching with it from another device would hand the kernels
// pointers they cannot reach.
int check_device(const cuvdia_desc *desc)
{
    int device = -1;
    const hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return CUVDIA_ENODEVICE;
    }
    return device == desc->device ? CUVDIA_OK : CUVDIA_EINVAL;
}

// For the entry points that take no descriptor: a device must be there.
int require_device()
{
    int ndev = 0;
    const hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev < 1) {
        t_hip_error = std::string("hipGetDeviceCount: ") + hipGetErrorString(e);
        (void)hipGetLastError();
        return CUVDIA_ENODEVICE;
    }
    return CUVDIA_OK;
}

int validate_shape(const int *offsets, int nd, int h, int w, int stride, int rf)
{
    if (!offsets || nd < 1 || h < 1 || w < 1 || rf < 1 || stride < 1) return CUVDIA_EINVAL;
    // src/cuv/basics/dia_matrix.hpp:131
    if (!(stride >= h || stride >= w)) return CUVDIA_EINVAL;
    if (h > DIM_LIMIT || w > DIM_LIMIT) return CUVDIA_EUNSUPPORTED;
    // A diagonal is stored by row: its last valid row must fit in its own
    // stride, or it would alias the next diagonal's storage.
    for (int d = 0; d < nd; ++d) {
        const long long k = offsets[d];
        if (k >= DIM_LIMIT || k <= -DIM_LIMIT) return CUVDIA_EUNSUPPORTED;
        const long long i0 = (long long)rf * std::max<long long>(0, -k);
        const long long j0 = std::max<long long>(0, k);
        const long long n = std::min<long long>(h - i0, (long long)rf * (w - j0));
        if (n > 0 && i0 + n > stride) return CUVDIA_ESHAPE;
    }
    return CUVDIA_OK;
}

}  // namespace

namespace cuvdia {
void note_kernel(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_last_kernel, sizeof t_last_kernel, fmt, ap);
    va_end(ap);
}
}  // namespace cuvdia

extern "C" {

int cuvdia_abi_version(void) { return 1; }

const char *cuvdia_strerror(int code)
{
    switch (code) {
        case CUVDIA_OK: return "ok";
        case CUVDIA_EINVAL: return "invalid argument";
        case CUVDIA_ESHAPE: return "operand shapes do not match the matrix";
        case CUVDIA_EHIP: return "HIP runtime call failed";
        case CUVDIA_ENOMEM: return "out of memory";
        case CUVDIA_EUNSUPPORTED: return "unsupported request";
        case CUVDIA_ENODEVICE: return "no gfx950 device";
        case CUVDIA_ETOOLARGE: return "offset table exceeds the fixed capacity of the allocation-free entry point";
        default: return "unknown cuvdia error";
    }
}

const char *cuvdia_last_hip_error(void) { return t_hip_error.c_str(); }

int cuvdia_set_path(int path)
{
    if (path != CUVDIA_PATH_AUTO && path != CUVDIA_PATH_GENERIC && path != CUVDIA_PATH_TILED &&
        path != CUVDIA_PATH_TILED_NOWALK && path != CUVDIA_PATH_WALK && path != CUVDIA_PATH_WINDOW)
        return CUVDIA_EINVAL;
    g_path.store(path);
    return CUVDIA_OK;
}

int cuvdia_last_path(void) { return t_last_path; }
const char *cuvdia_last_kernel(void) { return t_last_kernel; }

int cuvdia_plan_chunks_max(const int *offsets_host, int nd, int transposed, int max_len,
                           int *s0, int *len, int *slot, int cap)
{
    if (!offsets_host || nd < 1 || max_len < 1 || max_len > SP_CHUNK_MAX) return CUVDIA_EINVAL;
    std::vector<Chunk> ch;
    try {
        ch = plan_chunks(offsets_host, nd, transposed != 0, max_len);
    } catch (const std::bad_alloc &) {
        return CUVDIA_ENOMEM;
    }
    const int n = (int)ch.size();
    if (n <= cap && s0 && len && slot) {
        for (int c = 0; c < n; ++c) {
            s0[c] = ch[c].s0;
            len[c] = ch[c].len;
            for (int j = 0; j < max_len; ++j) slot[c * max_len + j] = j < ch[c].len ? ch[c].slot[j] : -1;
        }
    }
    return n;
}

int cuvdia_plan_chunks(const int *offsets_host, int nd, int transposed,
                       int *s0, int *len, int *slot, int cap)
{
    return cuvdia_plan_chunks_max(offsets_host, nd, transposed, CHUNK_MAX, s0, len, slot, cap);
}

int cuvdia_plan_walk(const int *offsets_host, int nd, int stride, int transposed,
                     int *period, int *k, int *ngroups, int *lck)
{
    if (!offsets_host || nd < 1 || stride < 1) return CUVDIA_EINVAL;
    WalkPlan wp;
    try {
        plan_walk(plan_chunks(offsets_host, nd, transposed != 0, SP_CHUNK_MAX), stride, transposed != 0, wp);
    } catch (const std::bad_alloc &) {
        return CUVDIA_ENOMEM;
    }
    if (!wp.ok) return 0;
    if (period) *period = wp.period;
    if (k) *k = wp.k;
    if (ngroups) *ngroups = wp.ngroups;
    if (lck) *lck = wp.lck;
    const int rows = spmm_walk_tile_rows(wp.lck, wp.k, wp.s0);
    return rows > 0 && wp.period % rows == 0 ? 2 : 1;
}

long long cuvdia_plan_walk_launch(const int *offsets_host, int nd, int stride, int h, int w, int transposed,
                                  int batch)
{
    if (!offsets_host || nd < 1 || batch < 0) return CUVDIA_EINVAL;
    if (const int rc = validate_shape(offsets_host, nd, h, w, stride, 1)) return rc;
    const bool trans = transposed != 0;
    WalkPlan wp;
    DiaView view{};
    try {
        const std::vector<Chunk> chunks = plan_chunks(offsets_host, nd, trans, SP_CHUNK_MAX);
        plan_walk(chunks, stride, trans, wp);
        view.n_chunks_n = view.n_chunks_t = (int)chunks.size();
    } catch (const std::bad_alloc &) {
        return CUVDIA_ENOMEM;
    }
    if (!wp.ok) return 0;
    // the conditions of the automatic choice in cuvdia_spmm_layer_f32, for packed operands
    view.h = h; view.w = w; view.nd = nd; view.stride = stride; view.rf = 1;
    const long long n_out = trans ? w : h, n_in = trans ? h : w;
    if (batch < SPMM_TILED_MIN_BATCH || !spmm_tiled_ok(view, n_in, n_out, trans)) return 0;
    long long workgroups = 0;
    (void)spmm_walk_plan(wp.lck, wp.k, wp.s0, wp.period, n_out, n_in, ((long long)batch + 63) / 64, false, &workgroups);
    return workgroups;
}

long long cuvdia_plan_window_launch(const int *offsets_host, int nd, int stride, int h, int w, int batch)
{
    if (!offsets_host || nd < 1 || batch < 0) return CUVDIA_EINVAL;
    if (const int rc = validate_shape(offsets_host, nd, h, w, stride, 1)) return rc;
    WalkPlan wp;
    DiaView view{};
    try {
        const std::vector<Chunk> chunks = plan_chunks(offsets_host, nd, false, SP_CHUNK_MAX);
        plan_walk(chunks, stride, false, wp);
        const std::vector<Chunk> cp = plan_chunks(offsets_host, nd, false, CHUNK_MAX);
        view.max_len_p = 0;
        for (const Chunk &c : cp) view.max_len_p = std::max(view.max_len_p, c.len);
    } catch (const std::bad_alloc &) {
        return CUVDIA_ENOMEM;
    }
    if (!wp.ok || batch < 1) return 0;
    // the conditions of the automatic choice in cuvdia_dd2dia_f32, for packed operands
    static const int not_null = 0;          // the planner only asks whether the table is a window table
    bool rows4 = true;
    for (int r : wp.group_rows) rows4 = rows4 && r % 4 == 0;
    view.h = h; view.w = w; view.nd = nd; view.stride = stride; view.rf = 1;
    view.walk_n = WalkView{&not_null, wp.ngroups, wp.period, wp.s0, wp.k, wp.lck, wp.astep4, rows4};
    if (!dd2dia_tiled_ok(view, h, w, batch)) return 0;
    const long long workgroups = dd2dia_window_workgroups(view, batch);
    return workgroups > 0 && dd2dia_window_by_size(view, batch, workgroups) ? workgroups : 0;
}

int cuvdia_plan_units(const int *offsets_host, int nd, int *c1, int *c2, int cap)
{
    if (!offsets_host || nd < 1) return CUVDIA_EINVAL;
    std::vector<Unit> un;
    try {
        un = plan_units(plan_chunks(offsets_host, nd, false));
    } catch (const std::bad_alloc &) {
        return CUVDIA_ENOMEM;
    }
    const int n = (int)un.size();
    if (n <= cap && c1 && c2) {
        for (int u = 0; u < n; ++u) {
            c1[u] = un[u].c1;
            c2[u] = un[u].c2;
        }
    }
    return n;
}

int cuvdia_desc_create(cuvdia_desc **out, const int *offsets_host, int nd,
                       int h, int w, int stride, int row_fact)
{
    if (!out) return CUVDIA_EINVAL;
    *out = nullptr;
    const int rc = validate_shape(offsets_host, nd, h, w, stride, row_fact);
    if (rc) return rc;

    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev < 1) {
        t_hip_error = std::string("hipGetDeviceCount: ") + hipGetErrorString(e);
        (void)hipGetLastError();
        return CUVDIA_ENODEVICE;
    }

    cuvdia_desc *d = nullptr;
    std::vector<Chunk> cn, ct, cp;
    std::vector<Unit> un, us;
    try {
        d = new cuvdia_desc();
        d->offsets.assign(offsets_host, offsets_host + nd);
        cn = plan_chunks(offsets_host, nd, false, SP_CHUNK_MAX);
        ct = plan_chunks(offsets_host, nd, true, SP_CHUNK_MAX);
        cp = plan_chunks(offsets_host, nd, false, CHUNK_MAX);
        un = plan_units(cp);
        for (int c = 0; c < (int)cp.size(); ++c) us.push_back(Unit{c, -1});
    } catch (const std::bad_alloc &) {
        delete d;
        return CUVDIA_ENOMEM;
    }
    d->h = h; d->w = w; d->nd = nd; d->stride = stride; d->rf = row_fact;
    d->nnz = count_valid(offsets_host, nd, h, w, row_fact);
    d->n_chunks_n = (int)cn.size();
    d->n_chunks_t = (int)ct.size();
    d->dev_block = nullptr;
    if ((e = hipGetDevice(&d->device)) != hipSuccess) { delete d; return hip_fail(e, "hipGetDevice"); }

    // window-table forms of the products' tables (for the walking kernel)
    WalkPlan wn, wt;
    try {
        plan_walk(cn, stride, false, wn);
        plan_walk(ct, stride, true, wt);
    } catch (const std::bad_alloc &) {
        delete d;
        return CUVDIA_ENOMEM;
    }
    auto walk_ints = [](const WalkPlan &p) { return p.ok ? p.group_rows.size() + p.aoff4.size() : (size_t)0; };
    // one device block: offsets (padded to 64 B) | chunks_n | chunks_t | projection chunks | units | one unit per chunk
    // | window tables
    const size_t off_bytes = ((size_t)nd * sizeof(int) + 63) / 64 * 64;
    const size_t cn_bytes = cn.size() * sizeof(Chunk), ct_bytes = ct.size() * sizeof(Chunk);
    const size_t cp_bytes = cp.size() * sizeof(Chunk);
    const size_t un_bytes = un.size() * sizeof(Unit), us_bytes = us.size() * sizeof(Unit);
    const size_t cp_at = off_bytes + cn_bytes + ct_bytes, un_at = cp_at + cp_bytes, us_at = un_at + un_bytes;
    const size_t wn_at = (us_at + us_bytes + 63) / 64 * 64, wn_bytes = walk_ints(wn) * sizeof(int);
    const size_t wt_at = (wn_at + wn_bytes + 63) / 64 * 64, wt_bytes = walk_ints(wt) * sizeof(int);
    std::vector<unsigned char> staging(wt_at + wt_bytes + 64, 0);
    std::memcpy(staging.data(), offsets_host, (size_t)nd * sizeof(int));
    std::memcpy(staging.data() + off_bytes, cn.data(), cn_bytes);
    std::memcpy(staging.data() + off_bytes + cn_bytes, ct.data(), ct_bytes);
    std::memcpy(staging.data() + cp_at, cp.data(), cp_bytes);
    std::memcpy(staging.data() + un_at, un.data(), un_bytes);
    std::memcpy(staging.data() + us_at, us.data(), us_bytes);
    auto put_walk = [&](const WalkPlan &p, size_t at) {
        if (!p.ok) return;
        std::memcpy(staging.data() + at, p.group_rows.data(), p.group_rows.size() * sizeof(int));
        std::memcpy(staging.data() + at + p.group_rows.size() * sizeof(int), p.aoff4.data(), p.aoff4.size() * sizeof(int));
    };
    put_walk(wn, wn_at);
    put_walk(wt, wt_at);
    if ((e = hipMalloc(&d->dev_block, staging.size())) != hipSuccess) {
        delete d;
        return e == hipErrorOutOfMemory ? CUVDIA_ENOMEM : hip_fail(e, "hipMalloc(descriptor)");
    }
    if ((e = hipMemcpy(d->dev_block, staging.data(), staging.size(), hipMemcpyHostToDevice)) != hipSuccess) {
        (void)hipFree(d->dev_block);
        delete d;
        return hip_fail(e, "hipMemcpy(descriptor)");
    }
    unsigned char *base = static_cast<unsigned char *>(d->dev_block);
    d->view = DiaView{};
    d->view.h = h; d->view.w = w; d->view.nd = nd; d->view.stride = stride; d->view.rf = row_fact;
    d->view.offsets_dev = reinterpret_cast<const int *>(base);
    d->view.chunks_n_dev = reinterpret_cast<const Chunk *>(base + off_bytes);
    d->view.n_chunks_n = d->n_chunks_n;
    d->view.chunks_t_dev = reinterpret_cast<const Chunk *>(base + off_bytes + cn_bytes);
    d->view.n_chunks_t = d->n_chunks_t;
    d->view.chunks_p_dev = reinterpret_cast<const Chunk *>(base + cp_at);
    d->view.n_chunks_p = (int)cp.size();
    d->view.units_dev = reinterpret_cast<const Unit *>(base + un_at);
    d->view.n_units = (int)un.size();
    d->view.pair_delta_max = pair_delta_max(cp, un);
    d->view.single_units_dev = reinterpret_cast<const Unit *>(base + us_at);
    auto walk_view = [&](const WalkPlan &p, size_t at) {
        bool rows4 = true;
        for (int r : p.group_rows) rows4 = rows4 && r % 4 == 0;
        return p.ok ? WalkView{reinterpret_cast<const int *>(base + at), p.ngroups, p.period, p.s0, p.k, p.lck, p.astep4, rows4}
                    : WalkView{nullptr, 0, 0, 0, 0, 0, 0, false};
    };
    d->view.walk_n = walk_view(wn, wn_at);
    d->view.walk_t = walk_view(wt, wt_at);
    auto span = [](const std::vector<Chunk> &t, int &max_len, int &s_min, int &s_max, int *min_len = nullptr) {
        max_len = 0;
        if (min_len) {
            *min_len = t.empty() ? 0 : t.front().len;
            for (const Chunk &c : t) *min_len = std::min(*min_len, c.len);
        }
        s_min = t.empty() ? 0 : t.front().s0;
        s_max = s_min;
        for (const Chunk &c : t) {
            max_len = std::max(max_len, c.len);
            s_min = std::min(s_min, c.s0);
            s_max = std::max(s_max, c.s0);
        }
    };
    span(cn, d->view.max_len_n, d->view.s_min_n, d->view.s_max_n, &d->view.min_len_n);
    span(ct, d->view.max_len_t, d->view.s_min_t, d->view.s_max_t, &d->view.min_len_t);
    d->view.slot_step_n = common_slot_step(cn);
    d->view.slot_step_t = common_slot_step(ct);
    int unused_min = 0, unused_max = 0;
    span(cp, d->view.max_len_p, unused_min, unused_max);
    *out = d;
    return CUVDIA_OK;
}

int cuvdia_desc_destroy(cuvdia_desc *desc)
{
    if (!desc) return CUVDIA_OK;
    int rc = CUVDIA_OK;
    if (desc->dev_block) {
        const hipError_t e = hipFree(desc->dev_block);
        if (e != hipSuccess) rc = hip_fail(e, "hipFree(descriptor)");
    }
    delete desc;
    return rc;
}

int cuvdia_desc_info(const cuvdia_desc *desc, int *chunks_n, int *chunks_t, long long *nnz)
{
    if (!desc) return CUVDIA_EINVAL;
    if (chunks_n) *chunks_n = desc->n_chunks_n;
    if (chunks_t) *chunks_t = desc->n_chunks_t;
    if (nnz) *nnz = desc->nnz;
    return CUVDIA_OK;
}

int cuvdia_spmm_layer_f32(const cuvdia_desc *desc, const float *A_vals, const float *B, long long ldb,
                          float *dst, long long ldd, int batch, char transA,
                          float alpha, float beta, const float *bias, int act,
                          unsigned long long seed, void *stream)
{
    if (act != CUVDIA_ACT_NONE && act != CUVDIA_ACT_SIGMOID && act != CUVDIA_ACT_SIGMOID_SAMPLE) return CUVDIA_EINVAL;
    const SpEpilogue ep{bias, act, (unsigned)(seed & 0xffffffffull), (unsigned)(seed >> 32)};
    if (!desc || !A_vals || batch < 0) return CUVDIA_EINVAL;
    // make_spmv_header.pl:121-123: anything but 'n' / 't' is an error
    if (transA != 'n' && transA != 't') return CUVDIA_EINVAL;
    if (batch == 0) return CUVDIA_OK;
    if (!B || !dst) return CUVDIA_EINVAL;
    const bool trans = transA == 't';
    const int n_out = trans ? desc->w : desc->h;
    const int n_in = trans ? desc->h : desc->w;
    if (ldb < n_in || ldd < n_out) return CUVDIA_ESHAPE;
    if (const int rc = check_device(desc)) return rc;

    const int forced = g_path.load();
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool tiled_possible = spmm_tiled_ok(desc->view, ldb, ldd, trans);
    bool tiled;
    if (forced == CUVDIA_PATH_TILED || forced == CUVDIA_PATH_TILED_NOWALK || forced == CUVDIA_PATH_WALK ||
        forced == CUVDIA_PATH_WINDOW) {
        if (!tiled_possible) return CUVDIA_EUNSUPPORTED;
        tiled = true;
    } else if (forced == CUVDIA_PATH_GENERIC) {
        tiled = false;
    } else {
        tiled = tiled_possible && batch >= SPMM_TILED_MIN_BATCH;
    }
    bool walked = false;
    const int walk = forced == CUVDIA_PATH_WALK ? 1
                     : (forced == CUVDIA_PATH_TILED_NOWALK || forced == CUVDIA_PATH_WINDOW) ? -1 : 0;
    const hipError_t e = tiled
        ? launch_spmm_tiled(desc->view, A_vals, B, ldb, dst, ldd, batch, trans, alpha, beta, ep, s, walk, &walked)
        : launch_spmm_generic(desc->view, A_vals, B, ldb, dst, ldd, batch, trans, alpha, beta, ep, s);
    if (tiled && walk > 0 && e == hipErrorNotSupported) {
        (void)hipGetLastError();
        return CUVDIA_EUNSUPPORTED;
    }
    t_last_path = !tiled ? CUVDIA_PATH_GENERIC : walked ? CUVDIA_PATH_WALK : CUVDIA_PATH_TILED;
    return e == hipSuccess ? CUVDIA_OK : hip_fail(e, "spmm kernel launch");
}

int cuvdia_spmm_bias_act_f32(const cuvdia_desc *desc, const float *A_vals, const float *B, long long ldb,
                             float *dst, long long ldd, int batch, char transA,
                             float alpha, float beta, const float *bias, int act, void *stream)
{
    if (act == CUVDIA_ACT_SIGMOID_SAMPLE) return CUVDIA_EINVAL;      // sampling takes a seed: cuvdia_spmm_layer_f32
    return cuvdia_spmm_layer_f32(desc, A_vals, B, ldb, dst, ldd, batch, transA, alpha, beta, bias, act, 0ull, stream);
}

int cuvdia_learn_step_weight_decay_f32(float *W, const float *dW, long long n, float learnrate, float decay,
                                       void *stream)
{
    if (n < 0) return CUVDIA_EINVAL;
    if (n == 0) return CUVDIA_OK;
    if (!W || !dW) return CUVDIA_EINVAL;             // src/cuv/tensor_ops/rprop.cu:342-343
    if (const int rc = require_device()) return rc;
    // src/cuv/tensor_ops/rprop.cu:345: alpha = -learnrate, beta = 1 - learnrate*decay, both in fp32
    const float alpha = -learnrate, beta = 1.f - learnrate * decay;
    const hipError_t e = launch_axpby(W, dW, n, alpha, beta, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? CUVDIA_OK : hip_fail(e, "learn_step_weight_decay kernel launch");
}

int cuvdia_learn_step_weight_decay_momentum_f32(float *W, float *momentum, const float *dW, long long n,
                                                float learnrate, float momentum_weight, float decay, void *stream)
{
    if (n < 0) return CUVDIA_EINVAL;
    if (n == 0) return CUVDIA_OK;
    if (!W || !momentum || !dW) return CUVDIA_EINVAL;    // src/cuv/tensor_ops/rprop.cu:377-381
    if (const int rc = require_device()) return rc;
    const hipError_t e = launch_momentum(W, momentum, dW, n, learnrate, momentum_weight, decay,
                                         static_cast<hipStream_t>(stream));
    return e == hipSuccess ? CUVDIA_OK : hip_fail(e, "learn_step_weight_decay_momentum kernel launch");
}

int cuvdia_spmm_f32(const cuvdia_desc *desc, const float *A_vals, const float *B, long long ldb,
                    float *dst, long long ldd, int batch, char transA,
                    float alpha, float beta, void *stream)
{
    return cuvdia_spmm_bias_act_f32(desc, A_vals, B, ldb, dst, ldd, batch, transA, alpha, beta, nullptr,
                                    CUVDIA_ACT_NONE, stream);
}

int cuvdia_dd2dia_f32(const cuvdia_desc *desc, float *C_vals, const float *A, long long lda,
                      const float *B, long long ldb, int batch,
                      float alpha, float beta, void *stream)
{
    if (!desc || !C_vals || batch < 0) return CUVDIA_EINVAL;
    if (batch > 0 && (!A || !B)) return CUVDIA_EINVAL;
    if (batch > 0 && (lda < desc->h || ldb < desc->w)) return CUVDIA_ESHAPE;
    if (const int rc = check_device(desc)) return rc;

    const int forced = g_path.load();
    // The tiled kernel addresses its operands with 32-bit byte offsets.  A batch whose operands are larger is
    // walked in slabs of columns that fit: the sum over the batch is the sum of the slabs' sums, so the first slab
    // runs with the caller's beta and every later one adds to what is there (beta = 1), one launch after the other
    // on the caller's stream.
    int slab = batch;
    bool tiled_possible = dd2dia_tiled_ok(desc->view, lda, ldb, batch);
    if (!tiled_possible && batch > DD2DIA_SLAB_MIN) {
        const int fit = dd2dia_slab_columns(desc->view, lda, ldb);
        if (fit >= DD2DIA_SLAB_MIN && dd2dia_tiled_ok(desc->view, lda, ldb, fit)) {
            // slabs of about equal width rather than full ones and a sliver
            const int count = (batch + fit - 1) / fit;
            const int even = ((batch + count - 1) / count + DD2DIA_SLAB_MIN - 1) / DD2DIA_SLAB_MIN * DD2DIA_SLAB_MIN;
            slab = std::min(fit, even);
            tiled_possible = true;
        }
    }
    bool tiled;
    if (forced == CUVDIA_PATH_TILED || forced == CUVDIA_PATH_TILED_NOWALK || forced == CUVDIA_PATH_WALK ||
        forced == CUVDIA_PATH_WINDOW) {
        if (!tiled_possible) return CUVDIA_EUNSUPPORTED;
        tiled = true;
    } else if (forced == CUVDIA_PATH_GENERIC) {
        tiled = false;
    } else {
        tiled = tiled_possible;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipSuccess;
    bool windowed = false;
    if (!tiled) {
        e = launch_dd2dia_generic(desc->view, C_vals, A, lda, B, ldb, batch, alpha, beta, s);
    } else {
        const int window = forced == CUVDIA_PATH_WINDOW ? 1
                           : (forced == CUVDIA_PATH_TILED_NOWALK || forced == CUVDIA_PATH_WALK) ? -1 : 0;
        for (int c0 = 0; c0 < batch && e == hipSuccess; c0 += slab) {
            bool this_one = false;
            e = launch_dd2dia_tiled(desc->view, C_vals, A + (long long)c0 * lda, lda, B + (long long)c0 * ldb, ldb,
                                    std::min(slab, batch - c0), alpha, c0 == 0 ? beta : 1.f, s, window, &this_one);
            windowed = windowed || this_one;
        }
        if (window > 0 && e == hipErrorNotSupported) {
            (void)hipGetLastError();
            return CUVDIA_EUNSUPPORTED;
        }
    }
    t_last_path = !tiled ? CUVDIA_PATH_GENERIC : windowed ? CUVDIA_PATH_WINDOW : CUVDIA_PATH_TILED;
    return e == hipSuccess ? CUVDIA_OK : hip_fail(e, "dd2dia kernel launch");
}

}  // extern "C"

// ------------------------------------------------------- descriptor cache ----
namespace {

struct CacheEntry {
    int h, w, stride, rf, device;
    std::vector<int> offsets;
    cuvdia_desc *desc;
};
std::mutex g_cache_mutex;
std::list<CacheEntry> g_cache;              // most recently used first
constexpr size_t CACHE_CAPACITY = 32;

// Caller holds g_cache_mutex, and keeps holding it until the launch that uses
// the descriptor has been enqueued: an eviction by another thread (which
// waits for the device before freeing) can then never pull a table from
// under a launch in progress.
int cached_desc(const int *offsets, int nd, int stride, int h, int w, int rf, cuvdia_desc **out)
{
    *out = nullptr;
    if (!offsets || nd < 1) return CUVDIA_EINVAL;
    int device = 0;
    const hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return CUVDIA_ENODEVICE;
    }
    for (auto it = g_cache.begin(); it != g_cache.end(); ++it) {
        if (it->h == h && it->w == w && it->stride == stride && it->rf == rf &&
            it->device == device && (int)it->offsets.size() == nd &&
            std::memcmp(it->offsets.data(), offsets, (size_t)nd * sizeof(int)) == 0) {
            g_cache.splice(g_cache.begin(), g_cache, it);
            *out = g_cache.front().desc;
            return CUVDIA_OK;
        }
    }
    cuvdia_desc *d = nullptr;
    const int rc = cuvdia_desc_create(&d, offsets, nd, h, w, stride, rf);
    if (rc) return rc;
    try {
        g_cache.push_front(CacheEntry{h, w, stride, rf, device, std::vector<int>(offsets, offsets + nd), d});
    } catch (const std::bad_alloc &) {
        cuvdia_desc_destroy(d);
        return CUVDIA_ENOMEM;
    }
    if (g_cache.size() > CACHE_CAPACITY) {
        // Work enqueued with the evicted table may still be running.
        (void)hipDeviceSynchronize();
        cuvdia_desc_destroy(g_cache.back().desc);
        g_cache.pop_back();
    }
    *out = d;
    return CUVDIA_OK;
}

}  // namespace

extern "C" {

int cuvdia_cache_clear(void)
{
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    if (!g_cache.empty()) (void)hipDeviceSynchronize();
    int rc = CUVDIA_OK;
    for (auto &e : g_cache) {
        const int r = cuvdia_desc_destroy(e.desc);
        if (r) rc = r;
    }
    g_cache.clear();
    return rc;
}

int cuvdia_avg_diagonals_f32(const cuvdia_desc *desc, const float *A_vals, float *dst, void *stream)
{
    if (!desc || !A_vals || !dst) return CUVDIA_EINVAL;
    if (desc->rf != 1) return CUVDIA_EUNSUPPORTED;      // src/cuv/matrix_ops/diagonals.cu:28
    if (const int rc = check_device(desc)) return rc;
    const hipError_t e = launch_avg_diagonals(desc->view, A_vals, dst, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? CUVDIA_OK : hip_fail(e, "avg_diagonals kernel launch");
}

int cuvdia_spmm_offsets_f32(const float *A_vals, const int *offsets_host, int nd, int stride,
                            int h, int w, int row_fact, const float *B, long long ldb,
                            float *dst, long long ldd, int batch, char transA,
                            float alpha, float beta, void *stream)
{
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    cuvdia_desc *d = nullptr;
    const int rc = cached_desc(offsets_host, nd, stride, h, w, row_fact, &d);
    if (rc) return rc;
    return cuvdia_spmm_f32(d, A_vals, B, ldb, dst, ldd, batch, transA, alpha, beta, stream);
}

int cuvdia_spmm_offsets_noalloc_f32(const float *A_vals, const int *offsets_host, int nd, int stride,
                                    int h, int w, int row_fact, const float *B, long long ldb,
                                    float *dst, long long ldd, int batch, char transA,
                                    float alpha, float beta, void *stream)
{
    // the argument rules of cuvdia_spmm_offsets_f32 -> cuvdia_spmm_layer_f32, in the same order
    if (!offsets_host || nd < 1) return CUVDIA_EINVAL;
    if (const int rc = validate_shape(offsets_host, nd, h, w, stride, row_fact)) return rc;
    if (!A_vals || batch < 0) return CUVDIA_EINVAL;
    if (transA != 'n' && transA != 't') return CUVDIA_EINVAL;
    if (batch == 0) return CUVDIA_OK;
    if (!B || !dst) return CUVDIA_EINVAL;
    const bool trans = transA == 't';
    const int n_out = trans ? w : h, n_in = trans ? h : w;
    if (ldb < n_in || ldd < n_out) return CUVDIA_ESHAPE;
    if (nd > NOALLOC_MAX_DIAGONALS) return CUVDIA_ETOOLARGE;
    if (const int rc = require_device()) return rc;

    std::vector<Chunk> chunks;
    try {
        chunks = plan_chunks(offsets_host, nd, trans, SP_CHUNK_MAX);
    } catch (const std::bad_alloc &) {
        return CUVDIA_ENOMEM;
    }
    unsigned char *tables = nullptr;
    hipError_t e = noalloc_scratch(&tables);
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(static table block)");

    // The view a descriptor would hold, with its tables inside the static array.  Only the table of the
    // requested traversal is described (and uploaded); the other one is left empty.
    DiaView view{};
    view.h = h; view.w = w; view.nd = nd; view.stride = stride; view.rf = row_fact;
    view.offsets_dev = reinterpret_cast<const int *>(tables);
    const Chunk *chunks_dev = reinterpret_cast<const Chunk *>(tables + NOALLOC_CHUNKS_AT);
    int max_len = 0, min_len = chunks.front().len, s_min = chunks.front().s0, s_max = s_min;
    for (const Chunk &c : chunks) {
        max_len = std::max(max_len, c.len);
        min_len = std::min(min_len, c.len);
        s_min = std::min(s_min, c.s0);
        s_max = std::max(s_max, c.s0);
    }
    if (trans) {
        view.chunks_t_dev = chunks_dev; view.n_chunks_t = (int)chunks.size();
        view.max_len_t = max_len; view.min_len_t = min_len; view.s_min_t = s_min; view.s_max_t = s_max;
        view.slot_step_t = common_slot_step(chunks);
    } else {
        view.chunks_n_dev = chunks_dev; view.n_chunks_n = (int)chunks.size();
        view.max_len_n = max_len; view.min_len_n = min_len; view.s_min_n = s_min; view.s_max_n = s_max;
        view.slot_step_n = common_slot_step(chunks);
    }

    // the kernel family is chosen by the rule of cuvdia_spmm_layer_f32
    const int forced = g_path.load();
    if (forced == CUVDIA_PATH_WALK) return CUVDIA_EUNSUPPORTED;
    const bool tiled_possible = spmm_tiled_ok(view, ldb, ldd, trans);
    bool tiled;
    if (forced == CUVDIA_PATH_TILED || forced == CUVDIA_PATH_TILED_NOWALK || forced == CUVDIA_PATH_WINDOW) {
        if (!tiled_possible) return CUVDIA_EUNSUPPORTED;
        tiled = true;
    } else if (forced == CUVDIA_PATH_GENERIC) {
        tiled = false;
    } else {
        tiled = tiled_possible && batch >= SPMM_TILED_MIN_BATCH;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the tiled kernels read the chunk table only, the generic kernel the offset table only
    if (tiled) e = noalloc_upload(tables + NOALLOC_CHUNKS_AT, chunks.data(), chunks.size() * sizeof(Chunk), s);
    else e = noalloc_upload(tables, offsets_host, (size_t)nd * sizeof(int), s);
    if (e != hipSuccess) return hip_fail(e, "table fill kernel launch");
    const SpEpilogue ep{nullptr, CUVDIA_ACT_NONE, 0u, 0u};
    e = tiled ? launch_spmm_tiled(view, A_vals, B, ldb, dst, ldd, batch, trans, alpha, beta, ep, s)
              : launch_spmm_generic(view, A_vals, B, ldb, dst, ldd, batch, trans, alpha, beta, ep, s);
    t_last_path = tiled ? CUVDIA_PATH_TILED : CUVDIA_PATH_GENERIC;
    return e == hipSuccess ? CUVDIA_OK : hip_fail(e, "spmm kernel launch");
}

int cuvdia_dd2dia_offsets_f32(float *C_vals, const int *offsets_host, int nd, int stride,
                              int h, int w, int row_fact, const float *A, long long lda,
                              const float *B, long long ldb, int batch,
                              float alpha, float beta, void *stream)
{
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    cuvdia_desc *d = nullptr;
    const int rc = cached_desc(offsets_host, nd, stride, h, w, row_fact, &d);
    if (rc) return rc;
    return cuvdia_dd2dia_f32(d, C_vals, A, lda, B, ldb, batch, alpha, beta, stream);
}

}  // extern "C"
