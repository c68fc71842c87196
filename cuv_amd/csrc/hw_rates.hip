// Measures, on the GPU it runs on, the two rates the product kernels are laid out around:
//   * how fast a SIMD issues fp32 FMAs in the forms a kernel can give them -- three vector-register operands (with
//     the two multiplicands in different banks of the register file or in the same one), a DPP-broadcast operand
//     (v_fmac_f32_dpp .. row_newbcast), a scalar operand;
//   * how fast a CU's LDS answers 4-, 8- and 16-byte reads, with an address per lane and with one per wave;
//   * what one launch that only moves the headline up-pass's bytes costs -- 8.4 MB + 3.2 MB read, 8.4 MB written,
//     no arithmetic to speak of -- launched back to back from a HIP graph, with its operands in HBM (31 rotating
//     buffer sets) and in the caches (one set): the time no kernel of that traffic can go below on this machine.
// The kernels keep the batch along the lanes and broadcast a diagonal's value to them; this probe shows what that
// form costs against the plain one, and what feeding the plain form from LDS would need.
// Built by the Makefile into ../lib/hw_rates; prints one line per measurement.  Every wave runs a fixed number of
// iterations and the grid is one resident round of workgroups.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <vector>

#define HW_CHECK(call)                                                                      \
    do {                                                                                    \
        const hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess) {                                                             \
            std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));                 \
            return 1;                                                                       \
        }                                                                                   \
    } while (0)

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

// 16 independent running sums per lane, 64 FMAs per iteration
template <int FORM>
__global__ __launch_bounds__(256) void fma_kernel(float *out, long long *clk, int iters, float a, float sa)
{
    float acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = threadIdx.x * 0.001f + i;
    const float x = a + threadIdx.x;
    // FORM 3 and 4: three vector registers of the compiler's choosing, no two FMAs in a row sharing an operand
    // register -- 8 + 8 (FORM 4: 4 + 16) different ones, as in a tile's inner loop
    float xs[16], as[16];
    for (int i = 0; i < 16; ++i) {
        xs[i] = x + i;
        as[i] = a * (i + 1);
        asm volatile("" : "+v"(xs[i]), "+v"(as[i]));
    }
    const long long c0 = clock64(), w0 = wall_clock64();
    // FORM 5 .. 9: the same FMAs on registers named outright, to place the three operands in the register file's four
    // banks (a register's bank is its number modulo 4):
    //   5 -- sums in consecutive registers, multiplicands in banks 0 and 1
    //   6 -- sums in banks 2 and 3, multiplicands in banks 0 and 1: no two operands share a bank
    //   7 -- sums in consecutive registers, both multiplicands in bank 0
    //   8 -- sums in banks 2 and 3, both multiplicands in bank 0
    //   9 -- all three operands in bank 0
    //   10, 11 -- the DPP form with its two multiplicands in banks 0 and 1, and both in bank 0
    if (FORM >= 5) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (FORM == 5)
                asm volatile(
                    "v_fmac_f32 v108, v100, v101\n\t"
                    "v_fmac_f32 v109, v100, v101\n\t"
                    "v_fmac_f32 v110, v100, v101\n\t"
                    "v_fmac_f32 v111, v100, v101\n\t"
                    "v_fmac_f32 v112, v100, v101\n\t"
                    "v_fmac_f32 v113, v100, v101\n\t"
                    "v_fmac_f32 v114, v100, v101\n\t"
                    "v_fmac_f32 v115, v100, v101\n\t"
                    "v_fmac_f32 v116, v100, v101\n\t"
                    "v_fmac_f32 v117, v100, v101\n\t"
                    "v_fmac_f32 v118, v100, v101\n\t"
                    "v_fmac_f32 v119, v100, v101\n\t"
                    "v_fmac_f32 v120, v100, v101\n\t"
                    "v_fmac_f32 v121, v100, v101\n\t"
                    "v_fmac_f32 v122, v100, v101\n\t"
                    "v_fmac_f32 v123, v100, v101\n\t"
                    ::: "v100", "v101", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123");
                if (FORM == 6)
                asm volatile(
                    "v_fmac_f32 v110, v100, v101\n\t"
                    "v_fmac_f32 v111, v100, v101\n\t"
                    "v_fmac_f32 v114, v100, v101\n\t"
                    "v_fmac_f32 v115, v100, v101\n\t"
                    "v_fmac_f32 v118, v100, v101\n\t"
                    "v_fmac_f32 v119, v100, v101\n\t"
                    "v_fmac_f32 v122, v100, v101\n\t"
                    "v_fmac_f32 v123, v100, v101\n\t"
                    "v_fmac_f32 v126, v100, v101\n\t"
                    "v_fmac_f32 v127, v100, v101\n\t"
                    "v_fmac_f32 v130, v100, v101\n\t"
                    "v_fmac_f32 v131, v100, v101\n\t"
                    "v_fmac_f32 v134, v100, v101\n\t"
                    "v_fmac_f32 v135, v100, v101\n\t"
                    "v_fmac_f32 v138, v100, v101\n\t"
                    "v_fmac_f32 v139, v100, v101\n\t"
                    ::: "v100", "v101", "v110", "v111", "v114", "v115", "v118", "v119", "v122", "v123", "v126", "v127", "v130", "v131", "v134", "v135", "v138", "v139");
                if (FORM == 7)
                asm volatile(
                    "v_fmac_f32 v108, v100, v104\n\t"
                    "v_fmac_f32 v109, v100, v104\n\t"
                    "v_fmac_f32 v110, v100, v104\n\t"
                    "v_fmac_f32 v111, v100, v104\n\t"
                    "v_fmac_f32 v112, v100, v104\n\t"
                    "v_fmac_f32 v113, v100, v104\n\t"
                    "v_fmac_f32 v114, v100, v104\n\t"
                    "v_fmac_f32 v115, v100, v104\n\t"
                    "v_fmac_f32 v116, v100, v104\n\t"
                    "v_fmac_f32 v117, v100, v104\n\t"
                    "v_fmac_f32 v118, v100, v104\n\t"
                    "v_fmac_f32 v119, v100, v104\n\t"
                    "v_fmac_f32 v120, v100, v104\n\t"
                    "v_fmac_f32 v121, v100, v104\n\t"
                    "v_fmac_f32 v122, v100, v104\n\t"
                    "v_fmac_f32 v123, v100, v104\n\t"
                    ::: "v100", "v104", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123");
                if (FORM == 8)
                asm volatile(
                    "v_fmac_f32 v110, v100, v104\n\t"
                    "v_fmac_f32 v111, v100, v104\n\t"
                    "v_fmac_f32 v114, v100, v104\n\t"
                    "v_fmac_f32 v115, v100, v104\n\t"
                    "v_fmac_f32 v118, v100, v104\n\t"
                    "v_fmac_f32 v119, v100, v104\n\t"
                    "v_fmac_f32 v122, v100, v104\n\t"
                    "v_fmac_f32 v123, v100, v104\n\t"
                    "v_fmac_f32 v126, v100, v104\n\t"
                    "v_fmac_f32 v127, v100, v104\n\t"
                    "v_fmac_f32 v130, v100, v104\n\t"
                    "v_fmac_f32 v131, v100, v104\n\t"
                    "v_fmac_f32 v134, v100, v104\n\t"
                    "v_fmac_f32 v135, v100, v104\n\t"
                    "v_fmac_f32 v138, v100, v104\n\t"
                    "v_fmac_f32 v139, v100, v104\n\t"
                    ::: "v100", "v104", "v110", "v111", "v114", "v115", "v118", "v119", "v122", "v123", "v126", "v127", "v130", "v131", "v134", "v135", "v138", "v139");
                if (FORM == 9)
                asm volatile(
                    "v_fmac_f32 v108, v100, v104\n\t"
                    "v_fmac_f32 v112, v100, v104\n\t"
                    "v_fmac_f32 v116, v100, v104\n\t"
                    "v_fmac_f32 v120, v100, v104\n\t"
                    "v_fmac_f32 v124, v100, v104\n\t"
                    "v_fmac_f32 v128, v100, v104\n\t"
                    "v_fmac_f32 v132, v100, v104\n\t"
                    "v_fmac_f32 v136, v100, v104\n\t"
                    "v_fmac_f32 v140, v100, v104\n\t"
                    "v_fmac_f32 v144, v100, v104\n\t"
                    "v_fmac_f32 v148, v100, v104\n\t"
                    "v_fmac_f32 v152, v100, v104\n\t"
                    "v_fmac_f32 v156, v100, v104\n\t"
                    "v_fmac_f32 v160, v100, v104\n\t"
                    "v_fmac_f32 v164, v100, v104\n\t"
                    "v_fmac_f32 v168, v100, v104\n\t"
                    ::: "v100", "v104", "v108", "v112", "v116", "v120", "v124", "v128", "v132", "v136", "v140", "v144", "v148", "v152", "v156", "v160", "v164", "v168");
                if (FORM == 10)
                asm volatile(
                    "s_nop 1\n\t"
                    "v_fmac_f32_dpp v108, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v109, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v110, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v111, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v112, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v113, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v114, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v115, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v116, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v117, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v118, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v119, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v120, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v121, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v122, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v123, v100, v101 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    ::: "v100", "v101", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123");
                if (FORM == 11)
                asm volatile(
                    "s_nop 1\n\t"
                    "v_fmac_f32_dpp v108, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v109, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v110, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v111, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v112, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v113, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v114, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v115, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v116, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v117, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v118, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v119, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v120, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v121, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v122, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_fmac_f32_dpp v123, v100, v104 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
                    ::: "v100", "v104", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123");
            }
        }
    }
    for (int it = 0; FORM < 5 && it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if (FORM == 3)
                    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[i]) : "v"(xs[(i + 3 * r) % 8]), "v"(as[(i / 2 + r) % 8]));
                if (FORM == 4)
                    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[i]) : "v"(xs[i / 4]), "v"(as[(i % 4 + i / 4 + 4 * r) % 16]));
                if (FORM == 1)
                    asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:1 row_mask:0xf bank_mask:0xf"
                                 : "+v"(acc[i]) : "v"(x), "v"(a));
                if (FORM == 2) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[i]) : "s"(sa), "v"(a));
            }
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0;
    for (int i = 0; i < 16; ++i) s += acc[i];
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (threadIdx.x == 0) {
        clk[2 * blockIdx.x] = c1 - c0;
        clk[2 * blockIdx.x + 1] = w1 - w0;
    }
}

// every lane reads 4 W bytes per instruction at consecutive addresses (conflict-free), 8 instructions per iteration
// UNIFORM: every lane of a wave reads the same address (a value broadcast to the wave)
template <int W, bool UNIFORM = false>
__global__ __launch_bounds__(256) void lds_kernel(float *out, long long *clk, int iters)
{
    __shared__ __attribute__((aligned(16))) float buf[8192];
    for (int i = threadIdx.x; i < 8192; i += 256) buf[i] = i;
    __syncthreads();
    const unsigned base =
        (unsigned)(unsigned long long)(__attribute__((address_space(3))) float *)buf +
        (UNIFORM ? (threadIdx.x >> 6) * 64 : threadIdx.x * (W * 4));
    float sum = 0.f;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (W == 4) {
                f4 v;
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(base), "n"(r * 4096));
                asm volatile("s_waitcnt lgkmcnt(4)");
                if (r == 7) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v)); sum += v.x; }
            }
            if (W == 2) {
                f2 v;
                asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(base), "n"(r * 2048));
                asm volatile("s_waitcnt lgkmcnt(4)");
                if (r == 7) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v)); sum += v.x; }
            }
            if (W == 1) {
                float v;
                asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(base), "n"(r * 1024));
                asm volatile("s_waitcnt lgkmcnt(4)");
                if (r == 7) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v)); sum += v; }
            }
        }
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    out[blockIdx.x * 256 + threadIdx.x] = sum;
    if (threadIdx.x == 0) {
        clk[2 * blockIdx.x] = c1 - c0;
        clk[2 * blockIdx.x + 1] = w1 - w0;
    }
}

// y[i] = x[i] (+ a[i] for i < na4), 16-byte pieces, PT pieces per lane all requested before the first is stored
template <int PT>
__global__ __launch_bounds__(256) void stream_kernel(const f4 *__restrict__ x, const f4 *__restrict__ a,
                                                     f4 *__restrict__ y, int n4, int na4)
{
    const int t = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
    f4 v[PT];
#pragma unroll
    for (int k = 0; k < PT; ++k) {
        const int i = t + k * stride;
        v[k] = i < n4 ? x[i] : f4{0.f, 0.f, 0.f, 0.f};
        if (i < na4) v[k] += a[i];
    }
#pragma unroll
    for (int k = 0; k < PT; ++k) {
        const int i = t + k * stride;
        if (i < n4) __builtin_nontemporal_store(v[k], &y[i]);
    }
}

struct Probe {
    float *out = nullptr;
    long long *clk = nullptr;
    int cus = 0, wgs = 0;
    hipEvent_t e0{}, e1{};
    std::vector<long long> host;
};

// shader clock during the kernel: s_memtime ticks per tick of the constant 100 MHz clock, averaged over workgroups
static int finish(Probe &p, float *ms, double *mhz)
{
    HW_CHECK(hipEventSynchronize(p.e1));
    HW_CHECK(hipEventElapsedTime(ms, p.e0, p.e1));
    HW_CHECK(hipMemcpy(p.host.data(), p.clk, (size_t)p.wgs * 16, hipMemcpyDeviceToHost));
    double cs = 0, ws = 0;
    for (int i = 0; i < p.wgs; ++i) { cs += (double)p.host[2 * i]; ws += (double)p.host[2 * i + 1]; }
    *mhz = ws > 0 ? cs / ws * 100.0 : 0.0;
    return 0;
}

template <int FORM>
static int run_fma(Probe &p, const char *name)
{
    const int iters = 20000;
    float ms = 0;
    double mhz = 0;
    for (int rep = 0; rep < 2; ++rep) {
        HW_CHECK(hipEventRecord(p.e0));
        hipLaunchKernelGGL(fma_kernel<FORM>, dim3(p.wgs), dim3(256), 0, 0, p.out, p.clk, iters, 1.0001f, 0.5f);
        HW_CHECK(hipGetLastError());
        HW_CHECK(hipEventRecord(p.e1));
        if (finish(p, &ms, &mhz)) return 1;
    }
    const double flops = 2.0 * 64 * iters * 256.0 * p.wgs;
    const double per_simd = (double)ms * 1e-3 * mhz * 1e6 / (64.0 * iters * (256.0 / 64.0) * p.wgs / (4.0 * p.cus));
    std::printf("fma  %-34s %8.3f ms  %6.1f TFLOP/s  %.2f clocks per wave64 FMA per SIMD  shader clock %.0f MHz\n",
                name, ms, flops / ms / 1e9, per_simd, mhz);
    std::fflush(stdout);
    return 0;
}

template <int W, bool UNIFORM = false>
static int run_lds(Probe &p, const char *name)
{
    const int iters = 20000;
    float ms = 0;
    double mhz = 0;
    for (int rep = 0; rep < 2; ++rep) {
        HW_CHECK(hipEventRecord(p.e0));
        hipLaunchKernelGGL((lds_kernel<W, UNIFORM>), dim3(p.wgs), dim3(256), 0, 0, p.out, p.clk, iters);
        HW_CHECK(hipGetLastError());
        HW_CHECK(hipEventRecord(p.e1));
        if (finish(p, &ms, &mhz)) return 1;
    }
    const double bytes = 8.0 * iters * 256.0 * p.wgs * W * 4;
    std::printf("lds  %-34s %8.3f ms  %6.1f B/clk/CU  shader clock %.0f MHz\n", name, ms,
                bytes / ((double)ms * 1e-3) / p.cus / (mhz * 1e6), mhz);
    std::fflush(stdout);
    return 0;
}

// One launch per buffer set, `sets` launches recorded into a HIP graph and replayed.
template <int PT>
static int run_stream(int sets, const char *name)
{
    const int n4 = 16384 * 128 / 4, na4 = 49 * 16384 / 4;          // the headline layer: batch 128, 49 diagonals
    const int total_sets = 31;
    static f4 *x[31], *a[31], *y[31];
    static bool ready = false;
    if (!ready) {
        for (int s = 0; s < total_sets; ++s) {
            HW_CHECK(hipMalloc(&x[s], (size_t)n4 * 16));
            HW_CHECK(hipMalloc(&a[s], (size_t)na4 * 16));
            HW_CHECK(hipMalloc(&y[s], (size_t)n4 * 16));
            HW_CHECK(hipMemset(x[s], 0, (size_t)n4 * 16));
            HW_CHECK(hipMemset(a[s], 0, (size_t)na4 * 16));
        }
        ready = true;
    }
    hipStream_t st;
    HW_CHECK(hipStreamCreate(&st));
    hipGraph_t graph;
    hipGraphExec_t exec;
    const int wgs = (n4 + 256 * PT - 1) / (256 * PT);
    HW_CHECK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
    for (int s = 0; s < total_sets; ++s) {
        const int b = s % sets;
        hipLaunchKernelGGL(stream_kernel<PT>, dim3(wgs), dim3(256), 0, st, x[b], a[b], y[b], n4, na4);
    }
    HW_CHECK(hipStreamEndCapture(st, &graph));
    HW_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    hipEvent_t e0, e1;
    HW_CHECK(hipEventCreate(&e0));
    HW_CHECK(hipEventCreate(&e1));
    const int reps = 40;
    for (int r = 0; r < 5; ++r) HW_CHECK(hipGraphLaunch(exec, st));
    HW_CHECK(hipEventRecord(e0, st));
    for (int r = 0; r < reps; ++r) HW_CHECK(hipGraphLaunch(exec, st));
    HW_CHECK(hipEventRecord(e1, st));
    HW_CHECK(hipEventSynchronize(e1));
    float ms = 0;
    HW_CHECK(hipEventElapsedTime(&ms, e0, e1));
    const double us = (double)ms * 1e3 / (reps * total_sets);
    const double bytes = 16.0 * (2.0 * n4 + na4);
    std::printf("move %-34s %6.2f us per launch  %6.0f GB/s  (%d workgroups, %.2f MB per launch)\n", name, us,
                bytes / us / 1e3, wgs, bytes / 1e6);
    std::fflush(stdout);
    HW_CHECK(hipGraphExecDestroy(exec));
    HW_CHECK(hipGraphDestroy(graph));
    HW_CHECK(hipEventDestroy(e0));
    HW_CHECK(hipEventDestroy(e1));
    HW_CHECK(hipStreamDestroy(st));
    return 0;
}

int main()
{
    hipDeviceProp_t prop;
    HW_CHECK(hipGetDeviceProperties(&prop, 0));
    Probe p;
    p.cus = prop.multiProcessorCount;
    p.wgs = p.cus * 4;                       // 16 waves per CU: one resident round
    p.host.resize((size_t)2 * p.wgs);
    HW_CHECK(hipMalloc(&p.out, (size_t)p.wgs * 256 * 4));
    HW_CHECK(hipMalloc(&p.clk, (size_t)p.wgs * 16));
    HW_CHECK(hipEventCreate(&p.e0));
    HW_CHECK(hipEventCreate(&p.e1));
    std::printf("%s, %d CUs\n", prop.name, p.cus);
    if (run_fma<1>(p, "v_fmac_f32_dpp row_newbcast")) return 1;
    if (run_fma<2>(p, "v_fmac_f32 v, s, v")) return 1;
    if (run_fma<5>(p, "v v v: sums consecutive, a b banks 0 1")) return 1;
    if (run_fma<6>(p, "v v v: sums banks 2 3, a b banks 0 1")) return 1;
    if (run_fma<7>(p, "v v v: sums consecutive, a b bank 0")) return 1;
    if (run_fma<8>(p, "v v v: sums banks 2 3, a b bank 0")) return 1;
    if (run_fma<9>(p, "v v v: all in bank 0")) return 1;
    if (run_fma<10>(p, "dpp: sums consecutive, a b banks 0 1")) return 1;
    if (run_fma<11>(p, "dpp: sums consecutive, a b bank 0")) return 1;
    if (run_fma<3>(p, "v_fmac_f32 v, v, v (8 x 8 operands)")) return 1;
    if (run_fma<4>(p, "v_fmac_f32 v, v, v (4 x 16 operands)")) return 1;
    if (run_lds<4>(p, "ds_read_b128")) return 1;
    if (run_lds<2>(p, "ds_read_b64")) return 1;
    if (run_lds<1>(p, "ds_read_b32")) return 1;
    if (run_lds<4, true>(p, "ds_read_b128, one address per wave")) return 1;
    if (run_lds<2, true>(p, "ds_read_b64, one address per wave")) return 1;
    if (run_lds<1, true>(p, "ds_read_b32, one address per wave")) return 1;
    if (run_stream<1>(31, "operands in HBM, 1 piece per lane")) return 1;
    if (run_stream<2>(31, "operands in HBM, 2 pieces per lane")) return 1;
    if (run_stream<4>(31, "operands in HBM, 4 pieces per lane")) return 1;
    if (run_stream<8>(31, "operands in HBM, 8 pieces per lane")) return 1;
    if (run_stream<1>(1, "operands cached,  1 piece per lane")) return 1;
    if (run_stream<2>(1, "operands cached,  2 pieces per lane")) return 1;
    if (run_stream<4>(1, "operands cached,  4 pieces per lane")) return 1;
    if (run_stream<8>(1, "operands cached,  8 pieces per lane")) return 1;
    HW_CHECK(hipFree(p.out));
    HW_CHECK(hipFree(p.clk));
    return 0;
}
