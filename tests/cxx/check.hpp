// Minimal test harness for the C++ API programs (stands in for Boost.Test).
#ifndef CUVDIA_TEST_CHECK_HPP
#define CUVDIA_TEST_CHECK_HPP
#include <cmath>
#include <cstdio>
#include <cstring>
#include <exception>
#include <functional>
#include <string>
#include <vector>

struct TestCase { const char *name; std::function<void()> fn; };
inline std::vector<TestCase> &registry() { static std::vector<TestCase> r; return r; }
struct Registrar { Registrar(const char *n, std::function<void()> f) { registry().push_back({n, f}); } };
inline int &failures() { static int f = 0; return f; }

#define TEST_CASE(NAME) \
    static void NAME(); \
    static Registrar reg_##NAME(#NAME, NAME); \
    static void NAME()

#define CHECK(X) \
    do { if (!(X)) { std::printf("    CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #X); ++failures(); } } while (0)

#define CHECK_THROWS(X) \
    do { bool t_ = false; try { X; } catch (const std::runtime_error &) { t_ = true; } \
         if (!t_) { std::printf("    expected std::runtime_error %s:%d: %s\n", __FILE__, __LINE__, #X); ++failures(); } } while (0)

// Boost's percent_tolerance semantics (src/cuv/tools/cuv_test.hpp:39-57):
// |a-b| <= pct/100 * |a| and <= pct/100 * |b|
inline bool close_pct(float a, float b, float pct)
{
    if (a == b) return true;
    const float d = std::fabs(a - b), t = pct / 100.f;
    return d <= t * std::fabs(a) && d <= t * std::fabs(b);
}

template <class M, class N>
bool matrix_eq(const M &w, const N &w2, float pct)
{
    for (unsigned i = 0; i < w.shape()[0]; i++)
        for (unsigned j = 0; j < w.shape()[1]; j++)
            if (!close_pct((float)w(i, j), (float)w2(i, j), pct)) {
                std::printf("    mismatch at (%u,%u): %g vs %g\n", i, j, (double)(float)w(i, j), (double)(float)w2(i, j));
                return false;
            }
    return true;
}
#define MAT_CMP(X, Y, PREC) CHECK(matrix_eq(X, Y, PREC))

inline int run_all(int argc, char **argv)
{
    int ran = 0;
    for (auto &t : registry()) {
        if (argc > 1 && std::strcmp(argv[1], t.name) != 0) continue;
        const int before = failures();
        std::printf("[ RUN  ] %s\n", t.name); std::fflush(stdout);
        try { t.fn(); }
        catch (const std::exception &e) { std::printf("    unexpected exception: %s\n", e.what()); ++failures(); }
        std::printf("[ %s ] %s\n", failures() == before ? " OK " : "FAIL", t.name); std::fflush(stdout);
        ++ran;
    }
    std::printf("%d test(s), %d failure(s)\n", ran, failures());
    return failures() ? 1 : 0;
}
#endif
