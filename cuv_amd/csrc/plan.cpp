#include "plan.hpp"

#include <algorithm>
#include <cstdint>
#include <utility>

namespace cuvdia {

std::vector<Chunk> plan_chunks(const int *offsets, int nd, bool transposed, int max_len)
{
    max_len = std::min(std::max(max_len, 1), CHUNK_SLOTS);
    std::vector<std::pair<long long, int>> s(nd);      // (shift, table position)
    for (int d = 0; d < nd; ++d)
        s[d] = { transposed ? -(long long)offsets[d] : (long long)offsets[d], d };
    std::stable_sort(s.begin(), s.end(),
                     [](const std::pair<long long, int> &a, const std::pair<long long, int> &b) {
                         return a.first < b.first;
                     });
    std::vector<Chunk> out;
    int i = 0;
    while (i < nd) {
        int j = i + 1;
        while (j < nd && s[j].first == s[j - 1].first + 1) ++j;
        const int run = j - i;
        const int pieces = (run + max_len - 1) / max_len;
        int done = 0;
        for (int p = 0; p < pieces; ++p) {
            const int len = (run - done + (pieces - p) - 1) / (pieces - p);
            Chunk c{};
            c.s0 = (int)s[i + done].first;
            c.len = len;
            for (int q = 0; q < CHUNK_SLOTS; ++q) c.slot[q] = q < len ? s[i + done + q].second : -1;
            out.push_back(c);
            done += len;
        }
        i = j;
    }
    return out;
}

namespace {
long long gcd_ll(long long a, long long b)
{
    while (b) { const long long t = a % b; a = b; b = t; }
    return a < 0 ? -a : a;
}
}  // namespace

void plan_walk(const std::vector<Chunk> &chunks, int stride, bool transposed, WalkPlan &plan)
{
    plan = WalkPlan{};
    const int n = (int)chunks.size();
    if (n < 2) return;
    // every chunk as long as the first, table positions in one arithmetic progression
    const int lck = chunks.front().len;
    long long step = 0;
    bool have_step = false;
    for (const Chunk &c : chunks) {
        if (c.len != lck) return;
        for (int j = 0; j < lck; ++j)
            if (c.slot[j] < 0) return;
        for (int j = 1; j < lck; ++j) {
            const long long d = (long long)c.slot[j] - c.slot[j - 1];
            if (!have_step) { step = d; have_step = true; }
            else if (d != step) return;
        }
    }
    const long long limit = 1LL << 29;               // 4 * value stays inside 32-bit signed arithmetic
    const long long astep = step * stride + (transposed ? 1 : 0);
    if (astep >= limit || astep <= -limit) return;
    // the period: what all the shifts' distances from the first are multiples of
    long long period = 0;
    for (int i = 1; i < n; ++i) {
        const long long d = (long long)chunks[i].s0 - chunks[0].s0;
        if (d <= 0) return;                          // shifts ascend strictly
        period = gcd_ll(period, d);
    }
    if (period <= 0 || period >= limit) return;
    // window rows: the leading shifts 0, period, 2 period, ...; then whole groups of the same k rows
    int k = 1;
    while (k < n && (long long)chunks[k].s0 - chunks[0].s0 == (long long)k * period) ++k;
    if (k < 2 || n % k != 0) return;                 // a window has at least two rows
    const int ngroups = n / k;
    std::vector<int> group_rows(ngroups), aoff4(n);
    for (int g = 0; g < ngroups; ++g) {
        const long long base = (long long)chunks[g * k].s0 - chunks[0].s0;
        if (base >= limit) return;
        group_rows[g] = (int)base;
        for (int dy = 0; dy < k; ++dy) {
            const Chunk &c = chunks[g * k + dy];
            if ((long long)c.s0 - chunks[0].s0 != base + (long long)dy * period) return;
            const long long aoff = (long long)c.slot[0] * stride + (transposed ? c.s0 : 0);
            if (aoff >= limit || aoff <= -limit) return;
            aoff4[g * k + dy] = (int)(4 * aoff);
        }
    }
    plan.ok = true;
    plan.period = (int)period;
    plan.k = k;
    plan.ngroups = ngroups;
    plan.s0 = chunks[0].s0;
    plan.lck = lck;
    plan.astep4 = (int)(4 * astep);
    plan.group_rows.swap(group_rows);
    plan.aoff4.swap(aoff4);
}

std::vector<Unit> plan_units(const std::vector<Chunk> &chunks)
{
    std::vector<Unit> out;
    const int n = (int)chunks.size();
    int c = 0;
    while (c < n) {
        if (c + 1 < n) {
            const long long delta = (long long)chunks[c + 1].s0 - chunks[c].s0;
            if (delta > 0 && delta <= PAIR_MAX_DELTA && delta % 4 == 0) {
                out.push_back(Unit{c, c + 1});
                c += 2;
                continue;
            }
        }
        out.push_back(Unit{c, -1});
        c += 1;
    }
    return out;
}

int common_slot_step(const std::vector<Chunk> &chunks)
{
    long long step = 0;
    bool have = false;
    for (const Chunk &c : chunks) {
        for (int j = 0; j < c.len; ++j)
            if (c.slot[j] < 0) return 0;
        for (int j = 1; j < c.len; ++j) {
            const long long d = (long long)c.slot[j] - c.slot[j - 1];
            if (!have) { step = d; have = true; }
            else if (d != step) return 0;
        }
    }
    // the kernels add j * step to a position below 2^31 / stride: keep it small
    return have && step != 0 && step > -(1 << 20) && step < (1 << 20) ? (int)step : 0;
}

int pair_delta_max(const std::vector<Chunk> &chunks, const std::vector<Unit> &units)
{
    int m = 0;
    for (const Unit &u : units)
        if (u.c2 >= 0) m = std::max(m, chunks[u.c2].s0 - chunks[u.c1].s0);
    return m;
}

long long count_valid(const int *offsets, int nd, int h, int w, int rf)
{
    long long total = 0;
    for (int d = 0; d < nd; ++d) {
        const long long k = offsets[d];
        const long long i0 = (long long)rf * std::max<long long>(0, -k);
        const long long j0 = std::max<long long>(0, k);
        const long long n = std::min<long long>(h - i0, (long long)rf * (w - j0));
        if (n > 0) total += n;
    }
    return total;
}

}  // namespace cuvdia
