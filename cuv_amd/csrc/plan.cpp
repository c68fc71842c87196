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
