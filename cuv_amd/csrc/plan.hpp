// Host-side decomposition of a DIA offset table into run chunks.
//
// A tiled kernel does not walk the offset table diagonal by diagonal; it
// walks *chunks*: a few consecutive shifts (s0, s0+1, ...) whose
// dense-operand rows overlap, so one staged window of the dense tile serves
// all of them.  The products take chunks of up to SP_CHUNK_MAX shifts (what
// the 76 dense rows they stage per chunk can serve for 64 output rows), the
// dense x dense^T projection chunks of up to CHUNK_MAX (it keeps 4 running
// sums per shift and lane).  For the normal product the shift of diagonal d is its offset
// k_d (input row = output row + k_d); for the transposed product it is -k_d.
#pragma once
#include <vector>

namespace cuvdia {

constexpr int CHUNK_MAX = 8;        // longest chunk of the projection's table
constexpr int SP_CHUNK_MAX = 13;    // longest chunk of the products' tables
constexpr int CHUNK_SLOTS = 14;

// 64 bytes; read by the kernels through scalar loads.
struct Chunk {
    int s0;                 // shift of the first position in the chunk
    int len;                // number of positions, 1..max_len of the table
    int slot[CHUNK_SLOTS];  // table position (d) of each, so values sit at vals[slot*stride + ...];
                            // -1 marks a position no diagonal occupies
};
static_assert(sizeof(Chunk) == 64 && SP_CHUNK_MAX <= CHUNK_SLOTS, "Chunk layout is part of the device table");

// A *window* table, the shape a 2-d (or multi-channel 2-d) local connection pattern gives a DIA matrix: every
// chunk has `lck` diagonals at table positions in arithmetic progression (one step for the whole table), and
// the chunks' shifts form a complete grid
//     s(g, dy) = s0 + group_rows[g] + dy * period,    g < ngroups, dy < k,
// -- k window rows `period` rows apart, repeated for every group (channel offset).  Output tiles `period` rows
// apart then read the same dense rows for neighbouring window rows, which is what the products' walking kernel
// exploits.  aoff4[g * k + dy] is 4 * the element offset of chunk (g, dy)'s first diagonal for output row 0,
// astep4 4 * the element step between its diagonals (value of (chunk, diagonal j, output row r):
// element aoff + r + j * astep).
struct WalkPlan {
    bool ok = false;
    int period = 0, k = 0, ngroups = 0, s0 = 0, lck = 0, astep4 = 0;
    std::vector<int> group_rows;     // ngroups, ascending, group_rows[0] == 0
    std::vector<int> aoff4;          // ngroups * k
};
// `chunks`: a table from plan_chunks (shifts ascending).  plan.ok is false when the table is no window table.
void plan_walk(const std::vector<Chunk> &chunks, int stride, bool transposed, WalkPlan &plan);

// Sort shifts (stable in table position), cut into maximal runs of
// consecutive shifts -- a repeated shift starts a new run -- and split each
// run into near-equal chunks of at most max_len (<= CHUNK_SLOTS).  Positions
// past a chunk's length carry slot -1.
std::vector<Chunk> plan_chunks(const int *offsets, int nd, bool transposed, int max_len = CHUNK_MAX);

// A unit of work of the tiled dense x dense^T projection: one chunk, or two
// chunks of the normal table whose first shifts differ by a multiple of 4 of
// at most PAIR_MAX_DELTA rows.  Up to PAIR_BAND_DELTA rows apart a wave can serve both chunks of a pair from one
// staged band of the second operand and one copy of the first operand's rows (up to PAIR_NARROW_DELTA the band
// fits two 16-byte pieces per lane and column; a table with a wider pair runs the kernel that takes three).  At any
// distance it can let the second chunk work on the rows that far above the first's: both then read the same rows of
// the second operand (window rows of a map of any width).
constexpr int PAIR_MAX_DELTA = 4096;
constexpr int PAIR_BAND_DELTA = 256;
constexpr int PAIR_NARROW_DELTA = 128;
struct Unit {
    int c1;                 // chunk index
    int c2;                 // second chunk index, or -1
};
// Greedy over the table in shift order: chunk c pairs with c + 1 when their
// shifts allow it.
std::vector<Unit> plan_units(const std::vector<Chunk> &chunks);
// The distance in table positions between neighbouring diagonals of a chunk when it is the same for every chunk
// of the table (1 for a table listed in ascending order of its offsets), else 0.  The products' kernels then
// compute a diagonal's table position instead of picking it out of the chunk's entry.
int common_slot_step(const std::vector<Chunk> &chunks);
// The largest distance between the first shifts of a pair (0 without pairs).
int pair_delta_max(const std::vector<Chunk> &chunks, const std::vector<Unit> &units);

// Number of matrix elements stored (slots the reference host loops touch):
// sum over diagonals of min(h - rf*max(0,-k), rf*(w - max(0,k))), clamped at 0
// (src/cuv/matrix_ops/spmv.cu:183-189).
long long count_valid(const int *offsets, int nd, int h, int w, int rf);

}  // namespace cuvdia
