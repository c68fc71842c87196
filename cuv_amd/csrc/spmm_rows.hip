// gfx950 (MI355X, CDNA4): the product with a diagonal-sparse matrix for LARGE operands, rows along the lanes.
//
// The tiled kernels of kernels.hip keep the batch along the lanes and hand a diagonal's value to all 64 lanes
// through DPP: such an FMA issues every 4 clocks.  A wave64 FMA on three plain vector registers issues every 2
// -- if its two multiplicands sit in different banks of the register file (bank = register number mod 4) and
// two waves share the SIMD.  This kernel is laid out for that form:
//
//   * lane l of a wave owns 8 consecutive output rows (row0 + 8 l ..) of 4 batch columns: 32 running sums;
//   * a diagonal's values for those rows are the lane's own: they are staged once per workgroup and chunk in
//     LDS (loads that write LDS directly, 16 bytes per lane) and read back as two 16-byte reads per diagonal;
//   * the dense rows a chunk of LCK consecutive shifts needs -- 8 + LCK - 1 per lane and column -- are the
//     lane's own 8 rows, loaded from memory straight into registers (two 16-byte loads per column), plus the
//     LCK - 1 that follow, which are the own rows of the next one or two lanes: those come through DPP
//     (v_mov_b32_dpp wave_shl:1), no LDS traffic and no barrier for the dense operand at all;
//   * every multiplicand has a fixed register, chosen so that no FMA reads two registers of one bank: the
//     window of column c sits in consecutive registers from a multiple of 4, the 8 values of diagonal j in
//     consecutive registers from 2 (mod 4) for j = 0, 1 (mod 4) and from 0 (mod 4) for j = 2, 3 (mod 4).  The
//     compiler cannot place registers, so the chunk's arithmetic is one assembly statement on named registers
//     (v64 and up; the compiler's own values stay below, which the build checks);
//   * the last one or two lanes of a wave have no neighbour to take their halo from: they compute nothing that
//     is stored, and a tile is 8 x 62 = 496 rows (LCK > 7) or 8 x 63 = 504 rows (LCK <= 7).
//
// Workgroup = 8 waves = one tile of rows x 32 batch columns (a wave per 4 columns), two waves per SIMD.  An
// instruction that is no plain FMA (DPP move, LDS read, load) costs the SIMD the slot of one or two FMAs, and
// the older of the two waves on a SIMD is served first: left alone it runs at the speed of a wave that is by
// itself and the other one starves.  The two therefore trade priority diagonal by diagonal (s_setprio), waves
// 0-3 high on even diagonals, waves 4-7 on odd ones.
//
// Accumulation order (per output element, fp32 fused multiply-add): acc = 0; the chunks that have rows inside
// the dense operand in ascending shift order, the diagonals of a chunk in ascending shift order,
// acc = fma(a, x, acc); then dst = alpha*acc (beta == 0, dst not read) or fma(beta, dst, alpha*acc).
#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace cuvdia {
namespace {

constexpr int RW_T = 8;                 // rows per lane
constexpr int RW_C = 4;                 // batch columns per lane
constexpr int RW_WAVES = 8;
constexpr int RW_COLS = RW_C * RW_WAVES;    // batch columns per workgroup
constexpr int RW_LOADED = 64 * RW_T;        // rows a wave loads per column
constexpr unsigned RW_OOB = 0x80000000u;    // a byte offset beyond every buffer resource used here
constexpr int RW_MAX_CHUNKS = 256;

constexpr int rw_valid_lanes(int lck) { return 64 - (lck - 1 + RW_T - 1) / RW_T; }
constexpr int rw_tile_rows(int lck) { return RW_T * rw_valid_lanes(lck); }
// LDS: two buffers of diagonal values, 2 x lck pieces of 1 KB each (piece 2 j + half: lane l's rows
// 8 l + 4 half .. + 3 of diagonal j at byte 16 l); at the end every wave passes its 4 x 512 sums through 8 KB.
constexpr int rw_abuf_bytes(int lck) { return 2 * lck * 1024; }
constexpr int rw_lds_bytes(int lck) { return 2 * rw_abuf_bytes(lck) > RW_WAVES * 8192 ? 2 * rw_abuf_bytes(lck) : RW_WAVES * 8192; }

// ---- the named registers --------------------------------------------------------------------------------
//   v66 ..  v99   four buffers of 8 diagonal values (RW_A0, RW_A1: first register 2 mod 4; RW_A2, RW_A3: 0 mod 4)
//   v100 .. v131  sums, RW_ACC + 8 c + t
//   v132 .. v163  own dense rows, set 0: RW_OWN0 + 8 c + k      (window positions 0 .. 7)
//   v164 .. v195  own dense rows, set 1 (chunks alternate between the sets: one is used while the other loads)
//   v196 .. v243  halo: RW_HALO + 12 c + m                      (window positions 8 + m)
#define RW_DEFS \
    ".set RW_A0, 66\n.set RW_A1, 74\n.set RW_A2, 84\n.set RW_A3, 92\n" \
    ".set RW_ACC, 100\n.set RW_OWN0, 132\n.set RW_OWN1, 164\n.set RW_HALO, 196\n" \
    ".macro RW_FMAD p, j, ab\n" \
    " .irp c,0,1,2,3\n" \
    "  .irp t,0,1,2,3,4,5,6,7\n" \
    "   .if (\\t+\\j) < 8\n" \
    "     v_fmac_f32 v[RW_ACC+8*\\c+\\t], v[\\ab+\\t], v[RW_OWN\\p+8*\\c+\\t+\\j]\n" \
    "   .else\n" \
    "     v_fmac_f32 v[RW_ACC+8*\\c+\\t], v[\\ab+\\t], v[RW_HALO+12*\\c+\\t+\\j-8]\n" \
    "   .endif\n" \
    "  .endr\n" \
    " .endr\n" \
    ".endm\n" \
    ".macro RW_HALOS p, n\n" \
    " .irp c,0,1,2,3\n" \
    "  .irp k,0,1,2,3,4,5,6,7\n" \
    "   .if \\k < \\n\n" \
    "   v_mov_b32_dpp v[RW_HALO+12*\\c+\\k], v[RW_OWN\\p+8*\\c+\\k] wave_shl:1 row_mask:0xf bank_mask:0xf\n" \
    "   .endif\n" \
    "  .endr\n" \
    " .endr\n" \
    " .irp c,0,1,2,3\n" \
    "  .irp k,0,1,2,3\n" \
    "   .if (\\k+8) < \\n\n" \
    "   v_mov_b32_dpp v[RW_HALO+12*\\c+8+\\k], v[RW_HALO+12*\\c+\\k] wave_shl:1 row_mask:0xf bank_mask:0xf\n" \
    "   .endif\n" \
    "  .endr\n" \
    " .endr\n" \
    ".endm\n" \
    ".macro RW_AREAD ab, j, vaddr, base\n" \
    "  ds_read_b128 v[\\ab:\\ab+3], \\vaddr offset:\\base+\\j*2048\n" \
    "  ds_read_b128 v[\\ab+4:\\ab+7], \\vaddr offset:\\base+\\j*2048+1024\n" \
    ".endm\n" \
    ".macro RW_AREADJ j, vaddr, base\n" \
    " .if ((\\j) & 3) == 0\n RW_AREAD RW_A0, (\\j), \\vaddr, \\base\n .endif\n" \
    " .if ((\\j) & 3) == 1\n RW_AREAD RW_A1, (\\j), \\vaddr, \\base\n .endif\n" \
    " .if ((\\j) & 3) == 2\n RW_AREAD RW_A2, (\\j), \\vaddr, \\base\n .endif\n" \
    " .if ((\\j) & 3) == 3\n RW_AREAD RW_A3, (\\j), \\vaddr, \\base\n .endif\n" \
    ".endm\n" \
    ".macro RW_FMADJ p, j\n" \
    " .if ((\\j) & 3) == 0\n RW_FMAD \\p, \\j, RW_A0\n .endif\n" \
    " .if ((\\j) & 3) == 1\n RW_FMAD \\p, \\j, RW_A1\n .endif\n" \
    " .if ((\\j) & 3) == 2\n RW_FMAD \\p, \\j, RW_A2\n .endif\n" \
    " .if ((\\j) & 3) == 3\n RW_FMAD \\p, \\j, RW_A3\n .endif\n" \
    ".endm\n"
#define RW_PURGE ".purgem RW_FMAD\n.purgem RW_HALOS\n.purgem RW_AREAD\n.purgem RW_AREADJ\n.purgem RW_FMADJ\n"

#define RW_CLOB_A "v66","v67","v68","v69","v70","v71","v72","v73","v74","v75","v76","v77","v78","v79","v80","v81","v82","v83","v84","v85","v86","v87","v88","v89","v90","v91","v92","v93","v94","v95","v96","v97","v98","v99"
#define RW_CLOB_ACC "v100","v101","v102","v103","v104","v105","v106","v107","v108","v109","v110","v111","v112","v113","v114","v115","v116","v117","v118","v119","v120","v121","v122","v123","v124","v125","v126","v127","v128","v129","v130","v131"
#define RW_CLOB_OWN0 "v132","v133","v134","v135","v136","v137","v138","v139","v140","v141","v142","v143","v144","v145","v146","v147","v148","v149","v150","v151","v152","v153","v154","v155","v156","v157","v158","v159","v160","v161","v162","v163"
#define RW_CLOB_OWN1 "v164","v165","v166","v167","v168","v169","v170","v171","v172","v173","v174","v175","v176","v177","v178","v179","v180","v181","v182","v183","v184","v185","v186","v187","v188","v189","v190","v191","v192","v193","v194","v195"
#define RW_CLOB_HALO "v196","v197","v198","v199","v200","v201","v202","v203","v204","v205","v206","v207","v208","v209","v210","v211","v212","v213","v214","v215","v216","v217","v218","v219","v220","v221","v222","v223","v224","v225","v226","v227","v228","v229","v230","v231","v232","v233","v234","v235","v236","v237","v238","v239","v240","v241","v242","v243"
#define RW_CLOB_ALL RW_CLOB_A, RW_CLOB_ACC, RW_CLOB_OWN0, RW_CLOB_OWN1, RW_CLOB_HALO

typedef int rw_int4 __attribute__((ext_vector_type(4)));

// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin, and each XCD has its own L2: spans of 64
// consecutive tiles go to one XCD (see kernels.hip), the tail split evenly.
__device__ __forceinline__ int rw_xcd_tile(int bid, int nblk)
{
    constexpr int XCDS = 8, SPAN = 64, GROUP = XCDS * SPAN;
    const int full = nblk / GROUP * GROUP;
    if (bid < full) {
        const int g = bid / GROUP, in = bid - g * GROUP;
        return g * GROUP + (in % XCDS) * SPAN + in / XCDS;
    }
    const int rest = nblk - full, b = bid - full;
    const int q = rest / XCDS, r = rest % XCDS;
    const int xcd = b % XCDS;
    return full + xcd * q + (xcd < r ? xcd : r) + b / XCDS;
}

// A wave-uniform value pinned to a scalar register, whatever the compiler infers about it (an "s" operand of
// an assembly statement is otherwise printed as a vector register when the compiler keeps the value in one).
// Two issue rules of this hardware apply, and the compiler, which pads for its own instructions, does not look
// inside assembly statements: a vector register must not be read by v_readfirstlane in the issue slot after the
// vector instruction that wrote it (the compiler copies the value into the register right before the
// statement), and a scalar register written by a vector instruction must not be read by a memory instruction
// in the next 5 issue slots (these values are used by loads inside assembly statements).  The padding is part
// of the statement.
__device__ __forceinline__ int rw_pin(int v)
{
    int s;
    asm volatile("s_nop 1\n\tv_readfirstlane_b32 %0, %1\n\ts_nop 4" : "=s"(s) : "v"(v));
    return s;
}
__device__ __forceinline__ rw_int4 rw_rsrc(const void *base, unsigned bytes)
{
    const unsigned long long b = reinterpret_cast<unsigned long long>(base);
    return rw_int4{rw_pin((int)(unsigned)b), rw_pin((int)((unsigned)(b >> 32) & 0xffffu)), rw_pin((int)bytes),
                   rw_pin(0x00020000)};
}
// Loads that write LDS directly: lane i's 16 (4) bytes land at lds_byte_addr + 16 i (4 i); an out-of-range lane
// writes zeros.  M0 is set inside the statement (the compiler keeps nothing there).  The s_nop pads, together
// with the s_mov, the 5 issue slots a scalar operand needs when a vector instruction (a v_readfirstlane the
// compiler placed) wrote it just before the statement.
__device__ __forceinline__ void rw_lds_load_b128(rw_int4 rsrc, unsigned lds_byte_addr, unsigned voff, unsigned soff)
{
    lds_byte_addr = __builtin_amdgcn_readfirstlane(lds_byte_addr);
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_mov_b32 m0, %0\n\t"
                 "s_nop 3\n\t"
                 "buffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_byte_addr), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void rw_lds_load_b32(rw_int4 rsrc, unsigned lds_byte_addr, unsigned voff)
{
    lds_byte_addr = __builtin_amdgcn_readfirstlane(lds_byte_addr);
    asm volatile("s_mov_b32 m0, %0\n\t"
                 "s_nop 3\n\t"
                 "buffer_load_dword %1, %2, 0 offen lds"
                 :: "s"(lds_byte_addr), "v"(voff), "s"(rsrc) : "memory");
}

// The arithmetic of one chunk: own set P (0 / 1), its diagonal values in LDS at byte BASE of the value block;
// WPAR says on which diagonals this wave takes the higher priority.
#define RW_DIAG(P, J, LAST) \
    ".if " #J " < " #LAST "\n RW_AREADJ (" #J "+1), %0, %1\n s_waitcnt lgkmcnt(2)\n .else\n s_waitcnt lgkmcnt(0)\n .endif\n" \
    ".if ((" #J " ^ %2) & 1)\n s_setprio 0\n .else\n s_setprio 3\n .endif\n" \
    "RW_FMADJ " #P ", " #J "\n"
#define RW_CHUNK7(P) \
    RW_DEFS "RW_AREADJ 0, %0, %1\n RW_HALOS " #P ", 6\n" \
    RW_DIAG(P, 0, 6) RW_DIAG(P, 1, 6) RW_DIAG(P, 2, 6) RW_DIAG(P, 3, 6) RW_DIAG(P, 4, 6) RW_DIAG(P, 5, 6) RW_DIAG(P, 6, 6) \
    "s_setprio 0\n" RW_PURGE
#define RW_CHUNK13(P) \
    RW_DEFS "RW_AREADJ 0, %0, %1\n RW_HALOS " #P ", 12\n" \
    RW_DIAG(P, 0, 12) RW_DIAG(P, 1, 12) RW_DIAG(P, 2, 12) RW_DIAG(P, 3, 12) RW_DIAG(P, 4, 12) RW_DIAG(P, 5, 12) RW_DIAG(P, 6, 12) \
    RW_DIAG(P, 7, 12) RW_DIAG(P, 8, 12) RW_DIAG(P, 9, 12) RW_DIAG(P, 10, 12) RW_DIAG(P, 11, 12) RW_DIAG(P, 12, 12) \
    "s_setprio 0\n" RW_PURGE

template <int LCK, int P, int WPAR>
__device__ __forceinline__ void rw_compute(unsigned a_read_addr)
{
    constexpr int BASE = P * rw_abuf_bytes(LCK);
    static_assert(LCK == 7 || LCK == 13, "instantiated chunk lengths");
    if constexpr (LCK == 7) {
        if constexpr (P == 0) asm volatile(RW_CHUNK7(0) :: "v"(a_read_addr), "n"(BASE), "n"(WPAR) : "memory", RW_CLOB_ALL);
        else asm volatile(RW_CHUNK7(1) :: "v"(a_read_addr), "n"(BASE), "n"(WPAR) : "memory", RW_CLOB_ALL);
    } else {
        if constexpr (P == 0) asm volatile(RW_CHUNK13(0) :: "v"(a_read_addr), "n"(BASE), "n"(WPAR) : "memory", RW_CLOB_ALL);
        else asm volatile(RW_CHUNK13(1) :: "v"(a_read_addr), "n"(BASE), "n"(WPAR) : "memory", RW_CLOB_ALL);
    }
}

// requests the wave's own dense rows of a chunk that lies wholly inside the operand: 8 loads of 16 bytes per lane
template <int P>
__device__ __forceinline__ void rw_load_own(unsigned voff, rw_int4 rsrc, unsigned s0, unsigned s1, unsigned s2, unsigned s3)
{
#define RW_OWN_LOADS(Q) \
    RW_DEFS \
    "s_nop 4\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+0:RW_OWN" #Q "+3], %0, %1, %2 offen\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+4:RW_OWN" #Q "+7], %0, %1, %2 offen offset:16\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+8:RW_OWN" #Q "+11], %0, %1, %3 offen\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+12:RW_OWN" #Q "+15], %0, %1, %3 offen offset:16\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+16:RW_OWN" #Q "+19], %0, %1, %4 offen\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+20:RW_OWN" #Q "+23], %0, %1, %4 offen offset:16\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+24:RW_OWN" #Q "+27], %0, %1, %5 offen\n" \
    "buffer_load_dwordx4 v[RW_OWN" #Q "+28:RW_OWN" #Q "+31], %0, %1, %5 offen offset:16\n" \
    RW_PURGE
    if constexpr (P == 0) asm volatile(RW_OWN_LOADS(0) :: "v"(voff), "s"(rsrc), "s"(s0), "s"(s1), "s"(s2), "s"(s3) : "memory", RW_CLOB_ALL);
    else asm volatile(RW_OWN_LOADS(1) :: "v"(voff), "s"(rsrc), "s"(s0), "s"(s1), "s"(s2), "s"(s3) : "memory", RW_CLOB_ALL);
#undef RW_OWN_LOADS
}
// the same for a chunk that crosses an end of the operand: element by element, every offset checked by its lane
// (v[k]: byte offset of the lane's row k inside a column, or the out-of-range marker)
template <int P, int COL>
__device__ __forceinline__ void rw_load_own_checked(const unsigned (&v)[8], rw_int4 rsrc)
{
#define RW_OWN_LOADS1(Q, CC) \
    RW_DEFS \
    "s_nop 4\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+0], %0, %8, 0 offen\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+1], %1, %8, 0 offen\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+2], %2, %8, 0 offen\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+3], %3, %8, 0 offen\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+4], %4, %8, 0 offen\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+5], %5, %8, 0 offen\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+6], %6, %8, 0 offen\n" \
    "buffer_load_dword v[RW_OWN" #Q "+8*" #CC "+7], %7, %8, 0 offen\n" \
    RW_PURGE
#define RW_OWN_ARGS "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]), "s"(rsrc)
    if constexpr (P == 0) {
        if constexpr (COL == 0) asm volatile(RW_OWN_LOADS1(0, 0) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
        if constexpr (COL == 1) asm volatile(RW_OWN_LOADS1(0, 1) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
        if constexpr (COL == 2) asm volatile(RW_OWN_LOADS1(0, 2) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
        if constexpr (COL == 3) asm volatile(RW_OWN_LOADS1(0, 3) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
    } else {
        if constexpr (COL == 0) asm volatile(RW_OWN_LOADS1(1, 0) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
        if constexpr (COL == 1) asm volatile(RW_OWN_LOADS1(1, 1) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
        if constexpr (COL == 2) asm volatile(RW_OWN_LOADS1(1, 2) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
        if constexpr (COL == 3) asm volatile(RW_OWN_LOADS1(1, 3) :: RW_OWN_ARGS : "memory", RW_CLOB_ALL);
    }
#undef RW_OWN_ARGS
#undef RW_OWN_LOADS1
}

template <int LCK>
__global__ __launch_bounds__(64 * RW_WAVES) void spmm_rows_kernel(
    const Chunk *__restrict__ chunks, int nchunks, const float *__restrict__ vals, int stride, int ashift,
    int slot_step, const float *__restrict__ X, long long ldx, float *__restrict__ Y, long long ldy,
    int n_out, int n_in, int batch, float alpha, float beta, int col_tiles, unsigned a_bytes)
{
    constexpr int TR = rw_tile_rows(LCK), ABUF = rw_abuf_bytes(LCK), PIECES = 2 * LCK;
    constexpr int PIECE_IT = (PIECES + RW_WAVES - 1) / RW_WAVES;          // pieces of diagonal values a wave fetches per chunk
    __shared__ __attribute__((aligned(16))) unsigned char lds[rw_lds_bytes(LCK)];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = rw_xcd_tile(blockIdx.x, gridDim.x);
    const int rowtile = tile / col_tiles, coltile = tile - rowtile * col_tiles;
    const int row0 = rowtile * TR, col0 = coltile * RW_COLS;
    const int cols_here = min(RW_COLS, batch - col0);

    // The chunks that have rows inside the operand: the table is sorted by shift, so they are a contiguous
    // range.  A chunk's valid rows read the dense rows [a0, a0 + TR + LCK - 1), a0 = row0 + its shift.
    int c_lo = nchunks, c_hi = 0;
    for (int k = 0; k < RW_MAX_CHUNKS; k += 64) {
        if (k >= nchunks) break;
        const int idx = k + lane;
        const int a0 = row0 + chunks[min(idx, nchunks - 1)].s0;
        const bool outside = (a0 + TR + LCK - 1 <= 0) | (a0 >= n_in);
        const unsigned long long m = __builtin_amdgcn_ballot_w64(!outside & (idx < nchunks));
        if (m) {
            c_lo = min(c_lo, k + (int)__builtin_ctzll(m));
            c_hi = max(c_hi, k + 64 - (int)__builtin_clzll(m));
        }
    }
    const int nk = __builtin_amdgcn_readfirstlane(max(c_hi - c_lo, 0));

    const rw_int4 xr_all = rw_rsrc(X + (long long)col0 * ldx, (unsigned)(((long long)(cols_here - 1) * ldx + n_in) * 4));
    const float *xcol0 = X + (long long)col0 * ldx;
    const rw_int4 ar = rw_rsrc(vals, a_bytes);
    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned char *)&lds[0];
    const unsigned a_read_addr = lds0 + 16u * (unsigned)lane;
    const unsigned x_voff = 32u * (unsigned)lane;
    // the wave's columns (one past the batch is replaced by the last valid one: its sums are never stored)
    unsigned colb[RW_C];
#pragma unroll
    for (int c = 0; c < RW_C; ++c)
        colb[c] = __builtin_amdgcn_readfirstlane((unsigned)min(RW_C * wave + c, cols_here - 1) * ((unsigned)ldx * 4u));
    // Diagonal values: a chunk's diagonals sit at evenly spaced table positions, slot_step apart (negative for the
    // transposed product of a table listed in ascending order), and for the transposed product a value is
    // indexed by its INPUT row, one further per diagonal.  A lane reaches diagonal j of a chunk through a
    // non-negative byte offset from the chunk's first diagonal in memory: diagonal 0 when slot_step > 0, the
    // last one otherwise.
    const bool ascending = slot_step > 0;
    const unsigned dj = ascending ? ((unsigned)slot_step * (unsigned)stride + (unsigned)ashift) * 4u
                                  : ((unsigned)(-slot_step) * (unsigned)stride - (unsigned)ashift) * 4u;
    unsigned a_voff[PIECE_IT];
#pragma unroll
    for (int it = 0; it < PIECE_IT; ++it) {
        const int pw = wave + RW_WAVES * it;                              // piece 2 j + half
        const int j = pw >> 1;
        a_voff[it] = (unsigned)(ascending ? j : LCK - 1 - j) * dj + (unsigned)(8 * lane + 4 * (pw & 1)) * 4u;
    }

    typedef const int __attribute__((address_space(4))) *sc_int_ptr;
    // requests chunk number i of the walk into value buffer / own set `par`
    auto issue = [&](int i, auto par_c) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        const sc_int_ptr e = (sc_int_ptr)(chunks + c_lo + i);
        const int s0 = e[0], slot0 = e[2];
        const int a0 = row0 + s0;
        const unsigned abuf = lds0 + (unsigned)(PAR * ABUF);
        const bool fast = (a0 >= 0) & (a0 + RW_LOADED + LCK - 1 <= n_in) & (row0 + RW_LOADED <= n_out);
        if (fast) {
            const int slot_first = ascending ? slot0 : slot0 + (LCK - 1) * slot_step;      // the first in memory
            const int in_first = ashift ? s0 + (ascending ? 0 : LCK - 1) : 0;
            const unsigned soff = ((unsigned)slot_first * (unsigned)stride + (unsigned)(row0 + in_first)) * 4u;
#pragma unroll
            for (int it = 0; it < PIECE_IT; ++it) {
                const int pw = wave + RW_WAVES * it;
                if (pw < PIECES) rw_lds_load_b128(ar, abuf + 1024u * (unsigned)pw, a_voff[it], soff);
            }
            const unsigned a0b = (unsigned)a0 * 4u;
            rw_load_own<PAR>(x_voff, xr_all, colb[0] + a0b, colb[1] + a0b, colb[2] + a0b, colb[3] + a0b);
        } else {
            // element by element: a value whose input row does not exist is padding and becomes 0, as does a
            // dense row outside the operand
#pragma unroll
            for (int it = 0; it < PIECE_IT; ++it) {
                const int pw = wave + RW_WAVES * it;
                if (pw < PIECES) {
                    const int j = pw >> 1, half = pw & 1;
                    const unsigned dbase = ((unsigned)(slot0 + j * slot_step) * (unsigned)stride) * 4u;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int o = row0 + 8 * (16 * q + (lane >> 2)) + 4 * half + (lane & 3);
                        const int in = o + s0 + j;
                        const bool ok = ((unsigned)in < (unsigned)n_in) & (o < n_out);
                        rw_lds_load_b32(ar, abuf + 1024u * (unsigned)pw + 256u * (unsigned)q,
                                        ok ? dbase + (unsigned)(ashift ? in : o) * 4u : RW_OOB);
                    }
                }
            }
            unsigned v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int r = a0 + 8 * lane + k;
                v[k] = (unsigned)r < (unsigned)n_in ? (unsigned)r * 4u : RW_OOB;
            }
            // (the range check of a buffer load counts the scalar offset in: every column gets a resource of its
            // own that ends with the column's last row)
            rw_load_own_checked<PAR, 0>(v, rw_rsrc(xcol0 + colb[0] / 4u, (unsigned)n_in * 4u));
            rw_load_own_checked<PAR, 1>(v, rw_rsrc(xcol0 + colb[1] / 4u, (unsigned)n_in * 4u));
            rw_load_own_checked<PAR, 2>(v, rw_rsrc(xcol0 + colb[2] / 4u, (unsigned)n_in * 4u));
            rw_load_own_checked<PAR, 3>(v, rw_rsrc(xcol0 + colb[3] / 4u, (unsigned)n_in * 4u));
        }
    };
    auto top = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory", RW_CLOB_ALL); };
    auto compute = [&](auto par_c) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        if (wave < 4) rw_compute<LCK, PAR, 0>(a_read_addr);
        else rw_compute<LCK, PAR, 1>(a_read_addr);
    };

    asm volatile(RW_DEFS ".irp i,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16,17,18,19,20,21,22,23,24,25,26,27,28,29,30,31\n"
                         " v_mov_b32 v[RW_ACC+\\i], 0\n.endr\n" RW_PURGE ::: RW_CLOB_ALL);
    if (nk > 0) issue(0, std::integral_constant<int, 0>{});
    for (int i = 0; i < nk; i += 2) {
        top();
        if (i + 1 < nk) issue(i + 1, std::integral_constant<int, 1>{});
        compute(std::integral_constant<int, 0>{});
        if (i + 1 >= nk) break;
        top();
        if (i + 2 < nk) issue(i + 2, std::integral_constant<int, 0>{});
        compute(std::integral_constant<int, 1>{});
    }

    // The sums leave through LDS so that a column's rows go to memory in 16-byte pieces, lane after lane: every
    // wave writes its 4 x 512 sums to its own 8 KB (column c at 2 KB c, the lane's 8 rows at 32 bytes x lane)
    // and reads back rows 4 l .. 4 l + 3 and 256 + 4 l .. of each column.
    __syncthreads();                                // every wave is through with the value buffers
    const unsigned out_addr = lds0 + 8192u * (unsigned)wave + 32u * (unsigned)lane;
    asm volatile(RW_DEFS
                 ".irp c,0,1,2,3\n"
                 " ds_write_b128 %0, v[RW_ACC+8*\\c:RW_ACC+8*\\c+3] offset:2048*\\c\n"
                 " ds_write_b128 %0, v[RW_ACC+8*\\c+4:RW_ACC+8*\\c+7] offset:2048*\\c+16\n"
                 ".endr\n"
                 "s_waitcnt lgkmcnt(0)\n" RW_PURGE :: "v"(out_addr) : "memory", RW_CLOB_ALL);
    __builtin_amdgcn_wave_barrier();
    const float *outw = reinterpret_cast<const float *>(&lds[0]) + 2048 * wave;
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
#pragma unroll
    for (int c = 0; c < RW_C; ++c) {
        const int col = col0 + RW_C * wave + c;
        if (col >= batch) break;                    // wave-uniform
        float *ycol = Y + (long long)col * ldy;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int r = 256 * hh + 4 * lane;      // row within the tile
            const float4 s = *reinterpret_cast<const float4 *>(outw + 512 * c + r);
            const long long row = (long long)row0 + r;
            const float sv[4] = {s.x, s.y, s.z, s.w};
            if (r + 3 < TR && row + 3 < n_out) {
                float o[4];
                if (beta == 0.f) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = alpha * sv[e];
                } else {
                    const f4u y = *reinterpret_cast<const f4u *>(ycol + row);
                    const float yv[4] = {y.x, y.y, y.z, y.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = __builtin_fmaf(beta, yv[e], alpha * sv[e]);
                }
                __builtin_nontemporal_store(f4u{o[0], o[1], o[2], o[3]}, reinterpret_cast<f4u *>(ycol + row));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (r + e < TR && row + e < n_out) {
                        const float o = beta == 0.f ? alpha * sv[e] : __builtin_fmaf(beta, ycol[row + e], alpha * sv[e]);
                        __builtin_nontemporal_store(o, ycol + row + e);
                    }
                }
            }
        }
    }
}

}  // namespace

// What the rows-along-lanes kernel serves: row_fact 1, a table all of whose chunks have LCK = 7 or 13 diagonals
// at evenly spaced table positions, operands within 32-bit byte offsets.
bool spmm_rows_ok(const DiaView &A, long long ldb, long long ldd, bool trans)
{
    const long long n_in = trans ? A.h : A.w;
    const int lck = trans ? A.max_len_t : A.max_len_n, lck_min = trans ? A.min_len_t : A.min_len_n;
    const int nchunks = trans ? A.n_chunks_t : A.n_chunks_n;
    const int step = trans ? A.slot_step_t : A.slot_step_n;
    const long long x_bytes = ((RW_COLS - 1) * ldb + n_in) * 4;
    const long long a_bytes = (long long)A.nd * A.stride * 4;
    if (A.rf != 1 || (lck != 7 && lck != 13) || lck_min != lck || step == 0 || nchunks > RW_MAX_CHUNKS) return false;
    // values are indexed by a row of the matrix (the output row, or the input row of the transposed product):
    // with every diagonal as long as the matrix has rows, a tile's 512 rows of a diagonal stay inside the array
    if (A.stride < A.h) return false;
    if (x_bytes >= (long long)RW_OOB || a_bytes >= (long long)RW_OOB || n_in * 4 >= (long long)RW_OOB) return false;
    // a chunk's diagonals are reached from its first one through a 32-bit byte offset per lane
    if (((long long)(step < 0 ? -step : step) * A.stride + 1) * 4 * lck + 4096 >= (long long)RW_OOB) return false;
    return true;
}

int spmm_rows_tile_rows(int lck) { return rw_tile_rows(lck); }

hipError_t launch_spmm_rows(const DiaView &A, const float *vals, const float *B, long long ldb,
                            float *dst, long long ldd, int batch, bool trans,
                            float alpha, float beta, hipStream_t stream)
{
    const int n_out = trans ? A.w : A.h, n_in = trans ? A.h : A.w;
    const int lck = trans ? A.max_len_t : A.max_len_n;
    const long long row_tiles = (n_out + rw_tile_rows(lck) - 1) / rw_tile_rows(lck);
    const long long col_tiles = (batch + RW_COLS - 1) / RW_COLS;
    if (row_tiles * col_tiles > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(row_tiles * col_tiles));
#define RW_ARGS trans ? A.chunks_t_dev : A.chunks_n_dev, trans ? A.n_chunks_t : A.n_chunks_n, vals, A.stride, trans ? 1 : 0, \
                trans ? A.slot_step_t : A.slot_step_n, B, ldb, dst, ldd, n_out, n_in, batch, alpha, beta, (int)col_tiles, \
                (unsigned)((long long)A.nd * A.stride * 4)
    if (lck == 7) hipLaunchKernelGGL((spmm_rows_kernel<7>), grid, dim3(64 * RW_WAVES), 0, stream, RW_ARGS);
    else if (lck == 13) hipLaunchKernelGGL((spmm_rows_kernel<13>), grid, dim3(64 * RW_WAVES), 0, stream, RW_ARGS);
    else return hipErrorNotSupported;
#undef RW_ARGS
    return hipGetLastError();
}

}  // namespace cuvdia
