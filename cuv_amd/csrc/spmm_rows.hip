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
//     (v44 and up; the compiler's own values stay below, which the build checks);
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
constexpr int RW_MAX_CHUNKS = 64;         // the walk keeps table entry l in lane l

constexpr int rw_valid_lanes(int lck) { return 64 - (lck - 1 + RW_T - 1) / RW_T; }
constexpr int rw_tile_rows(int lck) { return RW_T * rw_valid_lanes(lck); }
// LDS: three buffers of diagonal values (and a spare kilobyte behind them), 2 x lck pieces of 1 KB each (piece 2 j + half: lane l's rows
// 8 l + 4 half .. + 3 of diagonal j at byte 16 l); at the end every wave passes its 4 x 512 sums through 8 KB.
constexpr int rw_abuf_bytes(int lck) { return 2 * lck * 1024; }
constexpr int rw_lds_bytes(int lck) { return 3 * rw_abuf_bytes(lck) + 1024 > RW_WAVES * 8192 ? 3 * rw_abuf_bytes(lck) + 1024 : RW_WAVES * 8192; }

// ---- the named registers --------------------------------------------------------------------------------
//   v44 ..  v75   own dense rows, set 2: RW_OWN2 + 8 c + k (the compiler's own values stay below v44: the
//                 build checks the disassembly for that)
//   v78 ..  v111  four buffers of 8 diagonal values (RW_A0, RW_A1: first register 2 mod 4; RW_A2, RW_A3: 0 mod 4)
//   v112 .. v143  sums, RW_ACC + 8 c + t
//   v144 .. v175  own dense rows, set 0: RW_OWN0 + 8 c + k      (window positions 0 .. 7)
//   v176 .. v207  own dense rows, set 1 (chunk i uses set i mod 3 while the sets of chunks i + 1 and i + 2 load)
//   v208 .. v255  halo: RW_HALO + 12 c + m                      (window positions 8 + m)
// Every statement begins with RW_DEFS (symbols and macros are per statement: the assembler keeps macros for the
// whole translation unit, and a statement can be instantiated more than once) and ends with RW_PURGE.  The
// statement sets RW_P (the own set of the chunk being computed), RW_Q (the set being loaded) and RW_LCK first.
#define RW_DEFS \
    ".set RW_A0, 78\n.set RW_A1, 86\n.set RW_A2, 96\n.set RW_A3, 104\n" \
    ".set RW_ACC, 112\n.set RW_OWN0, 144\n.set RW_OWN1, 176\n.set RW_OWN2, 44\n.set RW_HALO, 208\n" \
    ".macro RW_SETS p, q\n" \
    " .if \\p == 0\n .set RW_OWNP, RW_OWN0\n .endif\n .if \\p == 1\n .set RW_OWNP, RW_OWN1\n .endif\n .if \\p == 2\n .set RW_OWNP, RW_OWN2\n .endif\n" \
    " .if \\q == 0\n .set RW_OWNQ, RW_OWN0\n .endif\n .if \\q == 1\n .set RW_OWNQ, RW_OWN1\n .endif\n .if \\q == 2\n .set RW_OWNQ, RW_OWN2\n .endif\n" \
    ".endm\n" \
    ".macro RW_FMAD j, ab\n" \
    " .irp c,0,1,2,3\n" \
    "  .irp t,0,1,2,3,4,5,6,7\n" \
    "   .if (\\t+\\j) < 8\n" \
    "     v_fmac_f32 v[RW_ACC+8*\\c+\\t], v[\\ab+\\t], v[RW_OWNP+8*\\c+\\t+\\j]\n" \
    "   .else\n" \
    "     v_fmac_f32 v[RW_ACC+8*\\c+\\t], v[\\ab+\\t], v[RW_HALO+12*\\c+\\t+\\j-8]\n" \
    "   .endif\n" \
    "  .endr\n" \
    " .endr\n" \
    ".endm\n" \
    ".macro RW_HALOS n\n" \
    " .irp c,0,1,2,3\n" \
    "  .irp k,0,1,2,3,4,5,6,7\n" \
    "   .if \\k < \\n\n" \
    "   v_mov_b32_dpp v[RW_HALO+12*\\c+\\k], v[RW_OWNP+8*\\c+\\k] wave_shl:1 row_mask:0xf bank_mask:0xf\n" \
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
    ".macro RW_AREAD ab, j, vaddr\n" \
    "  ds_read_b128 v[\\ab:\\ab+3], \\vaddr offset:\\j*2048\n" \
    "  ds_read_b128 v[\\ab+4:\\ab+7], \\vaddr offset:\\j*2048+1024\n" \
    ".endm\n" \
    ".macro RW_AREADJ j, vaddr\n" \
    " .if ((\\j) & 3) == 0\n RW_AREAD RW_A0, (\\j), \\vaddr\n .endif\n" \
    " .if ((\\j) & 3) == 1\n RW_AREAD RW_A1, (\\j), \\vaddr\n .endif\n" \
    " .if ((\\j) & 3) == 2\n RW_AREAD RW_A2, (\\j), \\vaddr\n .endif\n" \
    " .if ((\\j) & 3) == 3\n RW_AREAD RW_A3, (\\j), \\vaddr\n .endif\n" \
    ".endm\n" \
    ".macro RW_FMADJ j\n" \
    " .if ((\\j) & 3) == 0\n RW_FMAD \\j, RW_A0\n .endif\n" \
    " .if ((\\j) & 3) == 1\n RW_FMAD \\j, RW_A1\n .endif\n" \
    " .if ((\\j) & 3) == 2\n RW_FMAD \\j, RW_A2\n .endif\n" \
    " .if ((\\j) & 3) == 3\n RW_FMAD \\j, RW_A3\n .endif\n" \
    ".endm\n" \
    ".macro RW_XLOAD n, voff, rsrc, soff\n" \
    " .if ((\\n) & 1) == 0\n" \
    "  buffer_load_dwordx4 v[RW_OWNQ+4*(\\n):RW_OWNQ+4*(\\n)+3], \\voff, \\rsrc, \\soff offen\n" \
    " .else\n" \
    "  buffer_load_dwordx4 v[RW_OWNQ+4*(\\n):RW_OWNQ+4*(\\n)+3], \\voff, \\rsrc, \\soff offen offset:16\n" \
    " .endif\n" \
    ".endm\n"
#define RW_PURGE ".purgem RW_SETS\n.purgem RW_FMAD\n.purgem RW_HALOS\n.purgem RW_AREAD\n.purgem RW_AREADJ\n.purgem RW_FMADJ\n.purgem RW_XLOAD\n"

#define RW_CLOB_OWN2 "v44","v45","v46","v47","v48","v49","v50","v51","v52","v53","v54","v55","v56","v57","v58","v59","v60","v61","v62","v63","v64","v65","v66","v67","v68","v69","v70","v71","v72","v73","v74","v75"
#define RW_CLOB_A "v78","v79","v80","v81","v82","v83","v84","v85","v86","v87","v88","v89","v90","v91","v92","v93","v94","v95","v96","v97","v98","v99","v100","v101","v102","v103","v104","v105","v106","v107","v108","v109","v110","v111"
#define RW_CLOB_ACC "v112","v113","v114","v115","v116","v117","v118","v119","v120","v121","v122","v123","v124","v125","v126","v127","v128","v129","v130","v131","v132","v133","v134","v135","v136","v137","v138","v139","v140","v141","v142","v143"
#define RW_CLOB_OWN0 "v144","v145","v146","v147","v148","v149","v150","v151","v152","v153","v154","v155","v156","v157","v158","v159","v160","v161","v162","v163","v164","v165","v166","v167","v168","v169","v170","v171","v172","v173","v174","v175"
#define RW_CLOB_OWN1 "v176","v177","v178","v179","v180","v181","v182","v183","v184","v185","v186","v187","v188","v189","v190","v191","v192","v193","v194","v195","v196","v197","v198","v199","v200","v201","v202","v203","v204","v205","v206","v207"
#define RW_CLOB_HALO "v208","v209","v210","v211","v212","v213","v214","v215","v216","v217","v218","v219","v220","v221","v222","v223","v224","v225","v226","v227","v228","v229","v230","v231","v232","v233","v234","v235","v236","v237","v238","v239","v240","v241","v242","v243","v244","v245","v246","v247","v248","v249","v250","v251","v252","v253","v254","v255"
#define RW_CLOB_ALL RW_CLOB_OWN2, RW_CLOB_A, RW_CLOB_ACC, RW_CLOB_OWN0, RW_CLOB_OWN1, RW_CLOB_HALO

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

// What a wave needs to request a chunk's operands: the dense rows of its 4 columns (8 loads of 16 bytes per
// lane into own set Q, the column in the lane's byte offset) and its share of the chunk's diagonal values (NP
// loads that write LDS directly).
struct RwRequest {
    rw_int4 xr;                 // dense operand of the tile's columns (an empty resource: nothing is fetched, zeros arrive)
    unsigned xs;                // scalar byte offset of the chunk's first dense row
    rw_int4 ar;                 // the diagonal values (or the empty resource)
    unsigned as;                // scalar byte offset of the chunk's first diagonal, at the tile's first row
    unsigned m0_base;           // LDS byte address of the wave's first piece in the value buffer
    unsigned m0_last;           // .. of its last piece (the spare kilobyte where the wave has none)
};

// One diagonal of a chunk: the values of the diagonal after the next are read from LDS, this one's are waited for, the
// two waves of a SIMD trade priority, a load or two of the chunk two steps ahead are issued, then 32 FMAs.
// (requests per diagonal: chunks of 13 -- one per diagonal, the 8 dense loads first, then the pieces of
// diagonal values; chunks of 7 -- two dense loads on each of the first four diagonals, a piece on the next two)
#define RW_DIAG(J) \
    ".if " #J " < RW_LCK\n" \
    " .if " #J " + 2 < RW_LCK\n RW_AREADJ (" #J "+2), %[aread]\n s_waitcnt lgkmcnt(4)\n .else\n  .if " #J " + 1 < RW_LCK\n s_waitcnt lgkmcnt(2)\n  .else\n s_waitcnt lgkmcnt(0)\n  .endif\n .endif\n" \
    " .if ((" #J " ^ RW_WPAR) & 1)\n s_setprio 0\n .else\n s_setprio 3\n .endif\n" \
    " .if RW_LCK > 8\n" \
    "  .if " #J " == 0\n RW_XLOAD 0, %[xv0], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 1\n RW_XLOAD 1, %[xv0], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 2\n RW_XLOAD 2, %[xv1], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 3\n RW_XLOAD 3, %[xv1], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 4\n RW_XLOAD 4, %[xv2], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 5\n RW_XLOAD 5, %[xv2], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 6\n RW_XLOAD 6, %[xv3], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 7\n RW_XLOAD 7, %[xv3], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 8\n s_mov_b32 m0, %[m0base]\n s_nop 0\n buffer_load_dwordx4 %[av0], %[ars], %[asoff] offen lds\n .endif\n" \
    "  .if " #J " == 9\n s_add_u32 m0, %[m0base], 8192\n s_nop 0\n buffer_load_dwordx4 %[av1], %[ars], %[asoff] offen lds\n .endif\n" \
    "  .if " #J " == 10\n s_add_u32 m0, %[m0base], 16384\n s_nop 0\n buffer_load_dwordx4 %[av2], %[ars], %[asoff] offen lds\n .endif\n" \
    "  .if " #J " == 11\n s_mov_b32 m0, %[m0last]\n s_nop 0\n buffer_load_dwordx4 %[av3], %[ars], %[asoff] offen lds\n .endif\n" \
    " .else\n" \
    "  .if " #J " == 0\n RW_XLOAD 0, %[xv0], %[xrs], %[xs]\n RW_XLOAD 1, %[xv0], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 1\n RW_XLOAD 2, %[xv1], %[xrs], %[xs]\n RW_XLOAD 3, %[xv1], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 2\n RW_XLOAD 4, %[xv2], %[xrs], %[xs]\n RW_XLOAD 5, %[xv2], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 3\n RW_XLOAD 6, %[xv3], %[xrs], %[xs]\n RW_XLOAD 7, %[xv3], %[xrs], %[xs]\n .endif\n" \
    "  .if " #J " == 4\n s_mov_b32 m0, %[m0base]\n s_nop 0\n buffer_load_dwordx4 %[av0], %[ars], %[asoff] offen lds\n .endif\n" \
    "  .if " #J " == 5\n s_mov_b32 m0, %[m0last]\n s_nop 0\n buffer_load_dwordx4 %[av1], %[ars], %[asoff] offen lds\n .endif\n" \
    " .endif\n" \
    " RW_FMADJ " #J "\n" \
    ".endif\n"
#define RW_CHUNK \
    RW_DEFS ".set RW_LCK, %[lck]\n.set RW_WPAR, %[wpar]\n RW_SETS %[p], %[q]\n" \
    "s_nop 4\n" \
    "RW_AREADJ 0, %[aread]\n RW_AREADJ 1, %[aread]\n RW_HALOS (RW_LCK-1)\n" \
    RW_DIAG(0) RW_DIAG(1) RW_DIAG(2) RW_DIAG(3) RW_DIAG(4) RW_DIAG(5) RW_DIAG(6) \
    RW_DIAG(7) RW_DIAG(8) RW_DIAG(9) RW_DIAG(10) RW_DIAG(11) RW_DIAG(12) \
    "s_setprio 0\n" RW_PURGE

// loads a wave issues per chunk (the same for every wave, so that the waits count exactly)
constexpr int rw_pieces_per_wave(int lck) { return (2 * lck + RW_WAVES - 1) / RW_WAVES; }
constexpr int rw_loads_per_chunk(int lck) { return 2 * RW_C + rw_pieces_per_wave(lck); }

// The arithmetic of the chunk whose operands sit in own set P and in the value buffer at a_read_addr, and the
// requests for the chunk two steps ahead (own set (P + 2) % 3) spread between its diagonals.
template <int LCK, int P, int WPAR>
__device__ __forceinline__ void rw_compute(unsigned a_read_addr, const unsigned (&x_voff)[RW_C], const unsigned (&a_voff)[4], const RwRequest &rq)
{
    static_assert(LCK == 7 || LCK == 13, "instantiated chunk lengths");
    asm volatile(RW_CHUNK
                 :: [aread] "v"(a_read_addr), [xv0] "v"(x_voff[0]), [xv1] "v"(x_voff[1]), [xv2] "v"(x_voff[2]), [xv3] "v"(x_voff[3]),
                    [xrs] "s"(rq.xr), [xs] "s"(rq.xs), [ars] "s"(rq.ar), [asoff] "s"(rq.as), [av0] "v"(a_voff[0]),
                    [av1] "v"(a_voff[1]), [av2] "v"(a_voff[2]), [av3] "v"(a_voff[3]), [m0base] "s"(rq.m0_base),
                    [m0last] "s"(rq.m0_last), [p] "n"(P), [q] "n"((P + 2) % 3), [wpar] "n"(WPAR), [lck] "n"(LCK)
                 : "memory", "scc", RW_CLOB_ALL);
}

// The same requests all at once (the first two chunks of a tile, before any arithmetic).
template <int LCK, int Q>
__device__ __forceinline__ void rw_request_now(const unsigned (&x_voff)[RW_C], const unsigned (&a_voff)[4], const RwRequest &rq)
{
    asm volatile(RW_DEFS "RW_SETS %[q], %[q]\n s_nop 4\n"
                 "RW_XLOAD 0, %[xv0], %[xrs], %[xs]\n RW_XLOAD 1, %[xv0], %[xrs], %[xs]\n"
                 "RW_XLOAD 2, %[xv1], %[xrs], %[xs]\n RW_XLOAD 3, %[xv1], %[xrs], %[xs]\n"
                 "RW_XLOAD 4, %[xv2], %[xrs], %[xs]\n RW_XLOAD 5, %[xv2], %[xrs], %[xs]\n"
                 "RW_XLOAD 6, %[xv3], %[xrs], %[xs]\n RW_XLOAD 7, %[xv3], %[xrs], %[xs]\n"
                 ".if %[lck] > 8\n"
                 " s_mov_b32 m0, %[m0base]\n s_nop 0\n buffer_load_dwordx4 %[av0], %[ars], %[asoff] offen lds\n"
                 " s_add_u32 m0, %[m0base], 8192\n s_nop 0\n buffer_load_dwordx4 %[av1], %[ars], %[asoff] offen lds\n"
                 " s_add_u32 m0, %[m0base], 16384\n s_nop 0\n buffer_load_dwordx4 %[av2], %[ars], %[asoff] offen lds\n"
                 " s_mov_b32 m0, %[m0last]\n s_nop 0\n buffer_load_dwordx4 %[av3], %[ars], %[asoff] offen lds\n"
                 ".else\n"
                 " s_mov_b32 m0, %[m0base]\n s_nop 0\n buffer_load_dwordx4 %[av0], %[ars], %[asoff] offen lds\n"
                 " s_mov_b32 m0, %[m0last]\n s_nop 0\n buffer_load_dwordx4 %[av1], %[ars], %[asoff] offen lds\n"
                 ".endif\n" RW_PURGE
                 :: [xv0] "v"(x_voff[0]), [xv1] "v"(x_voff[1]), [xv2] "v"(x_voff[2]), [xv3] "v"(x_voff[3]),
                    [xrs] "s"(rq.xr), [xs] "s"(rq.xs), [ars] "s"(rq.ar), [asoff] "s"(rq.as), [av0] "v"(a_voff[0]),
                    [av1] "v"(a_voff[1]), [av2] "v"(a_voff[2]), [av3] "v"(a_voff[3]), [m0base] "s"(rq.m0_base),
                    [m0last] "s"(rq.m0_last), [q] "n"(Q), [lck] "n"(LCK)
                 : "memory", "scc", RW_CLOB_ALL);
}

// the dense rows of one column of a chunk that crosses an end of the operand: element by element, every offset
// checked by its lane (v[k]: byte offset of the lane's row k inside the column, or the out-of-range marker)
template <int Q, int COL>
__device__ __forceinline__ void rw_load_own_checked(const unsigned (&v)[8], rw_int4 rsrc)
{
    asm volatile(RW_DEFS "RW_SETS %[q], %[q]\n s_nop 4\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+0], %[v0], %[rs], 0 offen\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+1], %[v1], %[rs], 0 offen\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+2], %[v2], %[rs], 0 offen\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+3], %[v3], %[rs], 0 offen\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+4], %[v4], %[rs], 0 offen\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+5], %[v5], %[rs], 0 offen\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+6], %[v6], %[rs], 0 offen\n"
                 "buffer_load_dword v[RW_OWNQ+8*%[c]+7], %[v7], %[rs], 0 offen\n" RW_PURGE
                 :: [v0] "v"(v[0]), [v1] "v"(v[1]), [v2] "v"(v[2]), [v3] "v"(v[3]), [v4] "v"(v[4]), [v5] "v"(v[5]),
                    [v6] "v"(v[6]), [v7] "v"(v[7]), [rs] "s"(rsrc), [q] "n"(Q), [c] "n"(COL)
                 : "memory", RW_CLOB_ALL);
}

template <int LCK>
__global__ __launch_bounds__(64 * RW_WAVES) void spmm_rows_kernel(
    const Chunk *__restrict__ chunks, int nchunks, const float *__restrict__ vals, int stride, int ashift,
    int slot_step, const float *__restrict__ X, long long ldx, float *__restrict__ Y, long long ldy,
    int n_out, int n_in, int batch, float alpha, float beta, int col_tiles, unsigned a_bytes)
{
    constexpr int TR = rw_tile_rows(LCK), ABUF = rw_abuf_bytes(LCK), PIECES = 2 * LCK;
    constexpr int NP = rw_pieces_per_wave(LCK);                           // pieces of diagonal values a wave fetches per chunk
    constexpr int NLOADS = rw_loads_per_chunk(LCK);
    constexpr unsigned DUMP = 3u * ABUF;                                  // a spare kilobyte behind the three value buffers
    static_assert(NP == (LCK > 8 ? 4 : 2), "the statements above issue this many pieces");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = rw_xcd_tile(blockIdx.x, gridDim.x);
    const int rowtile = tile / col_tiles, coltile = tile - rowtile * col_tiles;
    const int row0 = rowtile * TR, col0 = coltile * RW_COLS;
    const int cols_here = min(RW_COLS, batch - col0);

    // The chunks that have rows inside the operand: the table is sorted by shift, so they are a contiguous
    // range.  A chunk's valid rows read the dense rows [a0, a0 + TR + LCK - 1), a0 = row0 + its shift.
    // Lane l keeps what the walk needs of table entry l, ready-made, so that a step reads the entry of the
    // chunk it requests with three v_readlane and the two waves of a SIMD spend next to nothing between two
    // chunks' arithmetic (whatever one of them does there, the other runs alone, at half the rate).
    const Chunk *mine = chunks + min(lane, nchunks - 1);
    const int tab_s0 = mine->s0, tab_slot0 = mine->slot[0];
    int c_lo = nchunks, c_hi = 0;
    {
        const int a0 = row0 + tab_s0;
        const bool outside = (a0 + TR + LCK - 1 <= 0) | (a0 >= n_in);
        const unsigned long long m = __builtin_amdgcn_ballot_w64(!outside & (lane < nchunks));
        if (m) {
            c_lo = (int)__builtin_ctzll(m);
            c_hi = 64 - (int)__builtin_clzll(m);
        }
    }
    const int nk = __builtin_amdgcn_readfirstlane(max(c_hi - c_lo, 0));
    c_lo = __builtin_amdgcn_readfirstlane(c_lo);

    const float *xcol0 = X + (long long)col0 * ldx;
    const rw_int4 xr_all = rw_rsrc(xcol0, (unsigned)(((long long)(cols_here - 1) * ldx + n_in) * 4));
    const rw_int4 ar_all = rw_rsrc(vals, a_bytes);
    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned char *)&lds[0];
    const unsigned a_read_addr = lds0 + 16u * (unsigned)lane;
    // the wave's columns (one past the batch is replaced by the last valid one: its sums are never stored); a
    // lane's byte offset inside the tile's dense operand is its column's first row + its own 8 rows
    auto column_bytes = [&](int c) __attribute__((always_inline)) {
        return (unsigned)min(RW_C * wave + c, cols_here - 1) * ((unsigned)ldx * 4u);
    };
    unsigned x_voff[RW_C];
#pragma unroll
    for (int c = 0; c < RW_C; ++c) x_voff[c] = column_bytes(c) + 32u * (unsigned)lane;
    // Diagonal values: a chunk's diagonals sit at evenly spaced table positions, slot_step apart (negative for the
    // transposed product of a table listed in ascending order), and for the transposed product a value is
    // indexed by its INPUT row, one further per diagonal.  A lane reaches diagonal j of a chunk through a
    // non-negative byte offset from the chunk's first diagonal in memory: diagonal 0 when slot_step > 0, the
    // last one otherwise.  Piece 2 j + half (the rows 8 l + 4 half .. of diagonal j) is fetched by wave
    // (2 j + half) % 8; a wave without a last piece asks for nothing (out-of-range marker) into the spare kilobyte.
    const bool ascending = slot_step > 0;
    const unsigned dj = ascending ? ((unsigned)slot_step * (unsigned)stride + (unsigned)ashift) * 4u
                                  : ((unsigned)(-slot_step) * (unsigned)stride - (unsigned)ashift) * 4u;
    unsigned a_voff[4];
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int pw = wave + RW_WAVES * it;                              // piece 2 j + half
        const int j = pw >> 1;
        a_voff[it] = (it < NP && pw < PIECES) ? (unsigned)(ascending ? j : LCK - 1 - j) * dj + (unsigned)(8 * lane + 4 * (pw & 1)) * 4u
                                              : RW_OOB;
    }
    const bool has_last = wave + RW_WAVES * (NP - 1) < PIECES;
    const unsigned m0_wave = lds0 + 1024u * (unsigned)wave;

    // Table entry l as lane l holds it: can the chunk be requested with whole 16-byte pieces (its 512 rows of
    // every column and of every diagonal exist), and if so the scalar byte offsets of its first dense row and of
    // its first diagonal in memory at the tile's first row.
    int tab_whole;
    unsigned tab_xs, tab_as;
    {
        const int a0 = row0 + tab_s0;
        const bool w = (a0 >= 0) & (a0 + RW_LOADED + LCK - 1 <= n_in) & (row0 + RW_LOADED <= n_out);
        const int slot_first = ascending ? tab_slot0 : tab_slot0 + (LCK - 1) * slot_step;
        const int in_first = ashift ? tab_s0 + (ascending ? 0 : LCK - 1) : 0;
        tab_whole = w ? 1 : 0;
        tab_xs = w ? (unsigned)a0 * 4u : 0u;
        tab_as = w ? ((unsigned)slot_first * (unsigned)stride + (unsigned)(row0 + in_first)) * 4u : 0u;
    }
    // The requests of chunk ii of the walk into own set / value buffer q, or -- past the end of the walk, and
    // for a chunk that cannot be requested whole -- the empty resources (the same with a size of 0: every lane
    // is out of range, nothing is fetched, zeros arrive) with scalar offsets of 0.
    struct Next { RwRequest rq; int at; bool checked; };
    RwRequest rq_cur{xr_all, 0u, ar_all, 0u, 0u, 0u};
    auto prepare = [&](int ii, int q) __attribute__((always_inline)) {
        const int at = c_lo + min(ii, max(nk - 1, 0));
        const bool there = ii < nk;
        const bool w = __builtin_amdgcn_readlane(tab_whole, at) != 0;
        const bool real = there && w;
        rq_cur.xr.z = real ? xr_all.z : 0;
        rq_cur.ar.z = real ? ar_all.z : 0;
        rq_cur.xs = real ? (unsigned)__builtin_amdgcn_readlane((int)tab_xs, at) : 0u;
        rq_cur.as = real ? (unsigned)__builtin_amdgcn_readlane((int)tab_as, at) : 0u;
        rq_cur.m0_base = m0_wave + (unsigned)(q * ABUF);
        rq_cur.m0_last = has_last ? rq_cur.m0_base + 8192u * (unsigned)(NP - 1) : lds0 + DUMP;
        return Next{rq_cur, at, there && !w};
    };
    // a chunk that crosses an end of the operand, element by element: a value whose input row does not exist
    // is padding and becomes 0, as does a dense row outside the operand
    auto request_checked = [&](int at, auto q_c) __attribute__((always_inline)) {
        constexpr int Q = decltype(q_c)::value;
        const int s0 = __builtin_amdgcn_readlane(tab_s0, at), slot0 = __builtin_amdgcn_readlane(tab_slot0, at);
        const unsigned abuf = lds0 + (unsigned)(Q * ABUF);
        const int a0 = row0 + s0;
#pragma unroll
        for (int it = 0; it < NP; ++it) {
            const int pw = wave + RW_WAVES * it;
            if (pw < PIECES) {
                const int j = pw >> 1, half = pw & 1;
                const unsigned dbase = ((unsigned)(slot0 + j * slot_step) * (unsigned)stride) * 4u;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int o = row0 + 8 * (16 * q + (lane >> 2)) + 4 * half + (lane & 3);
                    const int in = o + s0 + j;
                    const bool ok = ((unsigned)in < (unsigned)n_in) & (o < n_out);
                    rw_lds_load_b32(ar_all, abuf + 1024u * (unsigned)pw + 256u * (unsigned)q,
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
        rw_load_own_checked<Q, 0>(v, rw_rsrc(xcol0 + column_bytes(0) / 4u, (unsigned)n_in * 4u));
        rw_load_own_checked<Q, 1>(v, rw_rsrc(xcol0 + column_bytes(1) / 4u, (unsigned)n_in * 4u));
        rw_load_own_checked<Q, 2>(v, rw_rsrc(xcol0 + column_bytes(2) / 4u, (unsigned)n_in * 4u));
        rw_load_own_checked<Q, 3>(v, rw_rsrc(xcol0 + column_bytes(3) / 4u, (unsigned)n_in * 4u));
    };

    asm volatile(RW_DEFS ".irp i,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16,17,18,19,20,21,22,23,24,25,26,27,28,29,30,31\n"
                         " v_mov_b32 v[RW_ACC+\\i], 0\n.endr\n" RW_PURGE ::: RW_CLOB_ALL);

    // Chunk i of the walk lives in own set and value buffer i % 3.  Its operands are requested while chunk
    // i - 2 is computed (the first two before anything else), so they have the whole of chunk i - 1 to arrive;
    // a chunk that crosses an end of the operand is requested element by element after chunk i - 2 instead (the
    // statement's own requests then go through the empty resources, so that every wave issues the same number
    // of loads per chunk whatever happens and the waits count exactly).
    bool exact = false;         // the loads in flight behind those of the chunk about to be computed are the NLOADS of one statement
    if (nk > 0) {
        const Next n0 = prepare(0, 0);
        if (!n0.checked) rw_request_now<LCK, 0>(x_voff, a_voff, n0.rq);
        else request_checked(n0.at, std::integral_constant<int, 0>{});
        if (nk > 1) {
            const Next n1 = prepare(1, 1);
            if (!n1.checked) {
                rw_request_now<LCK, 1>(x_voff, a_voff, n1.rq);
                exact = true;
            } else {
                request_checked(n1.at, std::integral_constant<int, 1>{});
            }
        }
    }
    // what the statement of a step requests (chunk i + 2) is prepared one step ahead
    Next nx = prepare(2, 2);
    auto step = [&](int i, auto p_c) __attribute__((always_inline)) {
        constexpr int P = decltype(p_c)::value, Q = (P + 2) % 3;
        // chunk i must be in: everything but the loads issued behind it
        if (exact) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(NLOADS) : "memory", RW_CLOB_ALL);
        else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory", RW_CLOB_ALL);
        const unsigned aread = a_read_addr + (unsigned)(P * ABUF);
        if (wave < 4) rw_compute<LCK, P, 0>(aread, x_voff, a_voff, nx.rq);
        else rw_compute<LCK, P, 1>(aread, x_voff, a_voff, nx.rq);
        exact = true;
        if (nx.checked) {
            request_checked(nx.at, std::integral_constant<int, Q>{});
            exact = false;
        }
        nx = prepare(i + 3, P);
    };
    for (int i = 0; i < nk;) {
        step(i, std::integral_constant<int, 0>{});
        if (++i >= nk) break;
        step(i, std::integral_constant<int, 1>{});
        if (++i >= nk) break;
        step(i, std::integral_constant<int, 2>{});
        ++i;
    }

    // The sums leave through LDS so that a column's rows go to memory in 16-byte pieces, lane after lane: every
    // wave writes its 4 x 512 sums to its own 8 KB (column c at 2 KB c, the lane's 8 rows at 32 bytes x lane)
    // and reads back rows 4 l .. 4 l + 3 and 256 + 4 l .. of each column.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the last statements' requests (empty, but they write LDS)
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
    if (A.rf != 1 || (lck != 7 && lck != 13) || lck_min != lck || step == 0 || nchunks > RW_MAX_CHUNKS) return false;   // (a lane per table entry)
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
    note_kernel("spmm_rows_kernel<%d>", lck);
    if (lck == 7) {
        hipLaunchKernelGGL((spmm_rows_kernel<7>), grid, dim3(64 * RW_WAVES), rw_lds_bytes(7), stream, RW_ARGS);
    } else if (lck == 13) {
        // more LDS than a kernel may use without saying so
        static const hipError_t allowed = hipFuncSetAttribute(reinterpret_cast<const void *>(&spmm_rows_kernel<13>),
                                                              hipFuncAttributeMaxDynamicSharedMemorySize, rw_lds_bytes(13));
        if (allowed != hipSuccess) return allowed;
        hipLaunchKernelGGL((spmm_rows_kernel<13>), grid, dim3(64 * RW_WAVES), rw_lds_bytes(13), stream, RW_ARGS);
    } else {
        return hipErrorNotSupported;
    }
#undef RW_ARGS
    return hipGetLastError();
}

}  // namespace cuvdia
