// A chain of independent mat-vecs of ONE shape in one launch: the steady state of matvec.hip's loop kernel with the whole
// per-layer loop written as one block of gfx950 assembly.
//
// Semantics per layer: rptc_kernels/csrc/rptc_kernels/inference.cu:189-277 of the reference (the op of matvec.hip).
// The decomposition is the loop kernel's: one 16-wave workgroup per CU owns a block of rows and every slab of those rows;
// a wave item is 64 consecutive stream elements; a wave keeps its (at most MAXI) elements of a layer in registers, asked
// for a layer ahead; two activation images and two sets of partial sums take turns, ONE workgroup barrier a layer.
// What is different: when all layers have one shape, everything about a wave's share that the loop kernel works out
// again in every layer (element offsets, lane clamps, which lanes start a row, where the partial sums go, where the
// activations are staged) is worked out once in front of the loop and kept in registers, and the loop body is written
// by hand:
//   * a layer costs a wave: one barrier, three scalar loads (the next layer's stream and activation pointers, the
//     previous layer's output pointer), per element one 16-byte request, the decode block and one LDS store, one or two
//     reloads of the 32 activation registers as sixteen two-dword LDS reads (an LDS read instruction costs the same for
//     4 and for 8 bytes a lane), eight LDS stores for its share of the next activations;
//   * requests and their waits are in one block, so a register with a request in flight is never the compiler's to
//     touch, and the wait in front of a decode is for that element only (`s_waitcnt vmcnt(N)`, N fixed because every
//     wave always makes the same number of requests a layer: a slot without an element asks for one cache line);
//   * LDS layout with fixed strides so that which image / which set of partial sums a layer uses is an immediate
//     offset (the loop is unrolled over the two parities): table [0, 64 KiB), images 32 KiB each, sets 16 KiB each;
//     the ragged last slab sits in the image at the full slabs' stride (slot 32 q + l), so its reload is the same
//     instruction sequence.
// Every sum has a fixed order: outputs are bit-identical from run to run.
//
// Compile-time switches, all off in the library's build, which is the kernel as it was timed (each switch is a variant
// to be timed against it; every one passes the same tests in the CPU wave model): ST_TUNED, four changes to the layer's
// chores (the activation reload without a wait of its own, the rows added by the waves with the fewest elements, the
// next activations staged behind the first element instead of behind the last, a last layer that asks for nothing);
// ST_MFMA, the element's products on the matrix unit instead of 32 two-term dot products; ST_ROLL, the decode block as a
// rolling pipeline of sixteen gathers (both on top of ST_TUNED); ST_NOPRIO, no s_setprio.
#include "matvec_loop.hpp"
#include "rptc_common.hpp"

namespace rptc {

constexpr int kStThreads = 1024, kStWaves = kStThreads / kWave;
constexpr int kStTableBytes = 65536;                       // 256 rows x 64 lane copies of one half2
constexpr int kStImageBytes = 32768;                       // one activation image: up to 8 slabs of 1024 slots
constexpr int kStPartBytes = 16384;                        // one set of partial sums: rows_per_block * (n / 64) floats
constexpr int kStPartBase = kStTableBytes + 2 * kStImageBytes;
constexpr int kStLdsBytes = kStPartBase + 2 * kStPartBytes;
static_assert(kStLdsBytes == kMaxLds, "the layout fills the LDS of a CU");

// ---- registers with fixed numbers: a request's 16 bytes are four consecutive registers, and an asm operand cannot
// name one register of a tuple
// stream elements of a wave: item u in v[80 + 4u : 83 + 4u]; next activations: v[72:75], v[76:79]
// activation pairs of the slab being decoded: slot q in v(96 + q / 2) for even q, v(112 + (q - 1) / 2) for odd q, so
// that slots q and q + 2 are neighbours and one ds_read2st64_b32 (two dwords 256 bytes apart) fills both
#if (defined(ST_MFMA) || defined(ST_ROLL)) && !defined(ST_TUNED)
#define ST_TUNED
#endif
// ST_TUNED is three switches that can be timed one by one: the reload's wait, who adds the rows, and the order of a
// layer's chores (staging behind the first element, a last layer that asks for nothing)
#ifdef ST_TUNED
#define ST_T_RELOAD
#define ST_T_ROWS
#define ST_T_FLOW
#endif
#ifndef ST_MFMA
#define ST_X0 "v96"
#define ST_X2 "v97"
#define ST_X4 "v98"
#define ST_X6 "v99"
#define ST_X8 "v100"
#define ST_X10 "v101"
#define ST_X12 "v102"
#define ST_X14 "v103"
#define ST_X16 "v104"
#define ST_X18 "v105"
#define ST_X20 "v106"
#define ST_X22 "v107"
#define ST_X24 "v108"
#define ST_X26 "v109"
#define ST_X28 "v110"
#define ST_X30 "v111"
#define ST_X1 "v112"
#define ST_X3 "v113"
#define ST_X5 "v114"
#define ST_X7 "v115"
#define ST_X9 "v116"
#define ST_X11 "v117"
#define ST_X13 "v118"
#define ST_X15 "v119"
#define ST_X17 "v120"
#define ST_X19 "v121"
#define ST_X21 "v122"
#define ST_X23 "v123"
#define ST_X25 "v124"
#define ST_X27 "v125"
#define ST_X29 "v126"
#define ST_X31 "v127"

#else
// With the products on the matrix unit (ST_MFMA) an operand is a PAIR of registers: the two windows of one window register
// (slots hi, lo) sit side by side, pair 4 j + i in v[96 + 8 j + 2 i : +1] for shift group j and window register i
#define ST_XP(J, I) "v[96+8*" #J "+2*" #I ":96+8*" #J "+2*" #I "+1]"
#endif
// a wave's priority at the instruction arbiter: highest in front of its first element and in the rows, lower with
// every element it has behind it, so that the waves of a SIMD drift apart instead of queueing at the same unit
#ifndef ST_NOPRIO
#define ST_PRIO(X) "s_setprio " X "\n"
#else
#define ST_PRIO(X) ""
#endif
#define ST_PRIO_OF_0 ST_PRIO("3")
#define ST_PRIO_OF_1 ST_PRIO("2")
#define ST_PRIO_OF_2 ST_PRIO("1")
#define ST_PRIO_OF_3 ST_PRIO("0")
#define ST_PRIO_OF_4 ST_PRIO("0")
#define ST_PRIO_OF_5 ST_PRIO("0")
#define ST_STR2(x) #x
#define ST_STR(x) ST_STR2(x)

// The 32 activation pairs of a lane for one slab: image P (0 / 1), XA = LDS address of the lane's slot 0 in image 0.
#ifndef ST_MFMA
#define ST_RD2(LO, HI, BASE, OFF, P)                                                                                  \
    "ds_read2st64_b32 v[" #LO ":" #HI "], " BASE " offset0:" #P "*128+" #OFF " offset1:" #P "*128+" #OFF "+1\n"
// ST_T_RELOAD: LDS reads complete in order and the decode block's first wait (at most 8 reads in flight, its own) comes
// before its first product, which is the first instruction to read an activation register: the reload then needs no wait
// of its own
#ifdef ST_T_RELOAD
#define ST_RELOAD_WAIT ""
#else
#define ST_RELOAD_WAIT "s_waitcnt lgkmcnt(0)\n"
#endif
#define ST_RELOAD(XA, P)                                                                                              \
    "v_add_u32 %[xb], 0x80, " XA "\n"                                                                                 \
    ST_RD2(96, 97, XA, 0, P) ST_RD2(98, 99, XA, 2, P) ST_RD2(100, 101, XA, 4, P) ST_RD2(102, 103, XA, 6, P)           \
    ST_RD2(104, 105, XA, 8, P) ST_RD2(106, 107, XA, 10, P) ST_RD2(108, 109, XA, 12, P) ST_RD2(110, 111, XA, 14, P)    \
    ST_RD2(112, 113, "%[xb]", 0, P) ST_RD2(114, 115, "%[xb]", 2, P) ST_RD2(116, 117, "%[xb]", 4, P)                   \
    ST_RD2(118, 119, "%[xb]", 6, P) ST_RD2(120, 121, "%[xb]", 8, P) ST_RD2(122, 123, "%[xb]", 10, P)                  \
    ST_RD2(124, 125, "%[xb]", 12, P) ST_RD2(126, 127, "%[xb]", 14, P)                                                 \
    ST_RELOAD_WAIT

#else
// pair (slot hi, slot lo) of a window register: both slots have the shift group's parity, so both are whole
// 256-byte units away from the base of that parity (XA for even slots, XA + 128 for odd ones)
#define ST_RDP(J, I, BASE, OHI, OLO, P)                                                                               \
    "ds_read2st64_b32 " ST_XP(J, I) ", " BASE " offset0:" #P "*128+" #OHI " offset1:" #P "*128+" #OLO "\n"
#define ST_RELOAD(XA, P)                                                                                              \
    "v_add_u32 %[xb], 0x80, " XA "\n"                                                                                 \
    ST_RDP(0, 0, XA, 14, 0, P) ST_RDP(0, 1, XA, 8, 2, P) ST_RDP(0, 2, XA, 10, 4, P) ST_RDP(0, 3, XA, 12, 6, P)        \
    ST_RDP(1, 0, "%[xb]", 14, 0, P) ST_RDP(1, 1, "%[xb]", 8, 2, P) ST_RDP(1, 2, "%[xb]", 10, 4, P) ST_RDP(1, 3, "%[xb]", 12, 6, P) \
    ST_RDP(2, 0, XA, 15, 1, P) ST_RDP(2, 1, XA, 9, 3, P) ST_RDP(2, 2, XA, 11, 5, P) ST_RDP(2, 3, XA, 13, 7, P)        \
    ST_RDP(3, 0, "%[xb]", 15, 1, P) ST_RDP(3, 1, "%[xb]", 9, 3, P) ST_RDP(3, 2, "%[xb]", 11, 5, P) ST_RDP(3, 3, "%[xb]", 13, 7, P)

#endif
// ---- the decode block (decode_asm.hpp's schedule with named registers): per 8 steps 4 v_alignbit_b32 (none for shift
// 0), 4 v_pk_mad_u16 (two window hashes each), 8 address ops, 8 gathers, 8 products; the gathers of 8 steps are in flight
// while the products of the 8 before are formed
#ifndef ST_MFMA
#define ST_RDPAIR(G, TH, TL)                                  \
    "v_perm_b32 " TH ", " G ", %[lane4], %[sel]\n"            \
    "v_and_or_b32 " TL ", " G ", %[mask], %[lane4]\n"         \
    "ds_read_b32 " TH ", " TH "\n"                            \
    "ds_read_b32 " TL ", " TL "\n"
#define ST_READS_A ST_RDPAIR("%[g0]", "%[t0]", "%[t1]") ST_RDPAIR("%[g1]", "%[t2]", "%[t3]") \
                   ST_RDPAIR("%[g2]", "%[t4]", "%[t5]") ST_RDPAIR("%[g3]", "%[t6]", "%[t7]")
#define ST_READS_B ST_RDPAIR("%[g0]", "%[u0]", "%[u1]") ST_RDPAIR("%[g1]", "%[u2]", "%[u3]") \
                   ST_RDPAIR("%[g2]", "%[u4]", "%[u5]") ST_RDPAIR("%[g3]", "%[u6]", "%[u7]")
#define ST_WINDOWS(SH, EX, EY, EZ, EW)                        \
    "v_alignbit_b32 %[g0], %[cy], " EX ", " #SH "\n"          \
    "v_alignbit_b32 %[g1], " EX ", " EY ", " #SH "\n"         \
    "v_alignbit_b32 %[g2], " EY ", " EZ ", " #SH "\n"         \
    "v_alignbit_b32 %[g3], " EZ ", " EW ", " #SH "\n"         \
    "v_pk_mad_u16 %[g0], %[g0], %[g0], %[g0]\n"               \
    "v_pk_mad_u16 %[g1], %[g1], %[g1], %[g1]\n"               \
    "v_pk_mad_u16 %[g2], %[g2], %[g2], %[g2]\n"               \
    "v_pk_mad_u16 %[g3], %[g3], %[g3], %[g3]\n"
#define ST_WINDOWS0(EX, EY, EZ, EW)                           \
    "v_pk_mad_u16 %[g0], " EX ", " EX ", " EX "\n"            \
    "v_pk_mad_u16 %[g1], " EY ", " EY ", " EY "\n"            \
    "v_pk_mad_u16 %[g2], " EZ ", " EZ ", " EZ "\n"            \
    "v_pk_mad_u16 %[g3], " EW ", " EW ", " EW "\n"
// window register g0 = {carry, x}: slots 28 + j (high window), j (low); g1 = {x, y}: 16 + j, 4 + j; g2 = {y, z}: 20 + j,
// 8 + j; g3 = {z, w}: 24 + j, 12 + j, for shift 12 - 4 j (inference.cu:237-250)
#define ST_DOTS_FIRST(T, XA, XB, XC, XD, XE, XF, XG, XH)      \
    "v_dot2_f32_f16 %[a0], %[" T "0], " XA ", 0\n"            \
    "v_dot2_f32_f16 %[a1], %[" T "1], " XB ", 0\n"            \
    "v_dot2_f32_f16 %[a2], %[" T "2], " XC ", 0\n"            \
    "v_dot2_f32_f16 %[a3], %[" T "3], " XD ", 0\n"            \
    "v_dot2c_f32_f16 %[a0], %[" T "4], " XE "\n"              \
    "v_dot2c_f32_f16 %[a1], %[" T "5], " XF "\n"              \
    "v_dot2c_f32_f16 %[a2], %[" T "6], " XG "\n"              \
    "v_dot2c_f32_f16 %[a3], %[" T "7], " XH "\n"
#define ST_DOTS(T, XA, XB, XC, XD, XE, XF, XG, XH)            \
    "v_dot2c_f32_f16 %[a0], %[" T "0], " XA "\n"              \
    "v_dot2c_f32_f16 %[a1], %[" T "1], " XB "\n"              \
    "v_dot2c_f32_f16 %[a2], %[" T "2], " XC "\n"              \
    "v_dot2c_f32_f16 %[a3], %[" T "3], " XD "\n"              \
    "v_dot2c_f32_f16 %[a0], %[" T "4], " XE "\n"              \
    "v_dot2c_f32_f16 %[a1], %[" T "5], " XF "\n"              \
    "v_dot2c_f32_f16 %[a2], %[" T "6], " XG "\n"              \
    "v_dot2c_f32_f16 %[a3], %[" T "7], " XH "\n"
// OWN: what a row's first lane takes for the 16 bits in front of its element (its own last word as written,
// inference.cu:232; the word in front of the row, or zero in slab 0, in continuous mode); FIRST: the lanes that start a row
#ifdef ST_ROLL
// The same work as a rolling pipeline: sixteen gathers stay in flight; a step waits for the oldest two, forms their two
// products and puts the next window register's two gathers in their place, so a gather has eight steps' time to return
// instead of the time of one group of eight.
#define ST_STEP_FIRST(G, TH, TL, AH, AL, XH, XL)              \
    "s_waitcnt lgkmcnt(14)\n"                                 \
    "v_dot2_f32_f16 " AH ", " TH ", " XH ", 0\n"              \
    "v_dot2_f32_f16 " AL ", " TL ", " XL ", 0\n"              \
    ST_RDPAIR(G, TH, TL)
#define ST_STEP(G, TH, TL, AH, AL, XH, XL)                    \
    "s_waitcnt lgkmcnt(14)\n"                                 \
    "v_dot2c_f32_f16 " AH ", " TH ", " XH "\n"                \
    "v_dot2c_f32_f16 " AL ", " TL ", " XL "\n"                \
    ST_RDPAIR(G, TH, TL)
#define ST_DRAIN(N, TH, TL, AH, AL, XH, XL)                   \
    "s_waitcnt lgkmcnt(" #N ")\n"                             \
    "v_dot2c_f32_f16 " AH ", " TH ", " XH "\n"                \
    "v_dot2c_f32_f16 " AL ", " TL ", " XL "\n"
#define ST_DECODE(EX, EY, EZ, EW, OWN, FIRST)                                                                         \
    "s_nop 1\n"                                                                                                       \
    "s_mov_b64 vcc, " FIRST "\n"                                                                                      \
    "v_cndmask_b32_dpp %[cy], " EW ", " OWN ", vcc wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n"              \
    ST_WINDOWS(12, EX, EY, EZ, EW) ST_READS_A                                                                         \
    ST_WINDOWS(8, EX, EY, EZ, EW) ST_READS_B                                                                          \
    ST_WINDOWS(4, EX, EY, EZ, EW)                                                                                     \
    ST_STEP_FIRST("%[g0]", "%[t0]", "%[t1]", "%[a0]", "%[a1]", ST_X28, ST_X0)                                         \
    ST_STEP_FIRST("%[g1]", "%[t2]", "%[t3]", "%[a2]", "%[a3]", ST_X16, ST_X4)                                         \
    ST_STEP("%[g2]", "%[t4]", "%[t5]", "%[a0]", "%[a1]", ST_X20, ST_X8)                                               \
    ST_STEP("%[g3]", "%[t6]", "%[t7]", "%[a2]", "%[a3]", ST_X24, ST_X12)                                              \
    ST_WINDOWS0(EX, EY, EZ, EW)                                                                                       \
    ST_STEP("%[g0]", "%[u0]", "%[u1]", "%[a0]", "%[a1]", ST_X29, ST_X1)                                               \
    ST_STEP("%[g1]", "%[u2]", "%[u3]", "%[a2]", "%[a3]", ST_X17, ST_X5)                                               \
    ST_STEP("%[g2]", "%[u4]", "%[u5]", "%[a0]", "%[a1]", ST_X21, ST_X9)                                               \
    ST_STEP("%[g3]", "%[u6]", "%[u7]", "%[a2]", "%[a3]", ST_X25, ST_X13)                                              \
    ST_DRAIN(14, "%[t0]", "%[t1]", "%[a0]", "%[a1]", ST_X30, ST_X2)                                                   \
    ST_DRAIN(12, "%[t2]", "%[t3]", "%[a2]", "%[a3]", ST_X18, ST_X6)                                                   \
    ST_DRAIN(10, "%[t4]", "%[t5]", "%[a0]", "%[a1]", ST_X22, ST_X10)                                                  \
    ST_DRAIN(8, "%[t6]", "%[t7]", "%[a2]", "%[a3]", ST_X26, ST_X14)                                                   \
    ST_DRAIN(6, "%[u0]", "%[u1]", "%[a0]", "%[a1]", ST_X31, ST_X3)                                                    \
    ST_DRAIN(4, "%[u2]", "%[u3]", "%[a2]", "%[a3]", ST_X19, ST_X7)                                                    \
    ST_DRAIN(2, "%[u4]", "%[u5]", "%[a0]", "%[a1]", ST_X23, ST_X11)                                                   \
    ST_DRAIN(0, "%[u6]", "%[u7]", "%[a2]", "%[a3]", ST_X27, ST_X15)
#else
#define ST_DECODE(EX, EY, EZ, EW, OWN, FIRST)                                                                         \
    /* a DPP operand must not have been written by a vector op in the two instructions before */                     \
    "s_nop 1\n"                                                                                                       \
    "s_mov_b64 vcc, " FIRST "\n"                                                                                      \
    "v_cndmask_b32_dpp %[cy], " EW ", " OWN ", vcc wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n"              \
    ST_WINDOWS(12, EX, EY, EZ, EW) ST_READS_A                                                                         \
    ST_WINDOWS(8, EX, EY, EZ, EW) ST_READS_B                                                                          \
    "s_waitcnt lgkmcnt(8)\n"                                                                                          \
    ST_DOTS_FIRST("t", ST_X28, ST_X0, ST_X16, ST_X4, ST_X20, ST_X8, ST_X24, ST_X12)                                   \
    ST_WINDOWS(4, EX, EY, EZ, EW) ST_READS_A                                                                          \
    "s_waitcnt lgkmcnt(8)\n"                                                                                          \
    ST_DOTS("u", ST_X29, ST_X1, ST_X17, ST_X5, ST_X21, ST_X9, ST_X25, ST_X13)                                         \
    ST_WINDOWS0(EX, EY, EZ, EW) ST_READS_B                                                                            \
    "s_waitcnt lgkmcnt(8)\n"                                                                                          \
    ST_DOTS("t", ST_X30, ST_X2, ST_X18, ST_X6, ST_X22, ST_X10, ST_X26, ST_X14)                                        \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    ST_DOTS("u", ST_X31, ST_X3, ST_X19, ST_X7, ST_X23, ST_X11, ST_X27, ST_X15)
#endif

#else
// The products on the matrix unit: v_mfma_f32_4x4x4_16b_f16 multiplies, in every group of four lanes, the 4 x 4 matrix
// whose row i is lane i's A operand (four halves: the two gathered pairs of one window register) by the one whose
// column j is lane j's B operand (the activation pairs of the same two slots), so the diagonal of the result, element
// (i, i), in register i of lane i, is lane i's own four products added to what was there.  Sixteen of them replace the
// element's 32 two-term dot products, run beside the vector ALU, and cost it one issue slot each.  The gathered pairs
// land in fixed register pairs (v[56:63], v[64:71]: a matrix operand is an aligned pair), the sum in v[52:55].
// Distances the hardware does not interlock: two instructions between a matrix instruction and the next one that
// accumulates into its result; five before anything else reads the result.
#define ST_RDPAIR(G, TH, TL)                                  \
    "v_perm_b32 " TH ", " G ", %[lane4], %[sel]\n"            \
    "v_and_or_b32 " TL ", " G ", %[mask], %[lane4]\n"         \
    "ds_read_b32 " TH ", " TH "\n"                            \
    "ds_read_b32 " TL ", " TL "\n"
#define ST_READS_A ST_RDPAIR("%[g0]", "v56", "v57") ST_RDPAIR("%[g1]", "v58", "v59") \
                   ST_RDPAIR("%[g2]", "v60", "v61") ST_RDPAIR("%[g3]", "v62", "v63")
#define ST_READS_B ST_RDPAIR("%[g0]", "v64", "v65") ST_RDPAIR("%[g1]", "v66", "v67") \
                   ST_RDPAIR("%[g2]", "v68", "v69") ST_RDPAIR("%[g3]", "v70", "v71")
#define ST_MM(A, J, I, C) "v_mfma_f32_4x4x4_16b_f16 v[52:55], " A ", " ST_XP(J, I) ", " C "\n"
#ifdef ST_ROLL
// the rolling form (see the dot-product build above): a step waits for the oldest two gathers, multiplies them and
// puts the next window register's two gathers in their registers
#define ST_STEP(G, TH, TL, J, I, C)                           \
    "s_waitcnt lgkmcnt(14)\n"                                 \
    ST_MM("v[" TH ":" TL "]", J, I, C)                        \
    ST_RDPAIR(G, "v" TH, "v" TL)
#define ST_DRAIN(N, TH, TL, J, I)                             \
    "s_nop 0\n"                                               \
    "s_waitcnt lgkmcnt(" #N ")\n"                             \
    ST_MM("v[" TH ":" TL "]", J, I, "v[52:55]")
#define ST_WIN(SH, EX, EY, EZ, EW)                                                                                    \
    "v_alignbit_b32 %[g0], %[cy], " EX ", " #SH "\n v_alignbit_b32 %[g1], " EX ", " EY ", " #SH "\n"                  \
    "v_alignbit_b32 %[g2], " EY ", " EZ ", " #SH "\n v_alignbit_b32 %[g3], " EZ ", " EW ", " #SH "\n"                 \
    "v_pk_mad_u16 %[g0], %[g0], %[g0], %[g0]\n v_pk_mad_u16 %[g1], %[g1], %[g1], %[g1]\n"                             \
    "v_pk_mad_u16 %[g2], %[g2], %[g2], %[g2]\n v_pk_mad_u16 %[g3], %[g3], %[g3], %[g3]\n"
#define ST_DECODE(EX, EY, EZ, EW, OWN, FIRST)                                                                         \
    "s_nop 1\n"                                                                                                       \
    "s_mov_b64 vcc, " FIRST "\n"                                                                                      \
    "v_cndmask_b32_dpp %[cy], " EW ", " OWN ", vcc wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n"              \
    ST_WIN(12, EX, EY, EZ, EW) ST_READS_A                                                                             \
    ST_WIN(8, EX, EY, EZ, EW) ST_READS_B                                                                              \
    ST_WIN(4, EX, EY, EZ, EW)                                                                                         \
    ST_STEP("%[g0]", "56", "57", 0, 0, "0") ST_STEP("%[g1]", "58", "59", 0, 1, "v[52:55]")                            \
    ST_STEP("%[g2]", "60", "61", 0, 2, "v[52:55]") ST_STEP("%[g3]", "62", "63", 0, 3, "v[52:55]")                     \
    "v_pk_mad_u16 %[g0], " EX ", " EX ", " EX "\n v_pk_mad_u16 %[g1], " EY ", " EY ", " EY "\n"                       \
    "v_pk_mad_u16 %[g2], " EZ ", " EZ ", " EZ "\n v_pk_mad_u16 %[g3], " EW ", " EW ", " EW "\n"                       \
    ST_STEP("%[g0]", "64", "65", 1, 0, "v[52:55]") ST_STEP("%[g1]", "66", "67", 1, 1, "v[52:55]")                     \
    ST_STEP("%[g2]", "68", "69", 1, 2, "v[52:55]") ST_STEP("%[g3]", "70", "71", 1, 3, "v[52:55]")                     \
    ST_DRAIN(14, "56", "57", 2, 0) ST_DRAIN(12, "58", "59", 2, 1) ST_DRAIN(10, "60", "61", 2, 2)                      \
    ST_DRAIN(8, "62", "63", 2, 3) ST_DRAIN(6, "64", "65", 3, 0) ST_DRAIN(4, "66", "67", 3, 1)                         \
    ST_DRAIN(2, "68", "69", 3, 2) ST_DRAIN(0, "70", "71", 3, 3)
#else
#define ST_DECODE(EX, EY, EZ, EW, OWN, FIRST)                                                                         \
    /* a DPP operand must not have been written by a vector op in the two instructions before */                     \
    "s_nop 1\n"                                                                                                       \
    "s_mov_b64 vcc, " FIRST "\n"                                                                                      \
    "v_cndmask_b32_dpp %[cy], " EW ", " OWN ", vcc wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n"              \
    /* shift 12 */                                                                                                    \
    "v_alignbit_b32 %[g0], %[cy], " EX ", 12\n v_alignbit_b32 %[g1], " EX ", " EY ", 12\n"                            \
    "v_alignbit_b32 %[g2], " EY ", " EZ ", 12\n v_alignbit_b32 %[g3], " EZ ", " EW ", 12\n"                           \
    "v_pk_mad_u16 %[g0], %[g0], %[g0], %[g0]\n v_pk_mad_u16 %[g1], %[g1], %[g1], %[g1]\n"                             \
    "v_pk_mad_u16 %[g2], %[g2], %[g2], %[g2]\n v_pk_mad_u16 %[g3], %[g3], %[g3], %[g3]\n"                             \
    ST_READS_A                                                                                                        \
    /* shift 8 */                                                                                                     \
    "v_alignbit_b32 %[g0], %[cy], " EX ", 8\n v_alignbit_b32 %[g1], " EX ", " EY ", 8\n"                              \
    "v_alignbit_b32 %[g2], " EY ", " EZ ", 8\n v_alignbit_b32 %[g3], " EZ ", " EW ", 8\n"                             \
    "v_pk_mad_u16 %[g0], %[g0], %[g0], %[g0]\n v_pk_mad_u16 %[g1], %[g1], %[g1], %[g1]\n"                             \
    "v_pk_mad_u16 %[g2], %[g2], %[g2], %[g2]\n v_pk_mad_u16 %[g3], %[g3], %[g3], %[g3]\n"                             \
    ST_READS_B                                                                                                        \
    "s_waitcnt lgkmcnt(8)\n"                                                                                          \
    /* products of shift 12 between the windows of shift 4 */                                                         \
    ST_MM("v[56:57]", 0, 0, "0")                                                                                      \
    "v_alignbit_b32 %[g0], %[cy], " EX ", 4\n v_alignbit_b32 %[g1], " EX ", " EY ", 4\n"                              \
    ST_MM("v[58:59]", 0, 1, "v[52:55]")                                                                               \
    "v_alignbit_b32 %[g2], " EY ", " EZ ", 4\n v_alignbit_b32 %[g3], " EZ ", " EW ", 4\n"                             \
    ST_MM("v[60:61]", 0, 2, "v[52:55]")                                                                               \
    "v_pk_mad_u16 %[g0], %[g0], %[g0], %[g0]\n v_pk_mad_u16 %[g1], %[g1], %[g1], %[g1]\n"                             \
    ST_MM("v[62:63]", 0, 3, "v[52:55]")                                                                               \
    "v_pk_mad_u16 %[g2], %[g2], %[g2], %[g2]\n v_pk_mad_u16 %[g3], %[g3], %[g3], %[g3]\n"                             \
    ST_READS_A                                                                                                        \
    "s_waitcnt lgkmcnt(8)\n"                                                                                          \
    /* products of shift 8 between the hashes of shift 0 (the words as they are) */                                   \
    ST_MM("v[64:65]", 1, 0, "v[52:55]")                                                                               \
    "v_pk_mad_u16 %[g0], " EX ", " EX ", " EX "\n v_pk_mad_u16 %[g1], " EY ", " EY ", " EY "\n"                       \
    ST_MM("v[66:67]", 1, 1, "v[52:55]")                                                                               \
    "v_pk_mad_u16 %[g2], " EZ ", " EZ ", " EZ "\n v_pk_mad_u16 %[g3], " EW ", " EW ", " EW "\n"                       \
    ST_MM("v[68:69]", 1, 2, "v[52:55]")                                                                               \
    "s_nop 1\n"                                                                                                       \
    ST_MM("v[70:71]", 1, 3, "v[52:55]")                                                                               \
    ST_READS_B                                                                                                        \
    "s_waitcnt lgkmcnt(8)\n"                                                                                          \
    ST_MM("v[56:57]", 2, 0, "v[52:55]") "s_nop 1\n" ST_MM("v[58:59]", 2, 1, "v[52:55]") "s_nop 1\n"                   \
    ST_MM("v[60:61]", 2, 2, "v[52:55]") "s_nop 1\n" ST_MM("v[62:63]", 2, 3, "v[52:55]")                               \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_nop 0\n"                                                                                                       \
    ST_MM("v[64:65]", 3, 0, "v[52:55]") "s_nop 1\n" ST_MM("v[66:67]", 3, 1, "v[52:55]") "s_nop 1\n"                   \
    ST_MM("v[68:69]", 3, 2, "v[52:55]") "s_nop 1\n" ST_MM("v[70:71]", 3, 3, "v[52:55]")
#endif

#endif
// ---- one element of a layer.  U: which of the wave's elements; X, Y, Z, W / QUAD: its four registers; P: parity of
// the layer; NEED: requests that may still be in flight when this element's has arrived.
// Behind the last product the next layer's request for this slot goes out at once (three instructions between a dot
// product and another kind of vector op that reads its result are needed anyway), then the four sums become one
// and go to LDS under the mask of the lanes that hold an element of a row that exists.
// A wave without a U-th element makes the request all the same (its offset register points at the first cache line of
// the stream): every wave then has the same number of requests in flight, and the waits can be immediates.
#define ST_ITEM_HEAD(U, P, NEED)                                                                                      \
    "s_cmp_le_u32 %[nitems], " #U "\n"                                                                                \
    "s_cbranch_scc1 7" #U "f\n"                                                                                       \
    ST_PRIO_OF_##U                                                                                                    \
    "s_bitcmp1_b32 %[rl], " #U "\n"                                                                                   \
    "s_cbranch_scc0 5" #U "f\n"                                                                                       \
    ST_RELOAD("%[xa" #U "]", P)                                                                                       \
    "5" #U ":\n"                                                                                                      \
    "s_waitcnt vmcnt(" #NEED ")\n"
#ifndef ST_MFMA
#define ST_ELEMENT_SUM(U)                                                                                             \
    "s_mov_b64 exec, %[keep" #U "]\n"                                                                                 \
    "s_nop 0\n"                                                                                                       \
    "v_add_f32 %[a0], %[a0], %[a1]\n"                                                                                 \
    "v_add_f32 %[a2], %[a2], %[a3]\n"                                                                                 \
    "v_add_f32 %[a0], %[a0], %[a2]\n"
#else
// the lane's sum is register (lane % 4) of the matrix result: two selects by the lane number's bit 0, one by bit 1
#define ST_ELEMENT_SUM(U)                                                                                             \
    /* five instructions' distance from the last matrix instruction, whether or not a request stands in between */   \
    "s_mov_b64 vcc, %[odd]\n"                                                                                         \
    "s_mov_b64 exec, %[keep" #U "]\n"                                                                                 \
    "s_nop 2\n"                                                                                                       \
    "v_cndmask_b32 %[a0], v52, v53, vcc\n"                                                                            \
    "v_cndmask_b32 %[a1], v54, v55, vcc\n"                                                                            \
    "v_cndmask_b32_e64 %[a0], %[a0], %[a1], %[upper]\n"
#endif
#define ST_ITEM_TAIL(U, P, REQUEST)                                                                                   \
    REQUEST                                                                                                           \
    ST_ELEMENT_SUM(U)                                                                                                 \
    "ds_write_b32 %[pa" #U "], %[a0] offset:" #P "*16384\n"                                                           \
    "s_mov_b64 exec, -1\n"                                                                                            \
    "s_branch 8" #U "f\n"                                                                                             \
    "7" #U ":\n"                                                                                                      \
    REQUEST                                                                                                           \
    "8" #U ":\n"
#define ST_REQUEST_AW(U, QUAD) "global_load_dwordx4 " QUAD ", %[vo" #U "], %[cn] nt\n"
#define ST_REQUEST_CT(U, QUAD) "global_load_dwordx4 " QUAD ", %[vo" #U "], %[cn] nt\n"                               \
                               "global_load_dword %[cw" #U "], %[co" #U "], %[cn]\n"
// as written (MODE 0): a row's first lane takes its own last word; continuous (MODE 1): the word in front of the row
#define ST_ITEM_0(U, X, Y, Z, W, P, NEED, REQUEST)                                                                    \
    ST_ITEM_HEAD(U, P, NEED) ST_DECODE(X, Y, Z, W, W, "%[first" #U "]") ST_ITEM_TAIL(U, P, REQUEST)
#define ST_ITEM_1(U, X, Y, Z, W, P, NEED, REQUEST)                                                                    \
    ST_ITEM_HEAD(U, P, NEED) "v_and_b32 %[own], %[cm" #U "], %[cw" #U "]\n"                                           \
    ST_DECODE(X, Y, Z, W, "%[own]", "%[first" #U "]") ST_ITEM_TAIL(U, P, REQUEST)

// ---- the rows of the layer in front: a wave adds a row's n / 64 partial sums (lanes i, i + 64, i + 128, i + 192 in
// that order, then across the lanes with DPP adds: rows of 16, row 0 into 1 and 2 into 3, rows 0-1 into 2-3), round
// once to fp16 and lane 63 stores.  P: parity of the set that is read.
// a row wave's next row: eight rows further, or (ST_T_ROWS) as many as there are row waves
#ifdef ST_T_ROWS
#define ST_NEXT_ROW "v_add_u32 %[g1], %[ostep], %[g1]\n"
#else
#define ST_NEXT_ROW "v_add_u32 %[g1], 16, %[g1]\n"
#endif
#define ST_DPP_ADD(CTRL) "s_nop 1\n v_add_f32_dpp %[a0], %[a0], %[a0] " CTRL "\n"
#define ST_ROWS(P)                                                                                                    \
    "s_cmp_eq_u32 %[nr], 0\n"                                                                                         \
    "s_cbranch_scc1 92f\n"                                                                                            \
    "v_mov_b32 %[g0], %[rs]\n"                                                                                        \
    "v_mov_b32 %[g1], %[oo]\n"                                                                                        \
    "s_mov_b32 %[j], %[nr]\n"                                                                                         \
    "91:\n"                                                                                                           \
    "v_mov_b32 %[t0], 0\n v_mov_b32 %[t1], 0\n v_mov_b32 %[t2], 0\n v_mov_b32 %[t3], 0\n"                             \
    "s_mov_b64 exec, %[rm0]\n ds_read_b32 %[t0], %[g0] offset:" #P "*16384\n"                                         \
    "s_mov_b64 exec, %[rm1]\n ds_read_b32 %[t1], %[g0] offset:" #P "*16384+256\n"                                     \
    "s_mov_b64 exec, %[rm2]\n ds_read_b32 %[t2], %[g0] offset:" #P "*16384+512\n"                                     \
    "s_mov_b64 exec, %[rm3]\n ds_read_b32 %[t3], %[g0] offset:" #P "*16384+768\n"                                     \
    "s_mov_b64 exec, -1\n"                                                                                            \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "v_add_f32 %[a0], %[t0], %[t1]\n"                                                                                 \
    "v_add_f32 %[a0], %[a0], %[t2]\n"                                                                                 \
    "v_add_f32 %[a0], %[a0], %[t3]\n"                                                                                 \
    ST_DPP_ADD("row_shr:1 row_mask:0xf bank_mask:0xf")                                                                \
    ST_DPP_ADD("row_shr:2 row_mask:0xf bank_mask:0xf")                                                                \
    ST_DPP_ADD("row_shr:4 row_mask:0xf bank_mask:0xf")                                                                \
    ST_DPP_ADD("row_shr:8 row_mask:0xf bank_mask:0xf")                                                                \
    ST_DPP_ADD("row_bcast:15 row_mask:0xa bank_mask:0xf")                                                             \
    ST_DPP_ADD("row_bcast:31 row_mask:0xc bank_mask:0xf")                                                             \
    "v_cvt_f16_f32 %[a0], %[a0]\n"                                                                                    \
    "s_mov_b64 exec, %[l63]\n"                                                                                        \
    "global_store_short %[g1], %[a0], %[op]\n"                                                                        \
    "s_mov_b64 exec, -1\n"                                                                                            \
    "v_add_u32 %[g0], %[rstep], %[g0]\n"                                                                              \
    ST_NEXT_ROW                                                                                                       \
    "s_sub_u32 %[j], %[j], 1\n"                                                                                       \
    "s_cmp_lg_u32 %[j], 0\n"                                                                                          \
    "s_cbranch_scc1 91b\n"                                                                                            \
    "92:\n"

// ---- a thread's share of the next layer's activations into image P (halves 8 idx .. 8 idx + 7 go to the four planes,
// inference.cu:215-221; the addresses were worked out in front of the loop)
#define ST_STAGE(P)                                                                                                   \
    "s_mov_b64 exec, %[stm0]\n"                                                                                       \
    "ds_write_b32 %[sa0], v72 offset:" #P "*32768\n ds_write_b32 %[sa1], v73 offset:" #P "*32768\n"                   \
    "ds_write_b32 %[sa2], v74 offset:" #P "*32768\n ds_write_b32 %[sa3], v75 offset:" #P "*32768\n"                   \
    "s_mov_b64 exec, %[stm1]\n"                                                                                       \
    "ds_write_b32 %[sa4], v76 offset:" #P "*32768\n ds_write_b32 %[sa5], v77 offset:" #P "*32768\n"                   \
    "ds_write_b32 %[sa6], v78 offset:" #P "*32768\n ds_write_b32 %[sa7], v79 offset:" #P "*32768\n"                   \
    "s_mov_b64 exec, -1\n"

// ---- the loop.  MODE: 0 as written, 1 continuous; LPI: requests per element (1; 2 continuous); M: elements a wave holds.
// Requests in flight, oldest first, when element u's is waited for: u's own, the later elements' of this layer, the two
// activation requests made at the top of this layer, the earlier elements' of the next layer: NEED = (M - 1) * LPI + 2
// may stay in flight.  When the activations are staged the M * LPI element requests made behind them may stay in
// flight (STW).  Stores of the rows phase sit in the same queue behind all of them: they only make a wait stricter.
#define ST_POINTERS                                                                                                   \
    /* the layer behind the one k counts (clamped to the last) and the layer in front of it (clamped to the first) */ \
    "s_add_u32 %[kn], %[k], 1\n"                                                                                      \
    "s_min_u32 %[kn], %[kn], %[last]\n"                                                                               \
    "s_lshl_b32 %[kn], %[kn], 6\n"                                                                                    \
    "s_load_dwordx2 %[cn], %[dc], %[kn]\n"                                                                            \
    "s_load_dwordx2 %[xn], %[dx], %[kn]\n"                                                                            \
    "s_max_u32 %[kn], %[k], 1\n"                                                                                      \
    "s_sub_u32 %[kn], %[kn], 1\n"                                                                                     \
    "s_lshl_b32 %[kn], %[kn], 6\n"                                                                                    \
    "s_load_dwordx2 %[op], %[dq], %[kn]\n"
#define ST_XREQUESTS                                                                                                  \
    "global_load_dwordx4 v[72:75], %[xo0], %[xn]\n"                                                                   \
    "global_load_dwordx4 v[76:79], %[xo1], %[xn]\n"

#ifdef ST_T_FLOW
// The next layer's activations are staged behind the first element: their requests went out at the top of the layer,
// and only the first element's next request has been made since (LPI requests may stay in flight).
#define ST_EARLY_STAGE(Q, LPI) "s_waitcnt vmcnt(" #LPI ")\n" ST_STAGE(Q)
#define ST_ITEMS_3(MODE, P, Q, NEED, LPI)                                                                             \
    ST_ITEM_##MODE(0, "v80", "v81", "v82", "v83", P, NEED, ST_REQUEST_##MODE(0, "v[80:83]"))                          \
    ST_EARLY_STAGE(Q, LPI)                                                                                            \
    ST_ITEM_##MODE(1, "v84", "v85", "v86", "v87", P, NEED, ST_REQUEST_##MODE(1, "v[84:87]"))                          \
    ST_ITEM_##MODE(2, "v88", "v89", "v90", "v91", P, NEED, ST_REQUEST_##MODE(2, "v[88:91]"))
#define ST_ITEMS_4(MODE, P, Q, NEED, LPI)                                                                             \
    ST_ITEMS_3(MODE, P, Q, NEED, LPI) ST_ITEM_##MODE(3, "v92", "v93", "v94", "v95", P, NEED, ST_REQUEST_##MODE(3, "v[92:95]"))
// the chain's last layer: nothing is requested any more, and everything requested has been waited for (vmcnt(63) waits for nothing)
#define ST_LAST_ITEMS_3(MODE, P)                                                                                      \
    ST_ITEM_##MODE(0, "v80", "v81", "v82", "v83", P, 63, "") ST_ITEM_##MODE(1, "v84", "v85", "v86", "v87", P, 63, "")  \
    ST_ITEM_##MODE(2, "v88", "v89", "v90", "v91", P, 63, "")
#define ST_LAST_ITEMS_4(MODE, P) ST_LAST_ITEMS_3(MODE, P) ST_ITEM_##MODE(3, "v92", "v93", "v94", "v95", P, 63, "")
#else
#define ST_ITEMS_3(MODE, P, Q, NEED, LPI)                                                                             \
    ST_ITEM_##MODE(0, "v80", "v81", "v82", "v83", P, NEED, ST_REQUEST_##MODE(0, "v[80:83]"))                          \
    ST_ITEM_##MODE(1, "v84", "v85", "v86", "v87", P, NEED, ST_REQUEST_##MODE(1, "v[84:87]"))                          \
    ST_ITEM_##MODE(2, "v88", "v89", "v90", "v91", P, NEED, ST_REQUEST_##MODE(2, "v[88:91]"))
#define ST_ITEMS_4(MODE, P, Q, NEED, LPI)                                                                             \
    ST_ITEMS_3(MODE, P, Q, NEED, LPI) ST_ITEM_##MODE(3, "v92", "v93", "v94", "v95", P, NEED, ST_REQUEST_##MODE(3, "v[92:95]"))
#endif
#define ST_REQUESTS_3(MODE) ST_REQUEST_##MODE(0, "v[80:83]") ST_REQUEST_##MODE(1, "v[84:87]") ST_REQUEST_##MODE(2, "v[88:91]")
#define ST_REQUESTS_4(MODE) ST_REQUESTS_3(MODE) ST_REQUEST_##MODE(3, "v[92:95]")
#define ST_REQUEST_0(U, QUAD) ST_REQUEST_AW(U, QUAD)
#define ST_REQUEST_1(U, QUAD) ST_REQUEST_CT(U, QUAD)

#ifdef ST_T_FLOW
// layer k of parity P (Q the other one): on entry the pointers of layer k + 1 and of layer k - 1 have arrived, image P
// holds layer k's activations and set Q layer k - 1's partial sums
#define ST_LAYER(P, Q, MODE, M, NEED, STW, LPI)                                                                       \
    ST_XREQUESTS                                                                                                      \
    ST_ITEMS_##M(MODE, P, Q, NEED, LPI)                                                                               \
    ST_PRIO("3")                                                                                                      \
    "s_cmp_eq_u32 %[k], 0\n"                                                                                          \
    "s_cbranch_scc1 93f\n"                                                                                            \
    ST_ROWS(Q)                                                                                                        \
    "93:\n"                                                                                                           \
    "s_add_u32 %[k], %[k], 1\n"                                                                                       \
    ST_POINTERS                                                                                                       \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_barrier\n"

// the last layer, of parity P: no requests (there is no layer behind it to ask for), the rows of the layer in front, then
// its own rows behind one more barrier
#define ST_LAST_LAYER(P, Q, MODE, M)                                                                                  \
    "s_waitcnt vmcnt(0)\n"                                                                                            \
    ST_LAST_ITEMS_##M(MODE, P)                                                                                        \
    ST_PRIO("3")                                                                                                      \
    "s_cmp_eq_u32 %[k], 0\n"                                                                                          \
    "s_cbranch_scc1 93f\n"                                                                                            \
    ST_ROWS(Q)                                                                                                        \
    "93:\n"                                                                                                           \
    "s_add_u32 %[k], %[k], 1\n"                                                                                       \
    ST_POINTERS                                                                                                       \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_barrier\n"                                                                                                     \
    ST_ROWS(P)

#define ST_BODY(MODE, M, NEED, STW, LPI)                                                                              \
    "s_mov_b32 %[k], 0\n"                                                                                             \
    "s_mov_b32 %[kn], 0\n"                                                                                            \
    "s_load_dwordx2 %[cn], %[dc], %[kn]\n"                                                                            \
    "s_load_dwordx2 %[xn], %[dx], %[kn]\n"                                                                            \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    ST_XREQUESTS                                                                                                      \
    ST_REQUESTS_##M(MODE)                                                                                             \
    "s_waitcnt vmcnt(" #STW ")\n"                                                                                     \
    ST_STAGE(0)                                                                                                       \
    ST_POINTERS                                                                                                       \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_barrier\n"                                                                                                     \
    /* layers 0 .. count - 2 ask for the layer behind them while they decode; the last one (k == last) does not */    \
    "s_cmp_eq_u32 %[k], %[last]\n"                                                                                    \
    "s_cbranch_scc1 11f\n"                                                                                            \
    "10:\n"                                                                                                           \
    ST_LAYER(0, 1, MODE, M, NEED, STW, LPI)                                                                           \
    "s_cmp_eq_u32 %[k], %[last]\n"                                                                                    \
    "s_cbranch_scc1 13f\n"                                                                                            \
    ST_LAYER(1, 0, MODE, M, NEED, STW, LPI)                                                                           \
    "s_cmp_lg_u32 %[k], %[last]\n"                                                                                    \
    "s_cbranch_scc1 10b\n"                                                                                            \
    "11:\n"                                                                                                           \
    ST_LAST_LAYER(0, 1, MODE, M)                                                                                      \
    "s_branch 12f\n"                                                                                                  \
    "13:\n"                                                                                                           \
    ST_LAST_LAYER(1, 0, MODE, M)                                                                                      \
    "12:\n"                                                                                                           \
    "s_waitcnt vmcnt(0)\n"
#else
// layer k of parity P (Q the other one): on entry the pointers of layer k + 1 and of layer k - 1 have arrived, image P
// holds layer k's activations and set Q layer k - 1's partial sums.  Behind the elements the next layer's activations
// are staged and the rows of the layer in front added up.
#define ST_LAYER(P, Q, MODE, M, NEED, STW, LPI)                                                                       \
    ST_XREQUESTS                                                                                                      \
    ST_ITEMS_##M(MODE, P, Q, NEED, LPI)                                                                               \
    ST_PRIO("3")                                                                                                      \
    "s_waitcnt vmcnt(" #STW ")\n"                                                                                     \
    ST_STAGE(Q)                                                                                                       \
    "s_cmp_eq_u32 %[k], 0\n"                                                                                          \
    "s_cbranch_scc1 93f\n"                                                                                            \
    ST_ROWS(Q)                                                                                                        \
    "93:\n"                                                                                                           \
    "s_add_u32 %[k], %[k], 1\n"                                                                                       \
    ST_POINTERS                                                                                                       \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_barrier\n"

// every layer asks for the layer behind it (the last one for itself again: the pointers are clamped)
#define ST_BODY(MODE, M, NEED, STW, LPI)                                                                              \
    "s_mov_b32 %[k], 0\n"                                                                                             \
    "s_mov_b32 %[kn], 0\n"                                                                                            \
    "s_load_dwordx2 %[cn], %[dc], %[kn]\n"                                                                            \
    "s_load_dwordx2 %[xn], %[dx], %[kn]\n"                                                                            \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    ST_XREQUESTS                                                                                                      \
    ST_REQUESTS_##M(MODE)                                                                                             \
    "s_waitcnt vmcnt(" #STW ")\n"                                                                                     \
    ST_STAGE(0)                                                                                                       \
    ST_POINTERS                                                                                                       \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_barrier\n"                                                                                                     \
    "10:\n"                                                                                                           \
    ST_LAYER(0, 1, MODE, M, NEED, STW, LPI)                                                                           \
    "s_cmp_ge_u32 %[k], %[count]\n"                                                                                   \
    "s_cbranch_scc1 11f\n"                                                                                            \
    ST_LAYER(1, 0, MODE, M, NEED, STW, LPI)                                                                           \
    "s_cmp_lt_u32 %[k], %[count]\n"                                                                                   \
    "s_cbranch_scc1 10b\n"                                                                                            \
    /* the last layer's rows: its partial sums are in set 1 (an even number of layers) or set 0 */                    \
    ST_ROWS(1)                                                                                                        \
    "s_branch 12f\n"                                                                                                  \
    "11:\n"                                                                                                           \
    ST_ROWS(0)                                                                                                        \
    "12:\n"                                                                                                           \
    "s_waitcnt vmcnt(0)\n"
#endif

// what the loop reads and the registers it works in
#ifndef ST_MFMA
#define ST_OUT_COMMON                                                                                                 \
    [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3), [cy] "=&v"(cy), [g0] "=&v"(g0), [g1] "=&v"(g1),  \
    [g2] "=&v"(g2), [g3] "=&v"(g3), [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3), [t4] "=&v"(t4),  \
    [t5] "=&v"(t5), [t6] "=&v"(t6), [t7] "=&v"(t7), [u0] "=&v"(u0), [u1] "=&v"(u1), [u2] "=&v"(u2), [u3] "=&v"(u3),  \
    [u4] "=&v"(u4), [u5] "=&v"(u5), [u6] "=&v"(u6), [u7] "=&v"(u7), [xb] "=&v"(xb), [k] "=&s"(k), [kn] "=&s"(kn),    \
    [j] "=&s"(j), [cn] "=&s"(cn), [xn] "=&s"(xn), [op] "=&s"(op)
#define ST_IN_SUM [mask] "s"(0xFF00u)
#define ST_CLOBBERS_SUM "memory"
#else
#define ST_OUT_COMMON                                                                                                 \
    [a0] "=&v"(a0), [a1] "=&v"(a1), [cy] "=&v"(cy), [g0] "=&v"(g0), [g1] "=&v"(g1), [g2] "=&v"(g2), [g3] "=&v"(g3),  \
    [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3), [xb] "=&v"(xb), [k] "=&s"(k), [kn] "=&s"(kn),    \
    [j] "=&s"(j), [cn] "=&s"(cn), [xn] "=&s"(xn), [op] "=&s"(op)
#define ST_IN_SUM [mask] "s"(0xFF00u), [odd] "s"(0xAAAAAAAAAAAAAAAAull), [upper] "s"(0xCCCCCCCCCCCCCCCCull)
#define ST_CLOBBERS_SUM                                                                                               \
    "memory", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", "v60", "v61", "v62", "v63", "v64", "v65", "v66", "v67",   \
    "v68", "v69", "v70", "v71"
#endif
#define ST_IN_COMMON                                                                                                  \
    [lane4] "v"(lane4), ST_IN_SUM, [sel] "s"(0x0C0C0700u), [dc] "s"(dc), [dx] "s"(dx), [dq] "s"(dout),      \
    [count] "s"(s_count), [last] "s"(s_count - 1), [nitems] "s"(s_nitems), [rl] "s"(rl), [xo0] "v"(xo[0]), [xo1] "v"(xo[1]),\
    [sa0] "v"(sa[0]), [sa1] "v"(sa[1]), [sa2] "v"(sa[2]), [sa3] "v"(sa[3]), [sa4] "v"(sa[4]), [sa5] "v"(sa[5]),       \
    [sa6] "v"(sa[6]), [sa7] "v"(sa[7]), [stm0] "s"(stm[0]), [stm1] "s"(stm[1]), [rs] "v"(rs), [oo] "v"(oo),           \
    [rstep] "s"(s_rstep), ST_IN_OSTEP [nr] "s"(s_nr), [rm0] "s"(rm[0]), [rm1] "s"(rm[1]), [rm2] "s"(rm[2]), [rm3] "s"(rm[3]),         \
    [l63] "s"(0x8000000000000000ull)
#ifdef ST_T_ROWS
#define ST_IN_OSTEP [ostep] "s"(s_ostep),
#else
#define ST_IN_OSTEP
#endif
#define ST_IN_ITEM(U) [vo##U] "v"(vo[U]), [xa##U] "v"(xa[U]), [pa##U] "v"(pa[U]), [first##U] "s"(first[U]), [keep##U] "s"(keep[U])
#define ST_IN_ITEM_CT(U) [co##U] "v"(co[U]), [cm##U] "s"(cm[U])
#define ST_CLOBBERS                                                                                                   \
    ST_CLOBBERS_SUM, "vcc", "scc", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79", "v80", "v81", "v82", "v83", "v84", "v85",   \
    "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101", "v102",   \
    "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117",     \
    "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127"

template <int S, int MODE, int MAXI>
__global__ __launch_bounds__(kStThreads) void matvec_steady_kernel(
    const LoopLayer *__restrict__ layers, const uint32_t *__restrict__ codebook, int count, int arg_m, int arg_n,
    int rows_per_block, int rw_tail, int items_tail, uint32_t full_magic)
{
    static_assert(MAXI == 3 || MAXI == 4, "a wave holds three or four elements of a layer");
    extern __shared__ uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;   // the table is at LDS address 0
    const int m = arg_m, n = arg_n;
    const int T = n >> 11, Lt = (n & 2047) >> 6, npr = n >> 6, n8 = n >> 3;
    const int items_full = rows_per_block >> 1;
    const int row0 = blockIdx.x * rows_per_block;
    const int rows = min(rows_per_block, m - row0);

    // the table: rows 16 wave .. 16 wave + 15 are this wave's to write (a row is 64 copies of one value; bit 7 of the row
    // number is the sign that replaces the first value's, inference.cu:259-262)
    constexpr int kRowsPerWave = 256 / kStWaves;
    {
        uint32_t cbv[kRowsPerWave];
#pragma unroll
        for (int i = 0; i < kRowsPerWave; i++) cbv[i] = codebook[(kRowsPerWave * wave + i) & ((1 << S) - 1)];
        const uint32_t table_sign = (uint32_t)((kRowsPerWave * wave) >> 7) << 15;
#pragma unroll
        for (int i = 0; i < kRowsPerWave; i++) lds[(kRowsPerWave * wave + i) * 64 + lane] = (cbv[i] & 0xFFFF7FFFu) | table_sign;
    }

    // ---- this wave's elements of a layer (the same in every layer): equal shares, the first total % 16 waves one more
    const int total = T * items_full + items_tail;
    const int per_wave = (int)((uint32_t)total / kStWaves), extra = (int)((uint32_t)total % kStWaves);
    const int it_begin = wave * per_wave + min(wave, extra);
    const int nitems = per_wave + (wave < extra ? 1 : 0);                // at most MAXI: the host checks
    uint32_t vo[MAXI], xa[MAXI], pa[MAXI], co[MAXI], cm[MAXI];
    uint64_t first[MAXI], keep[MAXI];
    uint32_t rl = 0;
    int prev_slab = -1;
#pragma unroll
    for (int u = 0; u < MAXI; u++) {
        const int it = it_begin + u;
        const bool mine = u < nitems;
        int slab = items_full == 1 ? it : (int)__umulhi((uint32_t)it, full_magic);
        slab = min(slab, T);
        const int idx = it - slab * items_full;
        const bool full = slab < T;
        const int lanes = full ? 32 : Lt, rpi = full ? 2 : rw_tail;
        const int row_first = idx * rpi;
        const int rows_here = mine ? min(rpi, rows - row_first) : 0;          // <= 0: an element past the block's last row
        const bool real = rows_here > 0;
        // lane -> (row inside the item, element inside the row); lanes past the last whole row of a ragged item idle on element 0
        int sub, l;
        if (full) {
            sub = lane >> 5, l = lane & 31;
        } else {
            sub = lane / max(lanes, 1), l = lane - sub * lanes;
            if (sub >= rpi) l = 0;
        }
        const uint32_t elem0 = (uint32_t)(full ? slab : T) * (uint32_t)m * 32u;
        const uint32_t elem = real ? elem0 + (uint32_t)(row0 + row_first) * (uint32_t)lanes : 0u;
        const uint32_t last = real ? (uint32_t)(rows_here * lanes - 1) : 0u;
        vo[u] = 16u * (elem + min((uint32_t)lane, last));
        xa[u] = (uint32_t)kStTableBytes + 4u * (uint32_t)(1024 * slab + l);
        pa[u] = (uint32_t)kStPartBase + 4u * (uint32_t)((row_first + sub) * npr + 32 * slab + l);
        first[u] = __builtin_amdgcn_ballot_w64(l == 0);
        const int nact = max(rows_here, 0) * lanes;
        keep[u] = nact >= 64 ? ~0ull : (1ull << nact) - 1ull;
        if (mine && slab != prev_slab) rl |= 1u << u;
        if (mine) prev_slab = slab;
        // continuous mode: the word in front of a row is the last word of the row's lane 31 in the slab before
        const bool prev = real && slab > 0;
        const int sub_c = min(sub, max(rows_here, 1) - 1);
        co[u] = prev ? 4u * ((((uint32_t)(slab - 1) * (uint32_t)m + (uint32_t)(row0 + row_first + sub_c)) * 32u + 31u) * 4u + 3u) : 0u;
        cm[u] = prev ? ~0u : 0u;
    }

    // ---- a thread's share of a layer's activations: 16 bytes at 8 idx (two of them), whose four words are the pairs of
    // slots i * n8 + idx (inference.cu:215-221); where each goes in an image (the ragged slab at the full slabs' stride)
    uint32_t xo[2], sa[8];
    uint64_t stm[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int idx = tid + u * kStThreads;
        xo[u] = 16u * (uint32_t)min(idx, n8 - 1);
        stm[u] = __builtin_amdgcn_ballot_w64(idx < n8);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int P = i * n8 + min(idx, n8 - 1);
            int pos = P;
            if (P >= 1024 * T) {
                const int r = P - 1024 * T, q = r / max(Lt, 1);
                pos = 1024 * T + 32 * q + (r - q * Lt);
            }
            sa[4 * u + i] = (uint32_t)kStTableBytes + 4u * (uint32_t)pos;
        }
    }

    // ---- the rows: added up by waves 0-7, or (ST_T_ROWS) by the waves that hold the fewest elements (all sixteen when the
    // shares are equal), the i-th of them taking rows i, i + their number, ...
#ifdef ST_T_ROWS
    const int first_row_wave = extra, row_waves = kStWaves - extra;
#else
    const int first_row_wave = 0, row_waves = 8;
#endif
    const int ri = wave - first_row_wave;
    const uint32_t rs = (uint32_t)kStPartBase + 4u * (uint32_t)(max(ri, 0) * npr + lane);
    const uint32_t oo = 2u * (uint32_t)(row0 + max(ri, 0));
    const uint32_t rstep = 4u * (uint32_t)(row_waves * npr), ostep = 2u * (uint32_t)row_waves;
    const uint32_t nr = ri >= 0 && ri < row_waves && ri < rows ? (uint32_t)(rows - ri + row_waves - 1) / (uint32_t)row_waves : 0u;
    uint64_t rm[4];
#pragma unroll
    for (int c = 0; c < 4; c++) rm[c] = __builtin_amdgcn_ballot_w64(lane + 64 * c < npr);

    const uint64_t dc = reinterpret_cast<uint64_t>(&layers[0].comp), dx = reinterpret_cast<uint64_t>(&layers[0].x),
                   dout = reinterpret_cast<uint64_t>(&layers[0].out);
    __syncthreads();                                          // the table is complete

    // what the block takes in scalar registers is wave-uniform by construction; say so, so that every one of them is
    // in a scalar register whatever the compiler's divergence analysis makes of the code above
    auto uni = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
    auto uni64 = [&](uint64_t v) { return (uint64_t)uni((uint32_t)v) | ((uint64_t)uni((uint32_t)(v >> 32)) << 32); };
    rl = uni(rl);
    const uint32_t s_nitems = uni((uint32_t)nitems), s_nr = uni(nr), s_rstep = uni(rstep), s_count = uni((uint32_t)count);
    [[maybe_unused]] const uint32_t s_ostep = uni(ostep);
#pragma unroll
    for (int u = 0; u < MAXI; u++) first[u] = uni64(first[u]), keep[u] = uni64(keep[u]), cm[u] = uni(cm[u]);
#pragma unroll
    for (int c = 0; c < 4; c++) rm[c] = uni64(rm[c]);
    stm[0] = uni64(stm[0]), stm[1] = uni64(stm[1]);

    uint32_t a0, a1, a2, a3, cy, g0, g1, g2, g3, t0, t1, t2, t3, t4, t5, t6, t7, u0, u1, u2, u3, u4, u5, u6, u7, xb, k, kn, j;
    uint64_t cn, xn, op;
    if constexpr (MODE == RPTC_AS_WRITTEN && MAXI == 3) {
        asm volatile(ST_BODY(0, 3, 4, 3, 1)
                     : ST_OUT_COMMON
                     : ST_IN_COMMON, ST_IN_ITEM(0), ST_IN_ITEM(1), ST_IN_ITEM(2)
                     : ST_CLOBBERS);
    } else if constexpr (MODE == RPTC_AS_WRITTEN) {
        asm volatile(ST_BODY(0, 4, 5, 4, 1)
                     : ST_OUT_COMMON
                     : ST_IN_COMMON, ST_IN_ITEM(0), ST_IN_ITEM(1), ST_IN_ITEM(2), ST_IN_ITEM(3)
                     : ST_CLOBBERS);
    } else if constexpr (MAXI == 3) {
        uint32_t own, cw0 = 0, cw1 = 0, cw2 = 0;
        asm volatile(ST_BODY(1, 3, 6, 6, 2)
                     : ST_OUT_COMMON, [own] "=&v"(own), [cw0] "+v"(cw0), [cw1] "+v"(cw1), [cw2] "+v"(cw2)
                     : ST_IN_COMMON, ST_IN_ITEM(0), ST_IN_ITEM(1), ST_IN_ITEM(2), ST_IN_ITEM_CT(0), ST_IN_ITEM_CT(1), ST_IN_ITEM_CT(2)
                     : ST_CLOBBERS);
    } else {
        uint32_t own, cw0 = 0, cw1 = 0, cw2 = 0, cw3 = 0;
        asm volatile(ST_BODY(1, 4, 8, 8, 2)
                     : ST_OUT_COMMON, [own] "=&v"(own), [cw0] "+v"(cw0), [cw1] "+v"(cw1), [cw2] "+v"(cw2), [cw3] "+v"(cw3)
                     : ST_IN_COMMON, ST_IN_ITEM(0), ST_IN_ITEM(1), ST_IN_ITEM(2), ST_IN_ITEM(3), ST_IN_ITEM_CT(0), ST_IN_ITEM_CT(1),
                       ST_IN_ITEM_CT(2), ST_IN_ITEM_CT(3)
                     : ST_CLOBBERS);
    }
}

#ifndef ST_MFMA
// ---------------------------------------------------------------- one layer per launch with the same hand-written body
// (behind -DRPTC_MV_ONE in matvec.hip's launcher until it is timed).  The launch is the per-launch op's
// (rptc_decompress_matvec_16_{S}_1: one layer, no descriptors); what it takes from the chain kernel is the decode of a
// wave's elements with everything about them worked out in front, the activation reload as two-dword reads and the
// rows as a counted loop - the per-launch kernel's own element loop spends 86 scalar and 146 vector instructions an
// element where this body spends 14 and 105.  The prologue is written for a short way to the first request: the
// activation and stream requests go out first (ordinary loads: the compiler waits for them in front of the block),
// the table and the rest of the geometry while they are on their way; the ragged slab's lane numbers and slots come
// from a multiplication (a 16-bit reciprocal of the ragged row's length from the host) instead of a division.
#define ST_ONE_ITEM_0(U) ST_ITEM_0(U, "%[e" #U "x]", "%[e" #U "y]", "%[e" #U "z]", "%[e" #U "w]", 0, 63, "")
#define ST_ONE_ITEM_1(U) ST_ITEM_1(U, "%[e" #U "x]", "%[e" #U "y]", "%[e" #U "z]", "%[e" #U "w]", 0, 63, "")
#define ST_ONE_ITEMS_3(MODE) ST_ONE_ITEM_##MODE(0) ST_ONE_ITEM_##MODE(1) ST_ONE_ITEM_##MODE(2)
#define ST_ONE_ITEMS_4(MODE) ST_ONE_ITEMS_3(MODE) ST_ONE_ITEM_##MODE(3)
#define ST_ONE_ITEMS_6(MODE) ST_ONE_ITEMS_4(MODE) ST_ONE_ITEM_##MODE(4) ST_ONE_ITEM_##MODE(5)
#define ST_ONE_BODY(MODE, M)                                                                                          \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_barrier\n"                                                                                                     \
    ST_ONE_ITEMS_##M(MODE)                                                                                            \
    ST_PRIO("3")                                                                                                      \
    "s_waitcnt lgkmcnt(0)\n"                                                                                          \
    "s_barrier\n"                                                                                                     \
    ST_ROWS(0)                                                                                                        \
    "s_waitcnt vmcnt(0)\n"
#define ST_ONE_OUT                                                                                                    \
    [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3), [cy] "=&v"(cy), [g0] "=&v"(g0), [g1] "=&v"(g1),  \
    [g2] "=&v"(g2), [g3] "=&v"(g3), [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3), [t4] "=&v"(t4),  \
    [t5] "=&v"(t5), [t6] "=&v"(t6), [t7] "=&v"(t7), [u0] "=&v"(u0), [u1] "=&v"(u1), [u2] "=&v"(u2), [u3] "=&v"(u3),  \
    [u4] "=&v"(u4), [u5] "=&v"(u5), [u6] "=&v"(u6), [u7] "=&v"(u7), [xb] "=&v"(xb), [j] "=&s"(j)
#define ST_ONE_IN                                                                                                     \
    [lane4] "v"(lane4), [mask] "s"(0xFF00u), [sel] "s"(0x0C0C0700u), [nitems] "s"(s_nitems), [rl] "s"(rl), [rs] "v"(rs), \
    [oo] "v"(oo), [rstep] "s"(s_rstep), ST_IN_OSTEP [nr] "s"(s_nr), [rm0] "s"(rm[0]), [rm1] "s"(rm[1]), [rm2] "s"(rm[2]), \
    [rm3] "s"(rm[3]), [l63] "s"(0x8000000000000000ull), [op] "s"(out_address)
#define ST_ONE_IN_ITEM(U)                                                                                             \
    [xa##U] "v"(xa[U]), [pa##U] "v"(pa[U]), [first##U] "s"(first[U]), [keep##U] "s"(keep[U]), [e##U##x] "v"(e[U].x),  \
    [e##U##y] "v"(e[U].y), [e##U##z] "v"(e[U].z), [e##U##w] "v"(e[U].w)
#define ST_ONE_IN_ITEM_CT(U) [cw##U] "v"(cw[U]), [cm##U] "s"(cm[U])
#define ST_ONE_CLOBBERS                                                                                               \
    "memory", "vcc", "scc", "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", \
    "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", \
    "v123", "v124", "v125", "v126", "v127"

// XMODE 1: x is [gate | up], 2n halves, and the activations are silu(gate) * up (the down projection of a decoder layer, as
// rptc_decompress_matvec_silu).  XMODE 2: the activations are the RMS norm of x + delta times norm_w, and workgroup 0
// writes x + delta to x_out (as rptc_decompress_matvec_rmsnorm; delta may be null).  The same operations in the same
// order as matvec.hip's prologues, so the same bits.
constexpr int kOnePlain = 0, kOneSilu = 1, kOneNorm = 2;
template <int S, int MODE, int MAXI, int XMODE>
__global__ __launch_bounds__(kStThreads) void matvec_one_kernel(
    const uint4 *__restrict__ comp, const uint32_t *__restrict__ codebook, const uint4 *__restrict__ x, int arg_m, int arg_n,
    int rows_per_block, int rw_tail, int items_tail, uint32_t full_magic, uint32_t tail_magic, uint16_t *__restrict__ out,
    const uint4 *delta, const uint4 *__restrict__ norm_w, uint4 *x_out, float eps)
{
    static_assert(MAXI == 3 || MAXI == 4 || MAXI == 6, "a wave holds up to three, four or six elements");
    extern __shared__ uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;   // the table is at LDS address 0
    const int m = arg_m, n = arg_n;
    const int T = n >> 11, Lt = (n & 2047) >> 6, npr = n >> 6, n8 = n >> 3;
    const int items_full = rows_per_block >> 1;
    const int row0 = blockIdx.x * rows_per_block;
    const int rows = min(rows_per_block, m - row0);
    // one layer needs one activation image and one set of partial sums: the set starts where the chain kernel keeps
    // its second image and has 64 KiB
    constexpr int kOnePartBase = kStTableBytes + kStImageBytes;

    // ---- requests first: a thread's share of the activations (16 bytes at 8 idx, two of them) ...
    const int i0 = tid, i1 = tid + kStThreads;
    uint4 xv0 = x[min(i0, n8 - 1)], xv1 = x[min(i1, n8 - 1)];
    uint4 second0 = make_uint4(0, 0, 0, 0), second1 = second0, weight0 = second0, weight1 = second0;
    if constexpr (XMODE == kOneSilu) second0 = x[n8 + min(i0, n8 - 1)], second1 = x[n8 + min(i1, n8 - 1)];
    if constexpr (XMODE == kOneNorm) {
        if (delta) second0 = delta[min(i0, n8 - 1)], second1 = delta[min(i1, n8 - 1)];
        weight0 = norm_w[min(i0, n8 - 1)], weight1 = norm_w[min(i1, n8 - 1)];
    }
    // ... and this wave's elements: equal shares, the first total % 16 waves one more.  Lane -> (row inside the item,
    // element inside the row): two rows of 32 in a full slab; in the ragged slab lane / Lt rows of Lt, the quotient from
    // the host's reciprocal (exact for lane < 64); lanes past the item's last whole row idle on element 0
    const int total = T * items_full + items_tail;
    const int per_wave = (int)((uint32_t)total / kStWaves), extra = (int)((uint32_t)total % kStWaves);
    const int it_begin = wave * per_wave + min(wave, extra);
    const int nitems = per_wave + (wave < extra ? 1 : 0);                // at most MAXI: the host checks
    const int sub_full = lane >> 5, l_full = lane & 31;
    int sub_tail = (int)(((uint32_t)lane * tail_magic) >> 16), l_tail = lane - sub_tail * Lt;
    if (sub_tail >= rw_tail) l_tail = 0;
    uint4 e[MAXI];
    uint32_t cw[MAXI], cm[MAXI], xa[MAXI], pa[MAXI];
    uint64_t first[MAXI], keep[MAXI];
    uint32_t rl = 0;
    int prev_slab = -1;
    const uint64_t first_tail = __builtin_amdgcn_ballot_w64(l_tail == 0);
#pragma unroll
    for (int u = 0; u < MAXI; u++) {
        const int it = it_begin + u;
        const bool mine = u < nitems;
        int slab = items_full == 1 ? it : (int)__umulhi((uint32_t)it, full_magic);
        slab = min(slab, T);
        const int idx = it - slab * items_full;
        const bool full = slab < T;
        const int lanes = full ? 32 : Lt, rpi = full ? 2 : rw_tail;
        const int sub = full ? sub_full : sub_tail, l = full ? l_full : l_tail;
        const int row_first = idx * rpi;
        const int rows_here = mine ? min(rpi, rows - row_first) : 0;          // <= 0: an element past the block's last row
        const bool real = rows_here > 0;
        const uint32_t elem0 = (uint32_t)slab * (uint32_t)m * 32u;
        const uint32_t elem = real ? elem0 + (uint32_t)(row0 + row_first) * (uint32_t)lanes : 0u;
        const uint32_t last = real ? (uint32_t)(rows_here * lanes - 1) : 0u;
        {
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(comp) + (elem + min((uint32_t)lane, last)));
            e[u] = make_uint4(v.x, v.y, v.z, v.w);
        }
        if constexpr (MODE == RPTC_CONTINUOUS) {
            // the word in front of a row: the last word of the row's lane 31 in the slab before
            const bool prev = real && slab > 0;
            const int sub_c = min(sub, max(rows_here, 1) - 1);
            const uint32_t co = prev ? (((uint32_t)(slab - 1) * (uint32_t)m + (uint32_t)(row0 + row_first + sub_c)) * 32u + 31u) * 4u + 3u : 0u;
            cw[u] = reinterpret_cast<const uint32_t *>(comp)[co];
            cm[u] = prev ? ~0u : 0u;
        } else {
            cw[u] = cm[u] = 0u;
        }
        xa[u] = (uint32_t)kStTableBytes + 4u * (uint32_t)(1024 * slab + l);
        pa[u] = (uint32_t)kOnePartBase + 4u * (uint32_t)((row_first + sub) * npr + 32 * slab + l);
        first[u] = full ? 0x0000000100000001ull : first_tail;
        const int nact = max(rows_here, 0) * lanes;
        keep[u] = nact >= 64 ? ~0ull : (1ull << nact) - 1ull;
        if (mine && slab != prev_slab) rl |= 1u << u;
        if (mine) prev_slab = slab;
    }

    // ---- the table: rows 16 wave .. 16 wave + 15 are this wave's to write (as in the chain kernel)
    constexpr int kRowsPerWave = 256 / kStWaves;
    {
        uint32_t cbv[kRowsPerWave];
#pragma unroll
        for (int i = 0; i < kRowsPerWave; i++) cbv[i] = codebook[(kRowsPerWave * wave + i) & ((1 << S) - 1)];
        const uint32_t table_sign = (uint32_t)((kRowsPerWave * wave) >> 7) << 15;
#pragma unroll
        for (int i = 0; i < kRowsPerWave; i++) lds[(kRowsPerWave * wave + i) * 64 + lane] = (cbv[i] & 0xFFFF7FFFu) | table_sign;
    }

    if constexpr (XMODE == kOneSilu) xv0 = silu_mul8(xv0, second0), xv1 = silu_mul8(xv1, second1);
    if constexpr (XMODE == kOneNorm) {
        // as matvec.hip's prologue: packed fp16 residual add, squares as two-term dot products with an fp32 sum, the sum
        // over the workgroup in a fixed order (a wave's lanes, then the sixteen waves), each half scaled and rounded
        // once, a packed fp16 multiply by the weight.  A thread past the end of the vector adds nothing.
        float *red = reinterpret_cast<float *>(lds + kOnePartBase / 4);       // free until the elements' sums go there
        uint32_t r[2][4];
        float ss = 0.f;
        const uint4 xin[2] = {xv0, xv1}, din[2] = {second0, second1}, win[2] = {weight0, weight1};
        const int idx_of[2] = {i0, i1};
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const bool inside = idx_of[u] < n8;
            const uint32_t xw[4] = {xin[u].x, xin[u].y, xin[u].z, xin[u].w}, dw[4] = {din[u].x, din[u].y, din[u].z, din[u].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                r[u][i] = delta ? __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, xw[i]) + __builtin_bit_cast(half2_t, dw[i])) : xw[i];
                if (!inside) r[u][i] = 0u;
                ss = dot2(r[u][i], r[u][i], ss);
            }
            if (blockIdx.x == 0 && inside) x_out[idx_of[u]] = make_uint4(r[u][0], r[u][1], r[u][2], r[u][3]);
        }
        ss = wave_sum(ss);
        if (lane == 63) red[wave] = ss;
        __syncthreads();
        float total_ss = wave_sum(lane < kStWaves ? red[lane] : 0.f);
        total_ss = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, total_ss), 63));
        const float inv = rsqrtf(total_ss / (float)n + eps);
        uint4 hv[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const uint32_t ww[4] = {win[u].x, win[u].y, win[u].z, win[u].w};
            uint32_t h[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const half2_t rv = __builtin_bit_cast(half2_t, r[u][i]);
                half2_t sv;
                sv.x = (_Float16)((float)rv.x * inv);
                sv.y = (_Float16)((float)rv.y * inv);
                h[i] = __builtin_bit_cast(uint32_t, sv * __builtin_bit_cast(half2_t, ww[i]));
            }
            hv[u] = make_uint4(h[0], h[1], h[2], h[3]);
        }
        xv0 = hv[0], xv1 = hv[1];
    }
    // ---- the activations into the image (slot i * n8 + idx for word i of the 16 bytes at 8 idx, inference.cu:215-221;
    // the ragged slab at the full slabs' stride: slot 32 q + l for its q-th step's lane l)
    {
        uint32_t *image = lds + kStTableBytes / 4;
        auto place = [&](int P, uint32_t v) {
            int pos = P;
            if (P >= 1024 * T) {
                const int r = P - 1024 * T, q = (int)(((uint32_t)r * tail_magic) >> 16);
                pos = 1024 * T + 32 * q + (r - q * Lt);
            }
            image[pos] = v;
        };
        if (i0 < n8) {
            place(i0, xv0.x), place(n8 + i0, xv0.y), place(2 * n8 + i0, xv0.z), place(3 * n8 + i0, xv0.w);
        }
        if (i1 < n8) {
            place(i1, xv1.x), place(n8 + i1, xv1.y), place(2 * n8 + i1, xv1.z), place(3 * n8 + i1, xv1.w);
        }
    }

    // ---- the rows (as in the chain kernel)
#ifdef ST_T_ROWS
    const int first_row_wave = extra, row_waves = kStWaves - extra;
#else
    const int first_row_wave = 0, row_waves = 8;
#endif
    const int ri = wave - first_row_wave;
    const uint32_t rs = (uint32_t)kOnePartBase + 4u * (uint32_t)(max(ri, 0) * npr + lane);
    const uint32_t oo = 2u * (uint32_t)(row0 + max(ri, 0));
    const uint32_t rstep = 4u * (uint32_t)(row_waves * npr), ostep = 2u * (uint32_t)row_waves;
    const uint32_t nr = ri >= 0 && ri < row_waves && ri < rows ? (uint32_t)(rows - ri + row_waves - 1) / (uint32_t)row_waves : 0u;
    uint64_t rm[4];
#pragma unroll
    for (int c = 0; c < 4; c++) rm[c] = __builtin_amdgcn_ballot_w64(lane + 64 * c < npr);

    auto uni = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
    auto uni64 = [&](uint64_t v) { return (uint64_t)uni((uint32_t)v) | ((uint64_t)uni((uint32_t)(v >> 32)) << 32); };
    rl = uni(rl);
    const uint32_t s_nitems = uni((uint32_t)nitems), s_nr = uni(nr), s_rstep = uni(rstep);
    [[maybe_unused]] const uint32_t s_ostep = uni(ostep);
#pragma unroll
    for (int u = 0; u < MAXI; u++) first[u] = uni64(first[u]), keep[u] = uni64(keep[u]), cm[u] = uni(cm[u]);
#pragma unroll
    for (int c = 0; c < 4; c++) rm[c] = uni64(rm[c]);
    const uint64_t out_address = uni64(reinterpret_cast<uint64_t>(out));

    uint32_t a0, a1, a2, a3, cy, g0, g1, g2, g3, t0, t1, t2, t3, t4, t5, t6, t7, u0, u1, u2, u3, u4, u5, u6, u7, xb, j;
    if constexpr (MODE == RPTC_AS_WRITTEN && MAXI == 3) {
        asm volatile(ST_ONE_BODY(0, 3) : ST_ONE_OUT : ST_ONE_IN, ST_ONE_IN_ITEM(0), ST_ONE_IN_ITEM(1), ST_ONE_IN_ITEM(2) : ST_ONE_CLOBBERS);
    } else if constexpr (MODE == RPTC_AS_WRITTEN && MAXI == 4) {
        asm volatile(ST_ONE_BODY(0, 4)
                     : ST_ONE_OUT
                     : ST_ONE_IN, ST_ONE_IN_ITEM(0), ST_ONE_IN_ITEM(1), ST_ONE_IN_ITEM(2), ST_ONE_IN_ITEM(3)
                     : ST_ONE_CLOBBERS);
    } else if constexpr (MODE == RPTC_AS_WRITTEN && MAXI == 6) {
        asm volatile(ST_ONE_BODY(0, 6)
                     : ST_ONE_OUT
                     : ST_ONE_IN, ST_ONE_IN_ITEM(0), ST_ONE_IN_ITEM(1), ST_ONE_IN_ITEM(2), ST_ONE_IN_ITEM(3), ST_ONE_IN_ITEM(4), ST_ONE_IN_ITEM(5)
                     : ST_ONE_CLOBBERS);
    } else if constexpr (MAXI == 6) {
        uint32_t own;
        asm volatile(ST_ONE_BODY(1, 6)
                     : ST_ONE_OUT, [own] "=&v"(own)
                     : ST_ONE_IN, ST_ONE_IN_ITEM(0), ST_ONE_IN_ITEM(1), ST_ONE_IN_ITEM(2), ST_ONE_IN_ITEM(3), ST_ONE_IN_ITEM(4), ST_ONE_IN_ITEM(5),
                       ST_ONE_IN_ITEM_CT(0), ST_ONE_IN_ITEM_CT(1), ST_ONE_IN_ITEM_CT(2), ST_ONE_IN_ITEM_CT(3), ST_ONE_IN_ITEM_CT(4),
                       ST_ONE_IN_ITEM_CT(5)
                     : ST_ONE_CLOBBERS);
    } else if constexpr (MAXI == 3) {
        uint32_t own;
        asm volatile(ST_ONE_BODY(1, 3)
                     : ST_ONE_OUT, [own] "=&v"(own)
                     : ST_ONE_IN, ST_ONE_IN_ITEM(0), ST_ONE_IN_ITEM(1), ST_ONE_IN_ITEM(2), ST_ONE_IN_ITEM_CT(0), ST_ONE_IN_ITEM_CT(1),
                       ST_ONE_IN_ITEM_CT(2)
                     : ST_ONE_CLOBBERS);
    } else {
        uint32_t own;
        asm volatile(ST_ONE_BODY(1, 4)
                     : ST_ONE_OUT, [own] "=&v"(own)
                     : ST_ONE_IN, ST_ONE_IN_ITEM(0), ST_ONE_IN_ITEM(1), ST_ONE_IN_ITEM(2), ST_ONE_IN_ITEM(3), ST_ONE_IN_ITEM_CT(0),
                       ST_ONE_IN_ITEM_CT(1), ST_ONE_IN_ITEM_CT(2), ST_ONE_IN_ITEM_CT(3)
                     : ST_ONE_CLOBBERS);
    }
}
#endif

template <typename F>
static int st_set_lds_limit(F *kernel)
{
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
}

#ifndef ST_MFMA
bool matvec_one_fits(int n, int rows_per_block, int items_tail)
{
    const int T = n >> 11, lt = (n & 2047) >> 6;
    const int total = T * (rows_per_block >> 1) + items_tail;
    return (T + (lt ? 1 : 0)) * 4096 <= kStImageBytes && (int64_t)rows_per_block * (n / 64) * 4 <= kStImageBytes + 2 * kStPartBytes &&
           (total + kStWaves - 1) / kStWaves <= 6;
}

int matvec_one_launch(const uint32_t *comp, const uint32_t *codebook, const uint4 *x, uint16_t *out, int m, int n,
                      int rows_per_block, int rw_tail, int items_tail, uint32_t full_magic, int grid, int S, int carry_mode,
                      int prologue, const uint4 *delta, const uint4 *norm_w, uint4 *x_out, float eps, hipStream_t stream)
{
    const int T = n >> 11, lt = (n & 2047) >> 6;
    const int total = T * (rows_per_block >> 1) + items_tail;
    const int per_wave = (total + kStWaves - 1) / kStWaves, max_items = per_wave <= 3 ? 3 : per_wave <= 4 ? 4 : 6;
    const uint32_t tail_magic = lt ? 65536u / (uint32_t)lt + 1u : 0u;       // (v * magic) >> 16 == v / lt for v < 1024
    auto a_comp = reinterpret_cast<const uint4 *>(comp);
#define RPTC_ONE_GO(SS, MM, II, XX)                                                                                  \
    hipLaunchKernelGGL((matvec_one_kernel<SS, MM, II, XX>), dim3(grid), dim3(kStThreads), kStLdsBytes, stream, a_comp, \
                       codebook, x, m, n, rows_per_block, rw_tail, items_tail, full_magic, tail_magic, out, delta, norm_w, x_out, eps)
#define RPTC_ONE_PICK_X(SS, MM, II)                             \
    do {                                                        \
        if (prologue == kOneSilu) RPTC_ONE_GO(SS, MM, II, kOneSilu);      \
        else if (prologue == kOneNorm) RPTC_ONE_GO(SS, MM, II, kOneNorm); \
        else RPTC_ONE_GO(SS, MM, II, kOnePlain);                          \
    } while (0)
#define RPTC_ONE_PICK(SS, MM)                        \
    do {                                             \
        if (max_items == 3) RPTC_ONE_PICK_X(SS, MM, 3); \
        else if (max_items == 4) RPTC_ONE_PICK_X(SS, MM, 4); \
        else RPTC_ONE_PICK_X(SS, MM, 6);             \
    } while (0)
    if (S == 6 && carry_mode == RPTC_AS_WRITTEN) RPTC_ONE_PICK(6, RPTC_AS_WRITTEN);
    else if (S == 6) RPTC_ONE_PICK(6, RPTC_CONTINUOUS);
    else if (carry_mode == RPTC_AS_WRITTEN) RPTC_ONE_PICK(8, RPTC_AS_WRITTEN);
    else RPTC_ONE_PICK(8, RPTC_CONTINUOUS);
#undef RPTC_ONE_PICK
#undef RPTC_ONE_PICK_X
#undef RPTC_ONE_GO
    return (int)hipGetLastError();
}
#else
bool matvec_one_fits(int, int, int) { return false; }
int matvec_one_launch(const uint32_t *, const uint32_t *, const uint4 *, uint16_t *, int, int, int, int, int, uint32_t, int, int, int, int,
                      const uint4 *, const uint4 *, uint4 *, float, hipStream_t)
{
    return RPTC_ESHAPE;
}
#endif

int prepare_matvec_steady()
{
    int rc;
#define RPTC_SET_LIMITS(MAXI)                                                                    \
    if ((rc = st_set_lds_limit(matvec_steady_kernel<6, RPTC_AS_WRITTEN, MAXI>))) return rc;        \
    if ((rc = st_set_lds_limit(matvec_steady_kernel<6, RPTC_CONTINUOUS, MAXI>))) return rc;        \
    if ((rc = st_set_lds_limit(matvec_steady_kernel<8, RPTC_AS_WRITTEN, MAXI>))) return rc;        \
    if ((rc = st_set_lds_limit(matvec_steady_kernel<8, RPTC_CONTINUOUS, MAXI>))) return rc;
    RPTC_SET_LIMITS(3)
    RPTC_SET_LIMITS(4)
#undef RPTC_SET_LIMITS
#ifndef ST_MFMA
#define RPTC_SET_LIMITS(MAXI, GG)                                                             \
    if ((rc = st_set_lds_limit(matvec_one_kernel<6, RPTC_AS_WRITTEN, MAXI, GG>))) return rc;    \
    if ((rc = st_set_lds_limit(matvec_one_kernel<6, RPTC_CONTINUOUS, MAXI, GG>))) return rc;    \
    if ((rc = st_set_lds_limit(matvec_one_kernel<8, RPTC_AS_WRITTEN, MAXI, GG>))) return rc;    \
    if ((rc = st_set_lds_limit(matvec_one_kernel<8, RPTC_CONTINUOUS, MAXI, GG>))) return rc;
    RPTC_SET_LIMITS(3, kOnePlain)
    RPTC_SET_LIMITS(4, kOnePlain)
    RPTC_SET_LIMITS(3, kOneSilu)
    RPTC_SET_LIMITS(4, kOneSilu)
    RPTC_SET_LIMITS(3, kOneNorm)
    RPTC_SET_LIMITS(4, kOneNorm)
    RPTC_SET_LIMITS(6, kOnePlain)
    RPTC_SET_LIMITS(6, kOneSilu)
    RPTC_SET_LIMITS(6, kOneNorm)
#undef RPTC_SET_LIMITS
#endif
    return 0;
}

bool matvec_steady_fits(const LoopLayer &d)
{
    const int T = d.n >> 11, lt = (d.n & 2047) >> 6;
    return (T + (lt ? 1 : 0)) * 4096 <= kStImageBytes && (int64_t)d.rows_per_block * (d.n / 64) * 4 <= kStPartBytes;
}

int matvec_steady_launch(const LoopLayer *device_layers, const LoopLayer &shape, const uint32_t *codebook, int count, int max_items,
                         int grid, int S, int carry_mode, hipStream_t stream)
{
    if (max_items != 3 && max_items != 4) return RPTC_ESHAPE;
#define RPTC_ST_GO(SS, MM, II)                                                                                              \
    hipLaunchKernelGGL((matvec_steady_kernel<SS, MM, II>), dim3(grid), dim3(kStThreads), kStLdsBytes, stream, device_layers, \
                       codebook, count, shape.m, shape.n, shape.rows_per_block, shape.rw_tail, shape.items_tail, shape.full_magic)
#define RPTC_ST_PICK(SS, MM)                     \
    do {                                         \
        if (max_items == 3) RPTC_ST_GO(SS, MM, 3); \
        else RPTC_ST_GO(SS, MM, 4);              \
    } while (0)
    if (S == 6 && carry_mode == RPTC_AS_WRITTEN) RPTC_ST_PICK(6, RPTC_AS_WRITTEN);
    else if (S == 6) RPTC_ST_PICK(6, RPTC_CONTINUOUS);
    else if (carry_mode == RPTC_AS_WRITTEN) RPTC_ST_PICK(8, RPTC_AS_WRITTEN);
    else RPTC_ST_PICK(8, RPTC_CONTINUOUS);
#undef RPTC_ST_PICK
#undef RPTC_ST_GO
    return (int)hipGetLastError();
}

}  // namespace rptc
