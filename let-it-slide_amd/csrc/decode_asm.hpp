// The 32 steps of one stream element as one hand-scheduled instruction block.
//
// The compiler serialises "LDS gather, wait, multiply" per step; here the gathers of 8 steps are
// in flight while the products of the previous 8 are formed, with explicit s_waitcnt.
// Per 8 steps (one shift amount): 4 v_alignbit_b32 (none for shift 0), 4 v_pk_mad_u16 (two
// window hashes each), 8 address ops (v_perm_b32 for the high window, v_and_or_b32 for the low
// one), 8 ds_read_b32, 8 v_dot2c_f32_f16.
#pragma once

#include "rptc_common.hpp"

namespace rptc {

// hash, two addresses, two gathers for window register G (high window -> TH, low window -> TL)
#define RPTC_RD2(G, TH, TL)                                   \
    "v_perm_b32 " TH ", " G ", %[lane4], %[sel]\n"            \
    "v_and_or_b32 " TL ", " G ", %[mask], %[lane4]\n"         \
    "ds_read_b32 " TH ", " TH "\n"                            \
    "ds_read_b32 " TL ", " TL "\n"

#define RPTC_WINDOWS(SH)                                      \
    "v_alignbit_b32 %[g0], %[cy], %[ex], " #SH "\n"           \
    "v_alignbit_b32 %[g1], %[ex], %[ey], " #SH "\n"           \
    "v_alignbit_b32 %[g2], %[ey], %[ez], " #SH "\n"           \
    "v_alignbit_b32 %[g3], %[ez], %[ew], " #SH "\n"           \
    "v_pk_mad_u16 %[g0], %[g0], %[g0], %[g0]\n"               \
    "v_pk_mad_u16 %[g1], %[g1], %[g1], %[g1]\n"               \
    "v_pk_mad_u16 %[g2], %[g2], %[g2], %[g2]\n"               \
    "v_pk_mad_u16 %[g3], %[g3], %[g3], %[g3]\n"

#define RPTC_WINDOWS_SH0                                      \
    "v_pk_mad_u16 %[g0], %[ex], %[ex], %[ex]\n"               \
    "v_pk_mad_u16 %[g1], %[ey], %[ey], %[ey]\n"               \
    "v_pk_mad_u16 %[g2], %[ez], %[ez], %[ez]\n"               \
    "v_pk_mad_u16 %[g3], %[ew], %[ew], %[ew]\n"

#define RPTC_READS(T0, T1, T2, T3, T4, T5, T6, T7)            \
    RPTC_RD2("%[g0]", T0, T1)                                 \
    RPTC_RD2("%[g1]", T2, T3)                                 \
    RPTC_RD2("%[g2]", T4, T5)                                 \
    RPTC_RD2("%[g3]", T6, T7)

// products of block j: {carry,x}: steps 28+j (high), j (low); {x,y}: 16+j, 4+j; {y,z}: 20+j, 8+j;
// {z,w}: 24+j, 12+j
#define RPTC_DOTS(T0, T1, T2, T3, T4, T5, T6, T7, XA, XB, XC, XD, XE, XF, XG, XH) \
    "v_dot2c_f32_f16 %[a0], " T0 ", %[" XA "]\n"              \
    "v_dot2c_f32_f16 %[a1], " T1 ", %[" XB "]\n"              \
    "v_dot2c_f32_f16 %[a2], " T2 ", %[" XC "]\n"              \
    "v_dot2c_f32_f16 %[a3], " T3 ", %[" XD "]\n"              \
    "v_dot2c_f32_f16 %[a0], " T4 ", %[" XE "]\n"              \
    "v_dot2c_f32_f16 %[a1], " T5 ", %[" XF "]\n"              \
    "v_dot2c_f32_f16 %[a2], " T6 ", %[" XG "]\n"              \
    "v_dot2c_f32_f16 %[a3], " T7 ", %[" XH "]\n"

// the first products of an element start the four sums (no accumulator to clear beforehand)
#define RPTC_DOTS_FIRST(T0, T1, T2, T3, T4, T5, T6, T7, XA, XB, XC, XD, XE, XF, XG, XH) \
    "v_dot2_f32_f16 %[a0], " T0 ", %[" XA "], 0\n"           \
    "v_dot2_f32_f16 %[a1], " T1 ", %[" XB "], 0\n"           \
    "v_dot2_f32_f16 %[a2], " T2 ", %[" XC "], 0\n"           \
    "v_dot2_f32_f16 %[a3], " T3 ", %[" XD "], 0\n"           \
    "v_dot2c_f32_f16 %[a0], " T4 ", %[" XE "]\n"             \
    "v_dot2c_f32_f16 %[a1], " T5 ", %[" XF "]\n"             \
    "v_dot2c_f32_f16 %[a2], " T6 ", %[" XG "]\n"             \
    "v_dot2c_f32_f16 %[a3], " T7 ", %[" XH "]\n"

// one more expansion pass so that a register-list macro can stand for eight arguments
#define RPTC_READS_X(...) RPTC_READS(__VA_ARGS__)
#define RPTC_DOTS_X(...) RPTC_DOTS(__VA_ARGS__)
#define RPTC_DOTS_FIRST_X(...) RPTC_DOTS_FIRST(__VA_ARGS__)

#define RPTC_TA "%[t0]", "%[t1]", "%[t2]", "%[t3]", "%[t4]", "%[t5]", "%[t6]", "%[t7]"
#define RPTC_TB "%[u0]", "%[u1]", "%[u2]", "%[u3]", "%[u4]", "%[u5]", "%[u6]", "%[u7]"

// lane4: LDS address of this lane's copy of table row 0.  xr[q]: activation pair of step q.
// a0..a3 receive four partial sums of the element's 32 products (they are written, not added to).
// The 16 bits in front of the element are the end of the previous lane's last word, except in the
// lanes of `first_lanes` (the first element of a row), which take the end of `own`.
// WAIT_VMCNT >= 0: the block starts with s_waitcnt vmcnt(WAIT_VMCNT).  For a caller that issued the load of `e`
// (and `own`) by hand and has not touched those registers since: nothing outside this block then reads them
// before they have arrived.
#define RPTC_DECODE_BODY                                                                              \
        /* a DPP operand must not have been written by a vector op in the two instructions before */ \
        "s_nop 1\n"                                                                                   \
        "s_mov_b64 vcc, %[first]\n"                                                                   \
        "v_cndmask_b32_dpp %[cy], %[ew], %[own], vcc wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n" \
        RPTC_WINDOWS(12) RPTC_READS_X(RPTC_TA)                                                        \
        RPTC_WINDOWS(8) RPTC_READS_X(RPTC_TB)                                                         \
        "s_waitcnt lgkmcnt(8)\n"                                                                      \
        RPTC_DOTS_FIRST_X(RPTC_TA, "x28", "x0", "x16", "x4", "x20", "x8", "x24", "x12")               \
        RPTC_WINDOWS(4) RPTC_READS_X(RPTC_TA)                                                         \
        "s_waitcnt lgkmcnt(8)\n"                                                                      \
        RPTC_DOTS_X(RPTC_TB, "x29", "x1", "x17", "x5", "x21", "x9", "x25", "x13")                     \
        RPTC_WINDOWS_SH0 RPTC_READS_X(RPTC_TB)                                                        \
        "s_waitcnt lgkmcnt(8)\n"                                                                      \
        RPTC_DOTS_X(RPTC_TA, "x30", "x2", "x18", "x6", "x22", "x10", "x26", "x14")                    \
        "s_waitcnt lgkmcnt(0)\n"                                                                      \
        RPTC_DOTS_X(RPTC_TB, "x31", "x3", "x19", "x7", "x23", "x11", "x27", "x15")                    \
        /* a dot product's result must not be read by another kind of VALU op for 3 wait states, */  \
        /* and the compiler cannot see inside this block */                                          \
        "s_nop 3\n"
#define RPTC_DECODE_OUTPUTS                                                                           \
          [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3),                             \
          [cy] "=&v"(carry), [g0] "=&v"(g0), [g1] "=&v"(g1), [g2] "=&v"(g2), [g3] "=&v"(g3),          \
          [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3),                             \
          [t4] "=&v"(t4), [t5] "=&v"(t5), [t6] "=&v"(t6), [t7] "=&v"(t7),                             \
          [u0] "=&v"(u0), [u1] "=&v"(u1), [u2] "=&v"(u2), [u3] "=&v"(u3),                             \
          [u4] "=&v"(u4), [u5] "=&v"(u5), [u6] "=&v"(u6), [u7] "=&v"(u7)
#define RPTC_DECODE_INPUTS                                                                            \
          [ex] "v"(e.x), [ey] "v"(e.y), [ez] "v"(e.z), [ew] "v"(e.w), [own] "v"(own), [first] "s"(first_lanes), \
          [lane4] "v"(lane4), [mask] "s"(0xFF00u), [sel] "s"(0x0C0C0700u),                            \
          [x0] "v"(xr[0]), [x1] "v"(xr[1]), [x2] "v"(xr[2]), [x3] "v"(xr[3]),                         \
          [x4] "v"(xr[4]), [x5] "v"(xr[5]), [x6] "v"(xr[6]), [x7] "v"(xr[7]),                         \
          [x8] "v"(xr[8]), [x9] "v"(xr[9]), [x10] "v"(xr[10]), [x11] "v"(xr[11]),                     \
          [x12] "v"(xr[12]), [x13] "v"(xr[13]), [x14] "v"(xr[14]), [x15] "v"(xr[15]),                 \
          [x16] "v"(xr[16]), [x17] "v"(xr[17]), [x18] "v"(xr[18]), [x19] "v"(xr[19]),                 \
          [x20] "v"(xr[20]), [x21] "v"(xr[21]), [x22] "v"(xr[22]), [x23] "v"(xr[23]),                 \
          [x24] "v"(xr[24]), [x25] "v"(xr[25]), [x26] "v"(xr[26]), [x27] "v"(xr[27]),                 \
          [x28] "v"(xr[28]), [x29] "v"(xr[29]), [x30] "v"(xr[30]), [x31] "v"(xr[31])

template <int WAIT_VMCNT = -1, typename E>
__device__ __forceinline__ void decode_element_asm(const E &e, const uint32_t own, const uint64_t first_lanes,
                                                   const uint32_t lane4, const uint32_t (&xr)[32], float &a0,
                                                   float &a1, float &a2, float &a3)
{
    uint32_t carry;
    uint32_t g0, g1, g2, g3, t0, t1, t2, t3, t4, t5, t6, t7, u0, u1, u2, u3, u4, u5, u6, u7;
    if constexpr (WAIT_VMCNT >= 0) {
        asm volatile("s_waitcnt vmcnt(%[vm])\n" RPTC_DECODE_BODY
                     : RPTC_DECODE_OUTPUTS
                     : RPTC_DECODE_INPUTS, [vm] "n"(WAIT_VMCNT)
                     : "vcc", "memory");
    } else {
        asm volatile(RPTC_DECODE_BODY : RPTC_DECODE_OUTPUTS : RPTC_DECODE_INPUTS : "vcc");
    }
}

// The same block for 4 bits per weight: a step consumes 8 stream bits, an element is 8 words, and the
// window of step s is the 16 bits that end 8 (s + 1) bits into the element.  Word i as it is holds the
// windows of steps 4i + 1 (high half) and 4i + 3 (low half); the 32 bits that start 8 bits before word
// i - one v_alignbit_b32 with the word in front (the previous lane's last word for i = 0) - hold those
// of steps 4i and 4i + 2.  Per two words: 2 v_alignbit_b32, 4 v_pk_mad_u16, 8 address ops, 8 gathers,
// 8 products.
#define RPTC_WINDOWS4(WP, WA, WB)                             \
    "v_alignbit_b32 %[g0], " WP ", " WA ", 8\n"               \
    "v_alignbit_b32 %[g2], " WA ", " WB ", 8\n"               \
    "v_pk_mad_u16 %[g0], %[g0], %[g0], %[g0]\n"               \
    "v_pk_mad_u16 %[g1], " WA ", " WA ", " WA "\n"            \
    "v_pk_mad_u16 %[g2], %[g2], %[g2], %[g2]\n"               \
    "v_pk_mad_u16 %[g3], " WB ", " WB ", " WB "\n"

// xs[q]: activation pair of the q-th step in stream order.  The gathers of a block of eight steps land
// in the order of steps 0, 2, 1, 3, 4, 6, 5, 7 of the block.
__device__ __forceinline__ void decode_element_asm4(const uint32_t (&w)[8], const uint32_t own, const uint64_t first_lanes,
                                                    const uint32_t lane4, const uint32_t (&xs)[32], float &a0,
                                                    float &a1, float &a2, float &a3)
{
    uint32_t carry;
    uint32_t g0, g1, g2, g3, t0, t1, t2, t3, t4, t5, t6, t7, u0, u1, u2, u3, u4, u5, u6, u7;
    asm volatile(
        "s_nop 1\n"
        "s_mov_b64 vcc, %[first]\n"
        "v_cndmask_b32_dpp %[cy], %[w7], %[own], vcc wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n"
        RPTC_WINDOWS4("%[cy]", "%[w0]", "%[w1]") RPTC_READS_X(RPTC_TA)
        RPTC_WINDOWS4("%[w1]", "%[w2]", "%[w3]") RPTC_READS_X(RPTC_TB)
        "s_waitcnt lgkmcnt(8)\n"
        RPTC_DOTS_FIRST_X(RPTC_TA, "x0", "x2", "x1", "x3", "x4", "x6", "x5", "x7")
        RPTC_WINDOWS4("%[w3]", "%[w4]", "%[w5]") RPTC_READS_X(RPTC_TA)
        "s_waitcnt lgkmcnt(8)\n"
        RPTC_DOTS_X(RPTC_TB, "x8", "x10", "x9", "x11", "x12", "x14", "x13", "x15")
        RPTC_WINDOWS4("%[w5]", "%[w6]", "%[w7]") RPTC_READS_X(RPTC_TB)
        "s_waitcnt lgkmcnt(8)\n"
        RPTC_DOTS_X(RPTC_TA, "x16", "x18", "x17", "x19", "x20", "x22", "x21", "x23")
        "s_waitcnt lgkmcnt(0)\n"
        RPTC_DOTS_X(RPTC_TB, "x24", "x26", "x25", "x27", "x28", "x30", "x29", "x31")
        "s_nop 3\n"
        : [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3),
          [cy] "=&v"(carry), [g0] "=&v"(g0), [g1] "=&v"(g1), [g2] "=&v"(g2), [g3] "=&v"(g3),
          [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3),
          [t4] "=&v"(t4), [t5] "=&v"(t5), [t6] "=&v"(t6), [t7] "=&v"(t7),
          [u0] "=&v"(u0), [u1] "=&v"(u1), [u2] "=&v"(u2), [u3] "=&v"(u3),
          [u4] "=&v"(u4), [u5] "=&v"(u5), [u6] "=&v"(u6), [u7] "=&v"(u7)
        : [w0] "v"(w[0]), [w1] "v"(w[1]), [w2] "v"(w[2]), [w3] "v"(w[3]), [w4] "v"(w[4]), [w5] "v"(w[5]),
          [w6] "v"(w[6]), [w7] "v"(w[7]), [own] "v"(own), [first] "s"(first_lanes),
          [lane4] "v"(lane4), [mask] "s"(0xFF00u), [sel] "s"(0x0C0C0700u),
          [x0] "v"(xs[0]), [x1] "v"(xs[1]), [x2] "v"(xs[2]), [x3] "v"(xs[3]),
          [x4] "v"(xs[4]), [x5] "v"(xs[5]), [x6] "v"(xs[6]), [x7] "v"(xs[7]),
          [x8] "v"(xs[8]), [x9] "v"(xs[9]), [x10] "v"(xs[10]), [x11] "v"(xs[11]),
          [x12] "v"(xs[12]), [x13] "v"(xs[13]), [x14] "v"(xs[14]), [x15] "v"(xs[15]),
          [x16] "v"(xs[16]), [x17] "v"(xs[17]), [x18] "v"(xs[18]), [x19] "v"(xs[19]),
          [x20] "v"(xs[20]), [x21] "v"(xs[21]), [x22] "v"(xs[22]), [x23] "v"(xs[23]),
          [x24] "v"(xs[24]), [x25] "v"(xs[25]), [x26] "v"(xs[26]), [x27] "v"(xs[27]),
          [x28] "v"(xs[28]), [x29] "v"(xs[29]), [x30] "v"(xs[30]), [x31] "v"(xs[31])
        : "vcc");
}

}  // namespace rptc
