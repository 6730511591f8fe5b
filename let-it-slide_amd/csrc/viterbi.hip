// Viterbi search for the hashed pair stream: the quantizer's inner loop.
//
// The search is the reference's (rptc.py:13-71, diag_only path): path costs rho over all trellis
// states, rho[0] = 0 and infinity elsewhere at the start (rptc.py:55-56), per step the cheapest
// of the predecessors of every state (rptc.py:27-28, first index on ties as argmin does) plus the
// step's squared error (rptc.py:32), the cheapest end state traced back (rptc.py:60-65).  The
// trellis is the one the inference kernels decode (inference.cu:250-262): 65536 states, a step
// shifts 4 new bits in and emits the two weights the state's hash selects, so a state s' has the
// 16 predecessors (d << 12) | (s' >> 4).
//
// (The 3- and 4-bit streams take 6 and 8 bits a step: 64 and 256 predecessors, see vit_state.)
// One workgroup of 1024 threads searches one row.  Thread j keeps the costs of 64 states in
// registers: the four predecessor groups g = 4j .. 4j+3 with all 16 values of d, so the minimum
// over a group's predecessors never leaves the thread.  A step is
//   1. every thread: the minimum and its d for its four groups -> LDS (16 KiB) and the back
//      pointers (4 bits a group) -> memory; and the step's error for each distinct (entry, sign)
//      pair (256 of them at S = 8, where the sign is the entry's top bit; 128 at S = 6) -> an LDS
//      table with 32 copies of every value, so that the gathers below are free of bank conflicts;
//   2. barrier; every thread: new cost of its 64 states = minimum of the state's group (16 LDS
//      reads, each shared by four states) + the error of the state's pair (64 gathers).
// Both LDS tables are double-buffered, which makes the one barrier enough.
// All sums are fp32 in the order of the host-side restatement (rptc_kernels/quantize.py), with
// contraction off, so the chosen path is the same bit for bit.  The trace back is a second kernel
// with one thread per row: a chain of dependent loads, run for all rows side by side.
//
// viterbi_scalar_kernel is the same search on the reference's own trellis (rptc.py:13-71 as it
// stands: 2^L states, 2 bits a step, one value a state from an arbitrary alphabet — the stream
// decompress and decompress_matvec_t_* decode).  A state has four predecessors, thread j owns
// 2^L / 4096 predecessor groups with all four d, and with no structure in the alphabet a thread
// keeps its states' values in registers (two fp16 a register) and computes the error itself.
#include "rptc_common.hpp"

#include <math.h>

namespace rptc {

constexpr int kVitThreads = 1024;
constexpr int kVitGroups = 4096;           // states >> 4
constexpr int kVitCopies = 32;             // copies of a loss value, one per LDS bank
constexpr int kVitLossRow = 64;            // floats in a table row (256 bytes): 32 copies for even steps, 32 for odd
constexpr int kVitLossFloats = 256 * kVitLossRow;
constexpr int kVitLdsBytes = (kVitLossFloats + 2 * kVitGroups) * 4 + 2 * kVitThreads * 4;

#pragma clang fp contract(off)
__device__ __forceinline__ float pair_loss(float x0, float x1, float w0, float w1)
{
    const float d0 = x0 - w0, d1 = x1 - w1;
    return d0 * d0 + d1 * d1;
}

__device__ __forceinline__ float pair_loss_weighted(float x0, float x1, float w0, float w1, float c0, float c1)
{
    const float d0 = x0 - w0, d1 = x1 - w1;
    return c0 * (d0 * d0) + c1 * (d1 * d1);
}

// Which state register r of thread j holds, for a trellis that takes STEP bits per step (a state has
// 2^STEP predecessors (d << (16 - STEP)) | group, group = state >> STEP):
//   STEP 4: r = 16 * gi + d, state (d << 12) | (4j + gi): four groups with their 16 predecessors;
//   STEP 6: r = d,           state (d << 10) | j:          one group with its 64 predecessors;
//   STEP 8: r = d % 64,      state (d << 8) | (j / 4), d = 64 * (j % 4) + r: a quarter of a group's 256
//           predecessors; the four lanes of a group finish the minimum with two shuffles.
template <int STEP>
__device__ __forceinline__ uint32_t vit_state(int r, int j)
{
    if (STEP == 4) return ((uint32_t)(r & 15) << 12) | (uint32_t)(4 * j + (r >> 4));
    if (STEP == 6) return ((uint32_t)r << 10) | (uint32_t)j;
    return ((uint32_t)(64 * (j & 3) + r) << 8) | (uint32_t)(j >> 2);
}

template <int S, int STEP, bool WEIGHTED>
__global__ __launch_bounds__(kVitThreads) void viterbi_pairs_kernel(
    const float *__restrict__ targets, const float *__restrict__ weights, int64_t weights_row_stride,
    const uint16_t *__restrict__ codebook, uint16_t *__restrict__ back, int32_t *__restrict__ end_state,
    float *__restrict__ cost, int steps)
{
    extern __shared__ float lds[];
    // The loss table is the first thing in LDS and the kernel has no static LDS, so it starts at
    // LDS address 0 and a 16-bit byte offset reaches all of it.
    float *loss = lds;                                  // [256][2][32]: a row holds 32 copies for even steps, 32 for odd
    float *best = lds + kVitLossFloats;                 // [2][4096]
    float *red_v = best + 2 * kVitGroups;               // [1024]
    int *red_i = reinterpret_cast<int *>(red_v + kVitThreads);

    const int j = threadIdx.x, copy = j & (kVitCopies - 1);
    const int64_t row = blockIdx.x;
    const uint32_t loss_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(loss));

    // code[r / 4] byte r % 4 is the row of the loss table the state of register r reads: its codebook entry, with the hash's sign bit on top at S = 6
    // (at S = 8 the sign bit is the entry's own top bit, inference.cu:253-262).  A row starts every
    // 256 bytes, so one byte permute makes the address out of the code and the thread's copy.
    float rho[64];
    uint32_t code[16];
#pragma unroll
    for (int r = 0; r < 64; r++) {
        const uint32_t s = vit_state<STEP>(r, j);
        const uint32_t prod = s * (s + 1u);
        const uint32_t c = S == 8 ? (prod >> 8) & 0xFFu : ((prod >> 8) & 63u) | (((prod >> 15) & 1u) << 6);
        if (r & 3) code[r >> 2] |= c << (8 * (r & 3));
        else code[r >> 2] = c;
        rho[r] = (s == 0) ? 0.f : INFINITY;
    }
    const uint32_t copy4 = loss_base + 4u * (uint32_t)copy;

    // the table row this thread fills: four threads a row, 8 copies each
    const int c_mine = (j >> 2) & (S == 8 ? 255 : 127);
    const int e_mine = S == 8 ? c_mine : c_mine & 63;
    const bool neg_mine = S == 8 ? (c_mine >> 7) != 0 : (c_mine >> 6) != 0;
    const float w0 = fabsf(half_bits_to_float(codebook[2 * e_mine])) * (neg_mine ? -1.f : 1.f);
    const float w1 = half_bits_to_float(codebook[2 * e_mine + 1]);
    float4 *loss_mine = reinterpret_cast<float4 *>(loss + c_mine * kVitLossRow + (j & 3) * 8);

    const float *tg = targets + row * steps * 2;
    const float *wt = WEIGHTED ? weights + row * weights_row_stride : nullptr;
    uint16_t *back_row = back + row * steps * (int64_t)kVitThreads;
    float x0 = tg[0], x1 = tg[1], c0 = WEIGHTED ? wt[0] : 1.f, c1 = WEIGHTED ? wt[1] : 1.f;
    for (int t = 0; t < steps; t++) {
        // the next step's targets are on their way while this step is computed
        const int tn = t + 1 < steps ? t + 1 : t;
        const float nx0 = tg[2 * tn], nx1 = tg[2 * tn + 1];
        const float nc0 = WEIGHTED ? wt[2 * tn] : 1.f, nc1 = WEIGHTED ? wt[2 * tn + 1] : 1.f;

        const float l = WEIGHTED ? pair_loss_weighted(x0, x1, w0, w1, c0, c1) : pair_loss(x0, x1, w0, w1);
        const float4 l4 = make_float4(l, l, l, l);
        // Both LDS tables have two halves that take turns, so a step needs one barrier: what this
        // step overwrites was last read two steps ago, before the previous step's barrier.
        float4 *lm = loss_mine + (t & 1) * (kVitCopies / 4);
        lm[0] = l4;
        lm[1] = l4;

        float *bw = best + (t & 1) * kVitGroups;
        const uint32_t copy4_t = copy4 + (uint32_t)(t & 1) * (kVitCopies * 4u);
        // byte 0 of a gather's address: the copy's offset; byte 1: the state's code; the rest zero
        auto loss_of = [&](int r) {
            const uint32_t off = perm(code[r >> 2], copy4_t, 0x0C0C0400u + ((uint32_t)(r & 3) << 8));
            return __builtin_bit_cast(float, lds_read_abs(off));
        };
        if constexpr (STEP == 4) {
            uint32_t nib = 0;
#pragma unroll
            for (int gi = 0; gi < 4; gi++) {
                float m = rho[16 * gi];
                uint32_t arg = 0;
#pragma unroll
                for (int d = 1; d < 16; d++) {
                    const bool lt = rho[16 * gi + d] < m;      // the first minimum wins
                    m = lt ? rho[16 * gi + d] : m;
                    arg = lt ? (uint32_t)d : arg;
                }
                bw[4 * j + gi] = m;
                nib |= arg << (4 * gi);
            }
            back_row[(int64_t)t * kVitThreads + j] = (uint16_t)nib;
            __syncthreads();
            // state (d << 12) | g comes from group ((d << 12) | g) >> 4 = (d << 8) | (j >> 2) for all four g
#pragma unroll
            for (int d = 0; d < 16; d++) {
                const float b = bw[(d << 8) | (j >> 2)];
#pragma unroll
                for (int gi = 0; gi < 4; gi++) rho[16 * gi + d] = b + loss_of(16 * gi + d);
                // a few gathers in flight at a time: all 64 at once would push registers out to memory
                if ((d & 1) == 1) __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            float m = rho[0];
            uint32_t arg = STEP == 8 ? 64u * (uint32_t)(j & 3) : 0u;
#pragma unroll
            for (int r = 1; r < 64; r++) {
                const bool lt = rho[r] < m;                    // the first minimum wins
                m = lt ? rho[r] : m;
                arg = lt ? (STEP == 8 ? 64u * (uint32_t)(j & 3) : 0u) + (uint32_t)r : arg;
            }
            if constexpr (STEP == 8) {
                // the other three quarters of the group sit in the neighbouring lanes; equal minima
                // go to the lower d, i.e. the lower lane
#pragma unroll
                for (int off = 1; off <= 2; off <<= 1) {
                    const float om = __shfl_xor(m, off, 64);
                    const uint32_t oarg = __shfl_xor(arg, off, 64);
                    const bool take = om < m || (om == m && oarg < arg);
                    m = take ? om : m;
                    arg = take ? oarg : arg;
                }
                if ((j & 3) == 0) {
                    bw[j >> 2] = m;
                    back_row[(int64_t)t * kVitThreads + j] = (uint16_t)arg;
                }
            } else {
                bw[j] = m;
                back_row[(int64_t)t * kVitThreads + j] = (uint16_t)arg;
            }
            __syncthreads();
            // STEP 6: state (d << 10) | j comes from group (d << 4) | (j >> 6);
            // STEP 8: state (d << 8) | g comes from group d
#pragma unroll
            for (int r = 0; r < 64; r++) {
                const float b = STEP == 6 ? bw[(r << 4) | (j >> 6)] : bw[64 * (j & 3) + r];
                rho[r] = b + loss_of(r);
                if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
            }
        }
        x0 = nx0, x1 = nx1, c0 = nc0, c1 = nc1;
    }

    // cheapest end state, the lowest index among equals: in a thread the states are visited in
    // rising order (STEP 4: d outer, gi inner; otherwise r)
    float mv = rho[0];
    int mi = (int)vit_state<STEP>(0, j);
#pragma unroll
    for (int a = 0; a < 64; a++) {
        const int r = STEP == 4 ? 16 * (a & 3) + (a >> 2) : a;
        const float v = rho[r];
        if (v < mv) {
            mv = v;
            mi = (int)vit_state<STEP>(r, j);
        }
    }
    red_v[j] = mv;
    red_i[j] = mi;
    __syncthreads();
    for (int width = kVitThreads / 2; width > 0; width >>= 1) {
        if (j < width) {
            const float ov = red_v[j + width];
            const int oi = red_i[j + width];
            if (ov < red_v[j] || (ov == red_v[j] && oi < red_i[j])) {
                red_v[j] = ov;
                red_i[j] = oi;
            }
        }
        __syncthreads();
    }
    if (j == 0) {
        end_state[row] = red_i[0];
        cost[row] = red_v[0];
    }
}

// The same search on the trellis of the reference's rptc_lite.py (quantize, rptc_lite.py:19-60) for L = 16, R = 4, V = 2,
// the parameters its own driver uses (rptc_lite.py:134-139): state s' emits alphabet[index_fn(s')] (rptc_lite.py:12-16,27-29),
// a row of an fp32 alphabet of 2^S pairs, S <= 9, and a step costs sum_v importance[t][v] * (samples[t][v] - value)^2
// (rptc_lite.py:39).  Structure of viterbi_pairs_kernel<., 4, .>; what differs is the loss table: up to 512 distinct
// values a step instead of 256, so a row has 16 copies a step parity (128 bytes a row, 64 KiB in all) and a gather meets
// another lane's in the same bank about every second time; and a state's row number needs 9 bits, so the codes are 16-bit
// halves (the row's byte offset, ready to be or-ed with the copy's offset), two a register.
template <bool WEIGHTED>
__global__ __launch_bounds__(kVitThreads) void viterbi_lite_kernel(
    const float *__restrict__ targets, const float *__restrict__ weights, int64_t weights_row_stride,
    const float *__restrict__ alphabet, int S, uint16_t *__restrict__ back, int32_t *__restrict__ end_state,
    float *__restrict__ cost, int steps)
{
    extern __shared__ float lds[];
    constexpr int kCopies = 16, kRow = 2 * kCopies;     // floats in a table row: 16 copies for even steps, 16 for odd
    float *loss = lds;                                  // [512][2][16], at LDS address 0 (see viterbi_pairs_kernel)
    float *best = lds + kVitLossFloats;                 // [2][4096]
    float *red_v = best + 2 * kVitGroups;               // [1024]
    int *red_i = reinterpret_cast<int *>(red_v + kVitThreads);
    static_assert(512 * kRow == kVitLossFloats, "the table takes the room of the pair search's");

    const int j = threadIdx.x, copy = j & (kCopies - 1);
    const int64_t row = blockIdx.x;
    const uint32_t loss_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(loss));

    float rho[64];
    uint32_t code[32];                                  // half r % 2 of code[r / 2]: 128 * index_fn(state of register r)
#pragma unroll
    for (int r = 0; r < 64; r++) {
        const uint32_t st = vit_state<4>(r, j);
        uint32_t x = st * (2u * st + 1u);               // index_fn: only bits below 16 reach the result when L = 16
        x ^= x >> (16 - S);
        const uint32_t c = (x & ((1u << S) - 1u)) * (kRow * 4u);
        if (r & 1) code[r >> 1] |= c << 16;
        else code[r >> 1] = c;
        rho[r] = (st == 0) ? 0.f : INFINITY;
    }
    const uint32_t copy4 = loss_base + 4u * (uint32_t)copy;

    // the table row this thread fills: two threads a row, 8 copies each
    const int e_mine = (j >> 1) & ((1 << S) - 1);
    const float w0 = alphabet[2 * e_mine], w1 = alphabet[2 * e_mine + 1];
    float4 *loss_mine = reinterpret_cast<float4 *>(loss + e_mine * kRow + (j & 1) * 8);

    const float *tg = targets + row * steps * 2;
    const float *wt = WEIGHTED ? weights + row * weights_row_stride : nullptr;
    uint16_t *back_row = back + row * steps * (int64_t)kVitThreads;
    float x0 = tg[0], x1 = tg[1], c0 = WEIGHTED ? wt[0] : 1.f, c1 = WEIGHTED ? wt[1] : 1.f;
    for (int t = 0; t < steps; t++) {
        const int tn = t + 1 < steps ? t + 1 : t;
        const float nx0 = tg[2 * tn], nx1 = tg[2 * tn + 1];
        const float nc0 = WEIGHTED ? wt[2 * tn] : 1.f, nc1 = WEIGHTED ? wt[2 * tn + 1] : 1.f;

        const float l = WEIGHTED ? pair_loss_weighted(x0, x1, w0, w1, c0, c1) : pair_loss(x0, x1, w0, w1);
        const float4 l4 = make_float4(l, l, l, l);
        float4 *lm = loss_mine + (t & 1) * (kCopies / 4);
        lm[0] = l4;
        lm[1] = l4;

        float *bw = best + (t & 1) * kVitGroups;
        const uint32_t copy4_t = copy4 + (uint32_t)(t & 1) * (kCopies * 4u);
        auto loss_of = [&](int r) {
            const uint32_t off = (r & 1) ? (code[r >> 1] >> 16) | copy4_t : and_or(code[r >> 1], 0xFFFFu, copy4_t);
            return __builtin_bit_cast(float, lds_read_abs(off));
        };
        uint32_t nib = 0;
#pragma unroll
        for (int gi = 0; gi < 4; gi++) {
            float m = rho[16 * gi];
            uint32_t arg = 0;
#pragma unroll
            for (int d = 1; d < 16; d++) {
                const bool lt = rho[16 * gi + d] < m;          // the first minimum wins (argmin, rptc_lite.py:34)
                m = lt ? rho[16 * gi + d] : m;
                arg = lt ? (uint32_t)d : arg;
            }
            bw[4 * j + gi] = m;
            nib |= arg << (4 * gi);
        }
        back_row[(int64_t)t * kVitThreads + j] = (uint16_t)nib;
        __syncthreads();
#pragma unroll
        for (int d = 0; d < 16; d++) {
            const float b = bw[(d << 8) | (j >> 2)];
#pragma unroll
            for (int gi = 0; gi < 4; gi++) rho[16 * gi + d] = b + loss_of(16 * gi + d);
            if ((d & 1) == 1) __builtin_amdgcn_sched_barrier(0);
        }
        x0 = nx0, x1 = nx1, c0 = nc0, c1 = nc1;
    }

    // cheapest end state, the lowest index among equals (argmin, rptc_lite.py:52)
    float mv = rho[0];
    int mi = (int)vit_state<4>(0, j);
#pragma unroll
    for (int a = 0; a < 64; a++) {
        const int r = 16 * (a & 3) + (a >> 2);
        const float v = rho[r];
        if (v < mv) {
            mv = v;
            mi = (int)vit_state<4>(r, j);
        }
    }
    red_v[j] = mv;
    red_i[j] = mi;
    __syncthreads();
    for (int width = kVitThreads / 2; width > 0; width >>= 1) {
        if (j < width) {
            const float ov = red_v[j + width];
            const int oi = red_i[j + width];
            if (ov < red_v[j] || (ov == red_v[j] && oi < red_i[j])) {
                red_v[j] = ov;
                red_i[j] = oi;
            }
        }
        __syncthreads();
    }
    if (j == 0) {
        end_state[row] = red_i[0];
        cost[row] = red_v[0];
    }
}

// x - (fp16 in the low / high half of v) in one op: x * 1.0 + (-half), the product exact, so the
// result is the correctly rounded difference.  Written as asm also because the conversion alone
// does not change from step to step: the compiler would convert all values once and keep them as
// fp32, twice the registers.
__device__ __forceinline__ float sub_half_lo(float x, uint32_t v)
{
    float d;
    asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel_hi:[0,0,1]" : "=v"(d) : "v"(x), "v"(v));
    return d;
}

__device__ __forceinline__ float sub_half_hi(float x, uint32_t v)
{
    float d;
    asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "=v"(d) : "v"(x), "v"(v));
    return d;
}

constexpr int scalar_lds_bytes(int L) { return 2 * ((1 << L) / 4) * 4 + 2 * kVitThreads * 4; }

// L = 16 or 14.  NG = predecessor groups per thread; register r = 4 * gi + d holds state
// (d << (L-2)) | (NG * j + gi).  Back pointers: 2 bits a group, one 32-bit word per thread and step.
template <int L, bool WEIGHTED>
__global__ __launch_bounds__(kVitThreads) void viterbi_scalar_kernel(
    const float *__restrict__ targets, const float *__restrict__ weights, int64_t weights_row_stride,
    const uint16_t *__restrict__ alphabet, uint32_t *__restrict__ back, int32_t *__restrict__ end_state,
    float *__restrict__ cost, int steps)
{
    constexpr int M = 1 << L, G = M / 4, NG = G / kVitThreads, NS = 4 * NG;
    static_assert(NG % 4 == 0, "four consecutive groups of a thread share a minimum");
    extern __shared__ float lds[];
    float *best = lds;                                  // [2][G]
    float *red_v = best + 2 * G;                        // [1024]
    int *red_i = reinterpret_cast<int *>(red_v + kVitThreads);
    const int j = threadIdx.x;
    const int64_t row = blockIdx.x;

    float rho[NS];
    uint32_t val[NS / 2];                               // the states' alphabet values, two fp16 a register
#pragma unroll
    for (int r = 0; r < NS; r++) {
        const uint32_t s = ((uint32_t)(r & 3) << (L - 2)) | (uint32_t)(NG * j + (r >> 2));
        const uint32_t a = alphabet[s];
        if (r & 1) val[r >> 1] |= a << 16;
        else val[r >> 1] = a;
        rho[r] = (s == 0) ? 0.f : INFINITY;
    }
    const float *tg = targets + row * steps;
    const float *wt = WEIGHTED ? weights + row * weights_row_stride : nullptr;
    uint32_t *back_row = back + row * steps * (int64_t)kVitThreads;
    float x = tg[0], c = WEIGHTED ? wt[0] : 1.f;
    for (int t = 0; t < steps; t++) {
        const int tn = t + 1 < steps ? t + 1 : t;
        const float nx = tg[tn], nc = WEIGHTED ? wt[tn] : 1.f;
        float *bw = best + (t & 1) * G;
        uint32_t bp = 0;
#pragma unroll
        for (int gi = 0; gi < NG; gi++) {
            float m = rho[4 * gi];
            uint32_t arg = 0;
#pragma unroll
            for (int d = 1; d < 4; d++) {
                const bool lt = rho[4 * gi + d] < m;       // the first minimum wins
                m = lt ? rho[4 * gi + d] : m;
                arg = lt ? (uint32_t)d : arg;
            }
            bw[NG * j + gi] = m;
            bp |= arg << (2 * gi);
        }
        back_row[(int64_t)t * kVitThreads + j] = bp;
        __syncthreads();       // one barrier a step: the halves of `best` take turns (see above)
        // state (d << (L-2)) | g comes from group (d << (L-4)) | (g >> 2); g >> 2 = (NG/4) * j + gi / 4
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const float *brun = bw + (d << (L - 4)) + (NG / 4) * j;
            float bq[NG / 4];
            if constexpr (NG / 4 == 4) {
                const float4 b = *reinterpret_cast<const float4 *>(brun);
                bq[0] = b.x, bq[1] = b.y, bq[2] = b.z, bq[3] = b.w;
            } else {
#pragma unroll
                for (int q = 0; q < NG / 4; q++) bq[q] = brun[q];
            }
#pragma unroll
            for (int gi = 0; gi < NG; gi++) {
                const int r = 4 * gi + d;
                const float dd = (r & 1) ? sub_half_hi(x, val[r >> 1]) : sub_half_lo(x, val[r >> 1]);
                float sq = dd * dd;
                if (WEIGHTED) sq = c * sq;                 // rptc.py:32: c * (x - a)**2
                rho[r] = bq[gi >> 2] + sq;
            }
        }
        x = nx, c = nc;
    }

    float mv = rho[0];
    int mi = NG * j;
#pragma unroll
    for (int d = 0; d < 4; d++) {
#pragma unroll
        for (int gi = 0; gi < NG; gi++) {
            const float v = rho[4 * gi + d];
            const int s = (d << (L - 2)) | (NG * j + gi);
            if (v < mv) {
                mv = v;
                mi = s;
            }
        }
    }
    red_v[j] = mv;
    red_i[j] = mi;
    __syncthreads();
    for (int width = kVitThreads / 2; width > 0; width >>= 1) {
        if (j < width) {
            const float ov = red_v[j + width];
            const int oi = red_i[j + width];
            if (ov < red_v[j] || (ov == red_v[j] && oi < red_i[j])) {
                red_v[j] = ov;
                red_i[j] = oi;
            }
        }
        __syncthreads();
    }
    if (j == 0) {
        end_state[row] = red_i[0];
        cost[row] = red_v[0];
    }
}

template <int L>
__global__ __launch_bounds__(64) void viterbi_scalar_trace_kernel(const uint32_t *__restrict__ back,
                                                                  const int32_t *__restrict__ end_state,
                                                                  uint8_t *__restrict__ symbols, int rows, int steps)
{
    constexpr int NG = (1 << L) / 4 / kVitThreads;
    const int row = blockIdx.x * 64 + threadIdx.x;
    if (row >= rows) return;
    const uint32_t *back_row = back + (int64_t)row * steps * kVitThreads;
    uint8_t *sym = symbols + (int64_t)row * steps;
    uint32_t state = (uint32_t)end_state[row];
    for (int t = steps - 1; t >= 0; t--) {
        sym[t] = (uint8_t)(state & 3u);
        const uint32_t low = state >> 2;                // the predecessor's low L-2 bits = the group
        const uint32_t bp = back_row[(int64_t)t * kVitThreads + low / NG];
        state = (((bp >> (2 * (low % NG))) & 3u) << (L - 2)) | low;
    }
}

// The search of rptc_lite.py:19-60 for any other (L, S, R, V) the reference's function takes, within L <= 20, R <= 8,
// V <= 4: one workgroup a row, the 2^L path costs and the 2^(L-R) group minima in the caller's scratch (global memory that
// stays in the L2: the costs of L = 16 alone are 256 KiB, more than the LDS), two barriers a step.  A step is the
// reference's: minimum and first arg-minimum over the 2^R predecessors (d << (L - R)) | p of each group p
// (rptc_lite.py:33-34, the back pointer; a byte here, R bits packed into int32 words there), then
// cost[s] = minimum[s >> R] + sum_v importance[t][v] * (samples[t][v] - alphabet[index_fn(s)][v])^2 (rptc_lite.py:39-40),
// every sum fp32 in that order.  Not tuned: the trellis the reference's driver uses has the kernel above.
struct LiteGeneralScratch {
    int64_t row_floats;      // floats a row: 2^L costs, then 2^(L-R) minima
    int64_t back_offset;     // byte offset of the back pointers ([row][step][2^(L-R)] bytes) in the scratch
};

__host__ __device__ inline LiteGeneralScratch lite_general_scratch(int L, int R, int64_t rows)
{
    LiteGeneralScratch g;
    g.row_floats = ((int64_t)1 << L) + ((int64_t)1 << (L - R));
    g.back_offset = (rows * g.row_floats * 4 + 255) / 256 * 256;
    return g;
}

template <bool WEIGHTED>
__global__ __launch_bounds__(kVitThreads) void viterbi_lite_general_kernel(
    const float *__restrict__ targets, const float *__restrict__ weights, int64_t weights_row_stride,
    const float *__restrict__ alphabet, int L, int S, int R, int V, float *work, uint8_t *back,
    int32_t *__restrict__ end_state, float *__restrict__ cost, int steps)
{
    __shared__ float red_v[kVitThreads];
    __shared__ int red_i[kVitThreads];
    const int j = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int states = 1 << L, groups = 1 << (L - R), fan = 1 << R;
    float *rho = work + row * ((int64_t)states + groups);
    float *best = rho + states;
    uint8_t *back_row = back + row * steps * (int64_t)groups;
    const float *tg = targets + row * steps * V;
    const float *wt = WEIGHTED ? weights + row * weights_row_stride : nullptr;

    for (int s = j; s < states; s += kVitThreads) rho[s] = s == 0 ? 0.f : INFINITY;      // rptc_lite.py:43-44
    __syncthreads();
    for (int t = 0; t < steps; t++) {
        for (int p = j; p < groups; p += kVitThreads) {
            float m = rho[p];
            int arg = 0;
            for (int d = 1; d < fan; d++) {
                const float v = rho[(d << (L - R)) | p];
                if (v < m) {                            // the first minimum wins (argmin)
                    m = v;
                    arg = d;
                }
            }
            best[p] = m;
            back_row[(int64_t)t * groups + p] = (uint8_t)arg;
        }
        __syncthreads();
        float x[4], c[4];
        for (int v = 0; v < 4; v++) {
            x[v] = v < V ? tg[(int64_t)t * V + v] : 0.f;
            c[v] = (WEIGHTED && v < V) ? wt[(int64_t)t * V + v] : 1.f;
        }
        for (int s = j; s < states; s += kVitThreads) {
            uint32_t h = (uint32_t)s * (2u * (uint32_t)s + 1u);        // index_fn, rptc_lite.py:12-16 (bits below L decide)
            h ^= h >> (L - S);
            const float *a = alphabet + (int64_t)(h & ((1u << S) - 1u)) * V;
            float loss = 0.f;
            for (int v = 0; v < V; v++) {
                const float d = x[v] - a[v];
                float sq = d * d;
                if (WEIGHTED) sq = c[v] * sq;
                loss = v == 0 ? sq : loss + sq;
            }
            rho[s] = best[s >> R] + loss;
        }
        __syncthreads();
    }

    // cheapest end state, the lowest index among equals (argmin, rptc_lite.py:52)
    float mv = INFINITY;
    int mi = 0x7FFFFFFF;
    for (int s = j; s < states; s += kVitThreads) {
        const float v = rho[s];
        if (v < mv || mi == 0x7FFFFFFF) {
            mv = v;
            mi = s;
        }
    }
    red_v[j] = mv;
    red_i[j] = mi;
    __syncthreads();
    for (int width = kVitThreads / 2; width > 0; width >>= 1) {
        if (j < width) {
            const float ov = red_v[j + width];
            const int oi = red_i[j + width];
            if (ov < red_v[j] || (ov == red_v[j] && oi < red_i[j])) {
                red_v[j] = ov;
                red_i[j] = oi;
            }
        }
        __syncthreads();
    }
    if (j == 0) {
        end_state[row] = red_i[0];
        cost[row] = red_v[0];
    }
}

// one thread a row walks the general search's back pointers from the end state (rptc_lite.py:47-55)
__global__ __launch_bounds__(64) void viterbi_lite_general_trace_kernel(const uint8_t *__restrict__ back,
                                                                        const int32_t *__restrict__ end_state,
                                                                        uint8_t *__restrict__ symbols, int L, int R, int rows, int steps)
{
    const int row = blockIdx.x * 64 + threadIdx.x;
    if (row >= rows) return;
    const int64_t groups = (int64_t)1 << (L - R);
    const uint8_t *back_row = back + (int64_t)row * steps * groups;
    uint8_t *sym = symbols + (int64_t)row * steps;
    uint32_t state = (uint32_t)end_state[row];
    for (int t = steps - 1; t >= 0; t--) {
        sym[t] = (uint8_t)(state & ((1u << R) - 1u));
        const uint32_t p = state >> R;
        state = ((uint32_t)back_row[(int64_t)t * groups + p] << (L - R)) | p;
    }
}

// one thread per row walks the back pointers from the end state (rptc.py:60-65)
template <int STEP>
__global__ __launch_bounds__(64) void viterbi_trace_kernel(const uint16_t *__restrict__ back,
                                                           const int32_t *__restrict__ end_state,
                                                           uint8_t *__restrict__ symbols, int rows, int steps)
{
    const int row = blockIdx.x * 64 + threadIdx.x;
    if (row >= rows) return;
    const uint16_t *back_row = back + (int64_t)row * steps * kVitThreads;
    uint8_t *sym = symbols + (int64_t)row * steps;
    uint32_t state = (uint32_t)end_state[row];
    for (int t = steps - 1; t >= 0; t--) {
        sym[t] = (uint8_t)(state & ((1u << STEP) - 1u));
        const uint32_t low = state >> STEP;             // the predecessor's low bits = the group
        uint32_t d;
        if (STEP == 4) d = (back_row[(int64_t)t * kVitThreads + (low >> 2)] >> (4 * (low & 3u))) & 15u;
        else if (STEP == 6) d = back_row[(int64_t)t * kVitThreads + low];
        else d = back_row[(int64_t)t * kVitThreads + 4 * low];
        state = (d << (16 - STEP)) | low;
    }
}

template <typename K>
static int vit_allow_lds(K kernel)
{
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    kVitLdsBytes);
}

template <typename K>
static int vit_allow_scalar_lds(K kernel, int bytes)
{
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

int prepare_viterbi()
{
    int rc;
    if ((rc = vit_allow_scalar_lds(viterbi_scalar_kernel<16, false>, scalar_lds_bytes(16)))) return rc;
    if ((rc = vit_allow_scalar_lds(viterbi_scalar_kernel<16, true>, scalar_lds_bytes(16)))) return rc;
    if ((rc = vit_allow_scalar_lds(viterbi_scalar_kernel<14, false>, scalar_lds_bytes(14)))) return rc;
    if ((rc = vit_allow_scalar_lds(viterbi_scalar_kernel<14, true>, scalar_lds_bytes(14)))) return rc;
#define RPTC_VIT_ALLOW(STEP)                                                       \
    if ((rc = vit_allow_lds(viterbi_pairs_kernel<6, STEP, false>))) return rc;     \
    if ((rc = vit_allow_lds(viterbi_pairs_kernel<6, STEP, true>))) return rc;      \
    if ((rc = vit_allow_lds(viterbi_pairs_kernel<8, STEP, false>))) return rc;     \
    if ((rc = vit_allow_lds(viterbi_pairs_kernel<8, STEP, true>))) return rc;
    RPTC_VIT_ALLOW(4)
    RPTC_VIT_ALLOW(6)
    RPTC_VIT_ALLOW(8)
#undef RPTC_VIT_ALLOW
    if ((rc = vit_allow_lds(viterbi_lite_kernel<false>))) return rc;
    if ((rc = vit_allow_lds(viterbi_lite_kernel<true>))) return rc;
    return 0;
}

template <int S, int STEP>
static void launch_viterbi(const float *targets, const float *weights, int64_t weights_row_stride, const uint16_t *codebook,
                           uint16_t *back, uint8_t *symbols, int32_t *end_state, float *cost, int64_t rows, int64_t steps,
                           hipStream_t s)
{
    if (weights)
        hipLaunchKernelGGL((viterbi_pairs_kernel<S, STEP, true>), dim3((unsigned)rows), dim3(kVitThreads), kVitLdsBytes, s,
                           targets, weights, weights_row_stride, codebook, back, end_state, cost, (int)steps);
    else
        hipLaunchKernelGGL((viterbi_pairs_kernel<S, STEP, false>), dim3((unsigned)rows), dim3(kVitThreads), kVitLdsBytes, s,
                           targets, weights, weights_row_stride, codebook, back, end_state, cost, (int)steps);
    hipLaunchKernelGGL(viterbi_trace_kernel<STEP>, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, back, end_state, symbols,
                       (int)rows, (int)steps);
}

template <int L, bool WEIGHTED>
static void launch_viterbi_scalar(const float *targets, const float *weights, int64_t weights_row_stride,
                                  const uint16_t *alphabet, uint32_t *back, uint8_t *symbols, int32_t *end_state,
                                  float *cost, int64_t rows, int64_t steps, hipStream_t s)
{
    hipLaunchKernelGGL((viterbi_scalar_kernel<L, WEIGHTED>), dim3((unsigned)rows), dim3(kVitThreads), scalar_lds_bytes(L), s,
                       targets, weights, weights_row_stride, alphabet, back, end_state, cost, (int)steps);
    hipLaunchKernelGGL(viterbi_scalar_trace_kernel<L>, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, back, end_state,
                       symbols, (int)rows, (int)steps);
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_viterbi_scalar(const float *targets, const float *weights, int64_t weights_row_stride,
                                   const uint16_t *alphabet, int L, void *scratch, uint8_t *symbols, int32_t *end_state,
                                   float *cost, int64_t rows, int64_t steps, void *stream, float *ms)
{
    if (!targets || !alphabet || !scratch || !symbols || !end_state || !cost) return RPTC_ENULL;
    if (L != 16 && L != 14) return RPTC_ESHAPE;
    if (rows < 1 || steps < 1 || weights_row_stride < 0) return RPTC_ESHAPE;
    if (weights && weights_row_stride != 0 && weights_row_stride < steps) return RPTC_ESHAPE;
    if (rows >= ((int64_t)1 << 24) || steps >= ((int64_t)1 << 24)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    uint32_t *back = static_cast<uint32_t *>(scratch);
    if (L == 16) {
        if (weights) launch_viterbi_scalar<16, true>(targets, weights, weights_row_stride, alphabet, back, symbols, end_state, cost, rows, steps, s);
        else launch_viterbi_scalar<16, false>(targets, weights, weights_row_stride, alphabet, back, symbols, end_state, cost, rows, steps, s);
    } else {
        if (weights) launch_viterbi_scalar<14, true>(targets, weights, weights_row_stride, alphabet, back, symbols, end_state, cost, rows, steps, s);
        else launch_viterbi_scalar<14, false>(targets, weights, weights_row_stride, alphabet, back, symbols, end_state, cost, rows, steps, s);
    }
    return t.end();
}

extern "C" int64_t rptc_viterbi_scratch_bytes(int64_t rows, int64_t steps)
{
    if (rows < 1 || steps < 1) return 0;
    return rows * steps * (int64_t)kVitThreads * 2;
}

extern "C" int64_t rptc_viterbi_scalar_scratch_bytes(int64_t rows, int64_t steps)
{
    if (rows < 1 || steps < 1) return 0;
    return rows * steps * (int64_t)kVitThreads * 4;
}

extern "C" int rptc_viterbi_pairs_bits(const float *targets, const float *weights, int64_t weights_row_stride,
                                       const uint16_t *codebook, void *scratch, uint8_t *symbols, int32_t *end_state,
                                       float *cost, int64_t rows, int64_t steps, int S, int bits, void *stream, float *ms)
{
    if (!targets || !codebook || !scratch || !symbols || !end_state || !cost) return RPTC_ENULL;
    if ((S != 6 && S != 8) || bits < 2 || bits > 4) return RPTC_ESHAPE;
    if (rows < 1 || steps < 1 || weights_row_stride < 0) return RPTC_ESHAPE;
    if (weights && weights_row_stride != 0 && weights_row_stride < 2 * steps) return RPTC_ESHAPE;
    if (rows >= ((int64_t)1 << 24) || steps >= ((int64_t)1 << 24)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    uint16_t *back = static_cast<uint16_t *>(scratch);
#define RPTC_VIT_GO(SS, BB)                                                                                        \
    if (S == SS && bits == BB)                                                                                      \
        launch_viterbi<SS, 2 * BB>(targets, weights, weights_row_stride, codebook, back, symbols, end_state, cost, rows, steps, s);
    RPTC_VIT_GO(6, 2) RPTC_VIT_GO(6, 3) RPTC_VIT_GO(6, 4) RPTC_VIT_GO(8, 2) RPTC_VIT_GO(8, 3) RPTC_VIT_GO(8, 4)
#undef RPTC_VIT_GO
    return t.end();
}

extern "C" int rptc_viterbi_pairs(const float *targets, const float *weights, int64_t weights_row_stride,
                                  const uint16_t *codebook, void *scratch, uint8_t *symbols, int32_t *end_state,
                                  float *cost, int64_t rows, int64_t steps, int S, void *stream, float *ms)
{
    return rptc_viterbi_pairs_bits(targets, weights, weights_row_stride, codebook, scratch, symbols, end_state, cost, rows,
                                   steps, S, 2, stream, ms);
}


extern "C" int64_t rptc_lite_viterbi_scratch_bytes(int L, int R, int64_t rows, int64_t steps)
{
    if (L < 1 || L > 20 || R < 1 || R > L || R > 8 || rows < 1 || steps < 1) return 0;
    if (L == 16 && R == 4) return rptc_viterbi_scratch_bytes(rows, steps);
    return lite_general_scratch(L, R, rows).back_offset + rows * steps * ((int64_t)1 << (L - R));
}

extern "C" int rptc_lite_viterbi(const float *samples, const float *importance, int64_t importance_row_stride,
                                 const float *alphabet, int L, int S, int R, int V, void *scratch, uint8_t *symbols,
                                 int32_t *end_state, float *cost, int64_t rows, int64_t steps, void *stream, float *ms)
{
    if (!samples || !alphabet || !scratch || !symbols || !end_state || !cost) return RPTC_ENULL;
    if (L < 1 || S < 1 || S > L || R < 1 || R > L || V < 1) return RPTC_ESHAPE;
    if (L > 20 || R > 8 || V > 4) return RPTC_ELIMIT;
    if (rows < 1 || steps < 1 || importance_row_stride < 0) return RPTC_ESHAPE;
    if (importance && importance_row_stride != 0 && importance_row_stride < V * steps) return RPTC_ESHAPE;
    if (rows >= ((int64_t)1 << 24) || steps >= ((int64_t)1 << 24)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    if (L == 16 && R == 4 && V == 2 && S <= 9) {        // the trellis of the reference's driver: the register-resident kernel
        uint16_t *back = static_cast<uint16_t *>(scratch);
        if (importance)
            hipLaunchKernelGGL(viterbi_lite_kernel<true>, dim3((unsigned)rows), dim3(kVitThreads), kVitLdsBytes, s, samples, importance,
                               importance_row_stride, alphabet, S, back, end_state, cost, (int)steps);
        else
            hipLaunchKernelGGL(viterbi_lite_kernel<false>, dim3((unsigned)rows), dim3(kVitThreads), kVitLdsBytes, s, samples, importance,
                               importance_row_stride, alphabet, S, back, end_state, cost, (int)steps);
        hipLaunchKernelGGL(viterbi_trace_kernel<4>, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, back, end_state, symbols, (int)rows,
                           (int)steps);
        return t.end();
    }
    float *work = static_cast<float *>(scratch);
    uint8_t *back = static_cast<uint8_t *>(scratch) + lite_general_scratch(L, R, rows).back_offset;
    if (importance)
        hipLaunchKernelGGL(viterbi_lite_general_kernel<true>, dim3((unsigned)rows), dim3(kVitThreads), 0, s, samples, importance,
                           importance_row_stride, alphabet, L, S, R, V, work, back, end_state, cost, (int)steps);
    else
        hipLaunchKernelGGL(viterbi_lite_general_kernel<false>, dim3((unsigned)rows), dim3(kVitThreads), 0, s, samples, importance,
                           importance_row_stride, alphabet, L, S, R, V, work, back, end_state, cost, (int)steps);
    hipLaunchKernelGGL(viterbi_lite_general_trace_kernel, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, back, end_state, symbols, L, R,
                       (int)rows, (int)steps);
    return t.end();
}
