// The butterfly passes of the sign-Hadamard transform, shared by the stand-alone kernel and by the
// mat-vec that transforms its activations in its prologue.
#pragma once

#include "rptc_common.hpp"

namespace rptc {

// Element i of the vector lives at buf[had_pad(i)]: one unused float after every 32 keeps the
// 16-point gathers (lane stride 16 floats in the first pass) off the same LDS bank.
__device__ __forceinline__ int had_pad(int i) { return i + (i >> 5); }

// Stages s .. s+R_LOG-1 of the Walsh-Hadamard butterflies on the `count` floats in buf, done by
// THREADS threads: a thread gathers 2^R_LOG elements that are 2^s apart, transforms them in
// registers and scatters them back.  With blocks of P = 2^log_p elements and s + R_LOG <= log_p a
// gather never leaves its block, so the same pass serves one block or a whole vector of blocks.
template <int R_LOG, int THREADS>
__device__ __forceinline__ void hadamard_pass(float *buf, int count, int s, int tid)
{
    constexpr int R = 1 << R_LOG;
    const int low_mask = (1 << s) - 1;
    for (int grp = tid; grp < (count >> R_LOG); grp += THREADS) {
        const int base = ((grp >> s) << (s + R_LOG)) | (grp & low_mask);
        float v[R];
#pragma unroll
        for (int k = 0; k < R; k++) v[k] = buf[had_pad(base + (k << s))];
#pragma unroll
        for (int h = 1; h < R; h <<= 1) {
#pragma unroll
            for (int k = 0; k < R; k++) {
                if ((k & h) == 0) {
                    const float a = v[k], b = v[k | h];
                    v[k] = a + b;
                    v[k | h] = a - b;
                }
            }
        }
#pragma unroll
        for (int k = 0; k < R; k++) buf[had_pad(base + (k << s))] = v[k];
    }
}

// All log_p stages, four at a time, with a barrier after every pass.
template <int THREADS>
__device__ __forceinline__ void hadamard_stages(float *buf, int count, int log_p, int tid)
{
    int stage = 0;
    for (; stage + 4 <= log_p; stage += 4) {
        hadamard_pass<4, THREADS>(buf, count, stage, tid);
        __syncthreads();
    }
    const int rest = log_p - stage;
    if (rest == 3) hadamard_pass<3, THREADS>(buf, count, stage, tid);
    else if (rest == 2) hadamard_pass<2, THREADS>(buf, count, stage, tid);
    else if (rest == 1) hadamard_pass<1, THREADS>(buf, count, stage, tid);
    if (rest) __syncthreads();
}

}  // namespace rptc
