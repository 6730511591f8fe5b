// Random-sign Hadamard (incoherence) transform on activations.
//
// No counterpart in the reference (it conditions weights with a row/column scale-and-bias
// factorisation instead, quantize_hf.py:77-117); this is the transform the north star asks for.
// Definition: the vector of length n is cut into blocks of P elements, P a power of two dividing
// n (by default the largest one: 4096 for n = 4096, 256 for n = 11008 = 43 * 256, 4096 for
// n = 28672 = 7 * 4096), and each block is mapped by
//     forward   y = H_P (s .* x) / sqrt(P)        inverse   y = s .* (H_P x) / sqrt(P)
// with H_P the Sylvester Hadamard matrix (natural order) and s a vector of +-1.  H_P is symmetric
// and H_P H_P = P I, so the two are inverses and both are orthogonal.
//
// Kernel: one workgroup per (batch row, block); the block lives in LDS as fp32.  The log2(P)
// butterfly stages are done four at a time: a thread gathers 16 elements that are 2^s apart, runs
// a 16-point transform in registers and scatters them back, so a 4096-point block needs three
// passes and two barriers instead of twelve.  The op moves 4 bytes per element (fp16 in, fp16
// out): HBM-bound, LDS traffic is local.
#include "hadamard_pass.hpp"

namespace rptc {

constexpr int kHadThreads = 256;
constexpr int kHadMaxBlock = 32768;       // 132 KiB of fp32 in LDS (with padding)

__device__ __forceinline__ int pad(int i) { return had_pad(i); }

__global__ __launch_bounds__(kHadThreads) void sign_hadamard_kernel(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ signs, uint16_t *__restrict__ out,
    int n, int P, int log_p, int blocks_per_row, int signs_after, int wide)
{
    extern __shared__ float buf[];
    const int tid = threadIdx.x;
    const int row = blockIdx.x / blocks_per_row, blk = blockIdx.x - row * blocks_per_row;
    const size_t base = (size_t)row * n + (size_t)blk * P;
    const uint16_t *s = signs + (size_t)blk * P;
    // wide != 0: P % 8 == 0 and 16-byte aligned pointers: 8 halves per load, up to four loads of a
    // thread requested before the first is used (one at a time they would be a round trip each)
    constexpr int kInFlight = 4;
    if (wide) {
        const uint4 *x4 = reinterpret_cast<const uint4 *>(x + base), *s4 = reinterpret_cast<const uint4 *>(s);
        for (int c0 = tid; c0 < (P >> 3); c0 += kHadThreads * kInFlight) {
            uint4 xv[kInFlight], sv[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; u++) {
                const int c = c0 + u * kHadThreads;
                xv[u] = sv[u] = make_uint4(0, 0, 0, 0);
                if (c < (P >> 3)) {
                    xv[u] = x4[c];
                    if (!signs_after) sv[u] = s4[c];
                }
            }
#pragma unroll
            for (int u = 0; u < kInFlight; u++) {
                const int c = c0 + u * kHadThreads;
                if (c >= (P >> 3)) break;
                const uint32_t xw[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w}, sw[4] = {sv[u].x, sv[u].y, sv[u].z, sv[u].w};
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    float v = half_bits_to_float((uint16_t)(xw[k >> 1] >> (16 * (k & 1))));
                    if (!signs_after) v *= half_bits_to_float((uint16_t)(sw[k >> 1] >> (16 * (k & 1))));
                    buf[pad(8 * c + k)] = v;
                }
            }
        }
    } else {
        for (int i = tid; i < P; i += kHadThreads) {
            float v = half_bits_to_float(x[base + i]);
            if (!signs_after) v *= half_bits_to_float(s[i]);
            buf[pad(i)] = v;
        }
    }
    __syncthreads();
    hadamard_stages<kHadThreads>(buf, P, log_p, tid);
    const float scale = rsqrtf((float)P);
    if (wide) {
        const uint4 *s4 = reinterpret_cast<const uint4 *>(s);
        uint4 *o4 = reinterpret_cast<uint4 *>(out + base);
        for (int c0 = tid; c0 < (P >> 3); c0 += kHadThreads * kInFlight) {
            uint4 sv[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; u++) {
                const int c = c0 + u * kHadThreads;
                sv[u] = make_uint4(0, 0, 0, 0);
                if (signs_after && c < (P >> 3)) sv[u] = s4[c];
            }
#pragma unroll
            for (int u = 0; u < kInFlight; u++) {
                const int c = c0 + u * kHadThreads;
                if (c >= (P >> 3)) break;
                const uint32_t sw[4] = {sv[u].x, sv[u].y, sv[u].z, sv[u].w};
                uint32_t ow[4] = {0, 0, 0, 0};
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    float v = buf[pad(8 * c + k)] * scale;
                    if (signs_after) v *= half_bits_to_float((uint16_t)(sw[k >> 1] >> (16 * (k & 1))));
                    ow[k >> 1] |= (uint32_t)float_to_half_bits(v) << (16 * (k & 1));
                }
                o4[c] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
            }
        }
    } else {
        for (int i = tid; i < P; i += kHadThreads) {
            float v = buf[pad(i)] * scale;
            if (signs_after) v *= half_bits_to_float(s[i]);
            out[base + i] = float_to_half_bits(v);
        }
    }
}

int prepare_hadamard()
{
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(sign_hadamard_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (kHadMaxBlock + kHadMaxBlock / 32) * 4);
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_sign_hadamard(const uint16_t *x, const uint16_t *signs, uint16_t *out, int64_t batch,
                                  int64_t n, int64_t block, int inverse, void *stream, float *ms)
{
    if (!x || !signs || !out) return RPTC_ENULL;
    if (batch < 1 || n < 2) return RPTC_ESHAPE;
    int64_t P = block;
    if (P == 0) {
        P = 1;
        while (n % (2 * P) == 0 && 2 * P <= kHadMaxBlock) P *= 2;
    }
    if (P < 2 || (P & (P - 1)) != 0 || n % P != 0) return RPTC_ESHAPE;
    if (P > kHadMaxBlock || n >= ((int64_t)1 << 30) || batch * (n / P) >= ((int64_t)1 << 31)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    const int blocks_per_row = (int)(n / P);
    int log_p = 0;
    while (((int64_t)1 << log_p) < P) log_p++;
    hipLaunchKernelGGL(sign_hadamard_kernel, dim3((unsigned)(batch * blocks_per_row)), dim3(kHadThreads),
                       (size_t)(P + P / 32) * 4, s, x, signs, out, (int)n, (int)P, log_p, blocks_per_row, inverse ? 1 : 0,
                       (P % 8 == 0 && aligned16(x) && aligned16(signs) && aligned16(out)) ? 1 : 0);
    return t.end();
}
