// Decode-only kernel for the row-major stream with the scalar 2^16 codebook.
//
// Semantics: rptc_kernels/csrc/rptc_kernels/inference.cu:42-96 (kernel) and :99-160 (launcher)
// of the reference.  Output t of a row is codebook[the 16 stream bits ending at bit 2t+2], so
// nothing is sequential: a thread can produce any eight consecutive outputs from the 16 bits
// they add plus 14 bits of history.  The design follows from that:
//   * the whole 128 KiB codebook lives in LDS (gfx950 has 160 KiB per workgroup), so the 64
//     gathers per stream element never leave the CU;
//   * a thread owns 8 consecutive outputs = one 16-byte store, a wave writes 1 KiB contiguous;
//   * the stream is read with dword loads that hit the same cache lines the neighbours use
//     (the stream is 1/8 of the traffic, the fp16 output 8/8).
#include "rptc_common.hpp"

namespace rptc {

constexpr int kDecompressThreads = 1024;
constexpr int kLutBytes = 65536 * 2;

template <int MODE>
__global__ __launch_bounds__(kDecompressThreads) void decompress_kernel(
    const uint32_t *__restrict__ comp, const uint4 *__restrict__ codebook, uint4 *__restrict__ out,
    uint32_t words_per_row, uint32_t total_groups)
{
    extern __shared__ uint4 lds_u4[];
    const int tid = threadIdx.x;
    {
        // all of a thread's share of the table is requested before any of it is stored: one memory
        // round trip instead of eight
        constexpr int kPerThread = kLutBytes / 16 / kDecompressThreads;
        uint4 t[kPerThread];
#pragma unroll
        for (int i = 0; i < kPerThread; i++) t[i] = codebook[i * kDecompressThreads + tid];
#pragma unroll
        for (int i = 0; i < kPerThread; i++) lds_u4[i * kDecompressThreads + tid] = t[i];
    }
    __syncthreads();
    const uint16_t *lut = reinterpret_cast<const uint16_t *>(lds_u4);

    const uint32_t groups_per_row = words_per_row * 2;   // a word holds 16 outputs = two groups of 8
    const uint32_t stride = gridDim.x * kDecompressThreads;
    constexpr int kInFlight = 4;   // groups whose stream words are requested before any is decoded
    for (uint32_t g0 = blockIdx.x * kDecompressThreads + tid; g0 < total_groups; g0 += stride * kInFlight) {
        uint32_t cur[kInFlight], prev[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const uint32_t g = g0 + u * stride;
            cur[u] = prev[u] = 0;
            if (g < total_groups) {
                const uint32_t row = g / groups_per_row;
                const uint32_t w = (g - row * groups_per_row) >> 1;
                const uint32_t *rowp = comp + (size_t)row * words_per_row;
                cur[u] = rowp[w];
                if (w && !(g & 1)) prev[u] = rowp[w - 1];
            }
        }
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const uint32_t g = g0 + u * stride;
            if (g >= total_groups) break;
            const uint32_t w = (g % groups_per_row) >> 1;
            uint32_t v;   // 16 bits of history above the 16 new bits
            if (g & 1) {  // groups_per_row is even, so the parity of g is the parity within the row
                v = cur[u];
            } else {
                // inference.cu:56-62: lane 0 of a warp reads the uint16 just below its element,
                // the high half of the previous word; every other lane gets the low half.
                const uint32_t hist = (MODE == RPTC_AS_WRITTEN && (w & 127u) == 0) ? (prev[u] >> 16)
                                                                                   : (prev[u] & 0xFFFFu);
                v = (hist << 16) | (cur[u] >> 16);
            }
            uint32_t o[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t s0 = (v >> (14 - 4 * i)) & 0xFFFFu;
                const uint32_t s1 = (v >> (12 - 4 * i)) & 0xFFFFu;
                o[i] = (uint32_t)lut[s0] | ((uint32_t)lut[s1] << 16);
            }
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            u32x4 ov = {o[0], o[1], o[2], o[3]};
            __builtin_nontemporal_store(ov, reinterpret_cast<u32x4 *>(out) + g);
        }
    }
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_decompress(const int32_t *compressed, const uint16_t *codebook, uint16_t *out,
                               int64_t m, int64_t words_per_row, int carry_mode, void *stream,
                               float *ms)
{
    if (!compressed || !codebook || !out) return RPTC_ENULL;
    if (m < 1 || words_per_row < 128 || words_per_row % 128 != 0) return RPTC_ESHAPE;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(out)) return RPTC_EALIGN;
    const int64_t groups = m * words_per_row * 2;
    if (groups >= (int64_t)1 << 31 || words_per_row >= (int64_t)1 << 30) return RPTC_ELIMIT;

    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;

    const int64_t blocks_needed = (groups + kDecompressThreads - 1) / kDecompressThreads;
    const int grid = (int)(blocks_needed < dev->cus ? blocks_needed : dev->cus);
    auto args_comp = reinterpret_cast<const uint32_t *>(compressed);
    auto args_cb = reinterpret_cast<const uint4 *>(codebook);
    auto args_out = reinterpret_cast<uint4 *>(out);
    if (carry_mode == RPTC_AS_WRITTEN)
        hipLaunchKernelGGL(decompress_kernel<RPTC_AS_WRITTEN>, dim3(grid), dim3(kDecompressThreads),
                           kLutBytes, s, args_comp, args_cb, args_out, (uint32_t)words_per_row,
                           (uint32_t)groups);
    else
        hipLaunchKernelGGL(decompress_kernel<RPTC_CONTINUOUS>, dim3(grid), dim3(kDecompressThreads),
                           kLutBytes, s, args_comp, args_cb, args_out, (uint32_t)words_per_row,
                           (uint32_t)groups);
    return t.end();
}

namespace rptc {
int prepare_decompress()
{
    int rc = (int)hipFuncSetAttribute(reinterpret_cast<const void *>(decompress_kernel<RPTC_AS_WRITTEN>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, kLutBytes);
    if (rc) return rc;
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(decompress_kernel<RPTC_CONTINUOUS>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kLutBytes);
}
}  // namespace rptc
