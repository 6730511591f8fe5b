// Fused decode + mat-vec on the column-interleaved stream with a scalar 2^L codebook.
//
// Semantics: rptc_kernels/csrc/rptc_kernels/inference_t.cu:68-175 (kernel) and :178-256
// (launcher) of the reference.  The stream is uint4 c[col * m + row]: consecutive rows are
// consecutive in memory, so a lane is a row (coalesced 16-byte loads), the activations are the
// same for the whole wave and come through the scalar cache, and nothing crosses lanes.
//
// gfx950 design: the whole codebook (128 KiB at L = 16) sits in LDS; the reference's
// one-thread-per-row loop is split along the columns, over the 8 waves of a workgroup and, when
// there are fewer 64-row blocks than CUs, over several workgroups per row block.  The stream
// allows it because the decoder state after an element depends only on that element (as written:
// the top nibbles of its four words, inference_t.cu:131-142; continuous: its last L bits), so a
// wave warms its state up from the element before its range.  Waves are added in LDS in wave
// order; workgroups of a row block publish fp32 partial sums in a static scratch buffer with
// device-scope stores, and the one that arrives last at the row block's counter adds them in
// workgroup order and accumulates into `out`: every sum has a fixed order.
#include "rptc_common.hpp"

namespace rptc {

constexpr int kTThreads = 512;
constexpr int kTWaves = kTThreads / kWave;
constexpr int kTMaxParts = 4096;        // workgroups of a launch that splits the columns
constexpr int kTMaxSplit = 16;
constexpr int kTRing = 8;               // stream elements a wave has requested ahead of the decode

static __device__ __align__(256) float g_t_part[kTMaxParts * kWave];
static __device__ __align__(256) uint32_t g_t_arrived[kTMaxParts];

template <int L>
__device__ __forceinline__ uint32_t warm_state(const uint4 e, int mode)
{
    constexpr uint32_t mask = (1u << L) - 1u;
    if (mode == RPTC_CONTINUOUS) return e.w & mask;
    uint32_t c = 0;
    c = mask & ((c << 4) | (e.x >> 28));
    c = mask & ((c << 4) | (e.y >> 28));
    c = mask & ((c << 4) | (e.z >> 28));
    c = mask & ((c << 4) | (e.w >> 28));
    return c;
}

// Arguments in the order of their first use: the first 14 dwords arrive preloaded in SGPRs.
template <int L, int MODE>
__global__ __launch_bounds__(kTThreads) void matvec_t_kernel(
    const uint4 *__restrict__ comp, const uint4 *__restrict__ codebook, const uint32_t *__restrict__ x,
    int m, int cols, int ksplit, uint16_t *__restrict__ out, float *__restrict__ parts, uint32_t *__restrict__ arrived)
{
    extern __shared__ uint4 lds_u4[];
    constexpr int lut_u4 = (2 << L) / 16;
    constexpr uint32_t mask = (1u << L) - 1u;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rb = blockIdx.x / ksplit, sp = blockIdx.x - rb * ksplit;
    const int row = rb * kWave + lane;
    const bool valid = row < m;
    // this workgroup's columns, then this wave's share of them
    const int per_group = (cols + ksplit - 1) / ksplit;
    const int g0 = min(cols, sp * per_group), g1 = min(cols, g0 + per_group);
    const int per = (g1 - g0 + kTWaves - 1) / kTWaves;
    const int c0 = min(g1, g0 + wave * per), c1 = min(g1, c0 + per);

    // Requests in the order their data is needed: the thread's share of the table, then the element in
    // front of the wave's range (its state warms up the decoder) and the first kTRing elements of the range.
    // A wave's elements come from memory with a latency of a few thousand clocks and are decoded in a few
    // hundred each, so the time of the loop is the latency times the elements divided by the requests in
    // flight: the ring holds eight (all of a wave's elements when the columns are split eight ways or more).
    // The stream requests are unconditional (clamped to an element that exists) so that the table can be
    // stored while they are still on their way; what a clamped request returns is never used.
    constexpr int kPerThread = lut_u4 / kTThreads;
    uint4 xa = make_uint4(0u, 0u, 0u, 0u), xb = xa;
    if (MODE == RPTC_AS_WRITTEN && tid < 4 * (g1 - g0)) {
        const uint4 *xv = reinterpret_cast<const uint4 *>(x + 32 * g0 + 8 * tid);
        xa = xv[0];
        xb = xv[1];
    }
    uint4 t[kPerThread];
#pragma unroll
    for (int i = 0; i < kPerThread; i++) t[i] = codebook[i * kTThreads + tid];
    const int row_c = min(row, m - 1), last_col = cols - 1;
    const uint4 before = comp[(size_t)min(max(c0 - 1, 0), last_col) * m + row_c];
    uint4 ring[kTRing];
#pragma unroll
    for (int i = 0; i < kTRing; i++) ring[i] = comp[(size_t)min(c0 + i, last_col) * m + row_c];
    // As written, the eight steps of a stream word multiply the same two table values (inference_t.cu:125-134), so
    // what a word needs of its sixteen activations is the sum of the even and the sum of the odd ones: two fp32
    // values per word, added up here once per workgroup and kept in LDS (every lane of a wave reads the same ones:
    // a broadcast).  Their loads were the first requests of the kernel, so they are here before the table is.
    // (Reading the sixteen through the scalar cache in the loop, one wait per word for data requested a few
    // instructions earlier, made an element cost a thousand clocks.  The continuous mode, where every step has
    // table values of its own, still does that.)
    float *part = reinterpret_cast<float *>(lds_u4 + lut_u4);      // [wave][lane]
    uint32_t *xs = reinterpret_cast<uint32_t *>(part + kTThreads);
    if (MODE == RPTC_AS_WRITTEN) {
        for (int wd = tid; wd < 4 * (g1 - g0); wd += kTThreads) {
            const uint32_t d[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
            float lo = 0.f, hi = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                lo += half_bits_to_float((uint16_t)(d[j] & 0xFFFFu));
                hi += half_bits_to_float((uint16_t)(d[j] >> 16));
            }
            reinterpret_cast<float2 *>(xs)[wd] = make_float2(lo, hi);
            if (wd + kTThreads < 4 * (g1 - g0)) {
                const uint4 *xv = reinterpret_cast<const uint4 *>(x + 32 * g0 + 8 * (wd + kTThreads));
                xa = xv[0];
                xb = xv[1];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kPerThread; i++) lds_u4[i * kTThreads + tid] = t[i];
    __syncthreads();
    const uint16_t *lut = reinterpret_cast<const uint16_t *>(lds_u4);

    uint32_t carry = 0;
    if (c0 > 0 && c0 < c1 && valid) carry = warm_state<L>(before, MODE);
    float acc = 0.f;
    for (int col0 = c0; col0 < c1; col0 += kTRing) {
#pragma unroll
        for (int i = 0; i < kTRing; i++) {
            const int col = col0 + i;
            if (col >= c1) break;                                   // (wave-uniform)
            const uint4 e = ring[i];
            if (col + kTRing < c1) ring[i] = comp[(size_t)(col + kTRing) * m + row_c];
            const uint32_t words[4] = {e.x, e.y, e.z, e.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t word = words[k];
                if (MODE == RPTC_AS_WRITTEN) {
                    // all eight steps of a word see the carry the word started with
                    // (inference_t.cu:125-134), and the carry becomes the 4-bit-advanced state
                    const uint32_t s2 = mask & ((carry << 2) | (word >> 30));
                    const uint32_t s4 = mask & ((carry << 4) | (word >> 28));
                    carry = s4;
                    const float2 xw = reinterpret_cast<const float2 *>(xs)[4 * (col - g0) + k];     // wave-uniform
                    acc = fmaf(half_bits_to_float(lut[s2]), xw.x, acc);
                    acc = fmaf(half_bits_to_float(lut[s4]), xw.y, acc);
                } else {
                    const uint32_t *xp = x + 32 * col + 8 * k;                                         // wave-uniform, scalar loads
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const uint32_t s2 = mask & alignbit(carry, word, 30 - 4 * j);
                        const uint32_t s4 = mask & alignbit(carry, word, 28 - 4 * j);
                        const uint32_t w = (uint32_t)lut[s2] | ((uint32_t)lut[s4] << 16);
                        acc = dot2(w, xp[j], acc);
                    }
                    carry = word & mask;
                }
            }
        }
    }
    part[wave * kWave + lane] = acc;
    __syncthreads();
    float y = 0.f;
    if (tid < kWave) {
#pragma unroll
        for (int w = 0; w < kTWaves; w++) y += part[w * kWave + tid];
    }
    if (ksplit == 1) {
        // the product is added to what out holds (inference_t.cu:170-171)
        if (tid < kWave && valid) out[row] = float_to_half_bits(half_bits_to_float(out[row]) + y);
        return;
    }
    // (the hand-off between workgroups: see published() / arrive() in rptc_common.hpp)
    publishing();
    if (tid < kWave) __hip_atomic_store(&parts[(size_t)blockIdx.x * kWave + tid], y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    published();
    __syncthreads();
    uint32_t *flag = reinterpret_cast<uint32_t *>(part);
    if (tid == 0) {
        const uint32_t prev = arrive(&arrived[rb]);
        const bool last = prev == (uint32_t)(ksplit - 1);
        if (last) __hip_atomic_store(&arrived[rb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        *flag = last;
    }
    __syncthreads();
    if (!*flag || tid >= kWave || !valid) return;
    float p[kTMaxSplit];
    merging();
#pragma unroll
    for (int i = 0; i < kTMaxSplit; i++)
        p[i] = i < ksplit ? __hip_atomic_load(&parts[((size_t)rb * ksplit + i) * kWave + tid], __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT)
                          : 0.f;
    merged();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < kTMaxSplit; i++) total += p[i];
    out[row] = float_to_half_bits(half_bits_to_float(out[row]) + total);
}

// Dense export: one thread per stream element.
template <int L, int MODE>
__global__ __launch_bounds__(256) void matvec_t_dense_kernel(
    const uint4 *__restrict__ comp, const uint16_t *__restrict__ codebook, uint32_t *__restrict__ W,
    int m, int cols)
{
    constexpr uint32_t mask = (1u << L) - 1u;
    const int row = blockIdx.x * 256 + threadIdx.x;
    const int col = blockIdx.y;
    if (row >= m) return;
    uint32_t carry = col > 0 ? warm_state<L>(comp[(size_t)(col - 1) * m + row], MODE) : 0u;
    const uint4 e = comp[(size_t)col * m + row];
    const uint32_t words[4] = {e.x, e.y, e.z, e.w};
    uint32_t *wrow = W + (size_t)row * (cols * 32) + col * 32;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint32_t word = words[k];
        if (MODE == RPTC_AS_WRITTEN) {
            const uint32_t s2 = mask & ((carry << 2) | (word >> 30));
            const uint32_t s4 = mask & ((carry << 4) | (word >> 28));
            carry = s4;
            const uint32_t w = (uint32_t)codebook[s2] | ((uint32_t)codebook[s4] << 16);
#pragma unroll
            for (int j = 0; j < 8; j++) wrow[8 * k + j] = w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t s2 = mask & alignbit(carry, word, 30 - 4 * j);
                const uint32_t s4 = mask & alignbit(carry, word, 28 - 4 * j);
                wrow[8 * k + j] = (uint32_t)codebook[s2] | ((uint32_t)codebook[s4] << 16);
            }
            carry = word & mask;
        }
    }
}

// LDS: the table, one partial sum per thread and, as written, two fp32 sums of activations per stream word of the
// workgroup's columns (32 bytes a column)
template <int L>
static int lds_bytes_t(int cols_per_group, int mode)
{
    return (2 << L) + kTThreads * 4 + (mode == RPTC_AS_WRITTEN ? cols_per_group * 32 : 0);
}

struct TScratch {
    float *parts;
    uint32_t *arrived;
};
static TScratch g_t[64];   // per device: addresses of the static scratch arrays

template <int L>
static int launch_matvec_t(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                           uint16_t *out, int64_t m, int64_t n, int carry_mode, void *stream, float *ms)
{
    if (!compressed || !codebook || !x || !out) return RPTC_ENULL;
    if (m < 1 || n < 64 || n % 64 != 0) return RPTC_ESHAPE;
    if (n > 32768) return RPTC_ELIMIT;      // the reference's 64 KiB of constant memory (inference_t.cu:49)
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(x)) return RPTC_EALIGN;
    if (m >= (1 << 24)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    const int row_blocks = (int)((m + kWave - 1) / kWave);
    const int cols = (int)(n / 64);
    // Workgroups per row block.  Splitting the columns spreads the table look-ups, which bound the decode (two-byte
    // gathers from 128 KiB: about twelve clocks of a CU's LDS per wave and look-up), over more CUs, and costs three
    // dependent trips to memory at the end (partial sums out, arrival counted, partial sums in: 3-4 us measured).
    // As written a column costs a workgroup about 0.03 us, so the split pays from 128 columns on, and a workgroup
    // keeps at least 32; in continuous mode (eight times the look-ups) it nearly always pays, and a wave keeps at
    // least one column.  Never more workgroups than CUs: each one fills its own table first.
    int ksplit = dev->cus / row_blocks;
    if (ksplit > kTMaxSplit) ksplit = kTMaxSplit;
    const int keep = carry_mode == RPTC_AS_WRITTEN ? 32 : kTWaves;
    if (ksplit > cols / keep) ksplit = cols / keep;
    if (carry_mode == RPTC_AS_WRITTEN && cols < 128) ksplit = 1;
    if (ksplit < 1 || row_blocks * ksplit > kTMaxParts) ksplit = 1;
    const int lds_bytes = lds_bytes_t<L>((cols + ksplit - 1) / ksplit, carry_mode);     // (at most 146 KiB: n <= 32768)
    if (lds_bytes > kMaxLds) return RPTC_ELIMIT;
    const TScratch &sc = g_t[dev->device];
    auto a_comp = reinterpret_cast<const uint4 *>(compressed);
    auto a_cb = reinterpret_cast<const uint4 *>(codebook);
    auto a_x = reinterpret_cast<const uint32_t *>(x);
    if (carry_mode == RPTC_AS_WRITTEN)
        hipLaunchKernelGGL((matvec_t_kernel<L, RPTC_AS_WRITTEN>), dim3(row_blocks * ksplit), dim3(kTThreads),
                           lds_bytes, s, a_comp, a_cb, a_x, (int)m, cols, ksplit, out, sc.parts, sc.arrived);
    else
        hipLaunchKernelGGL((matvec_t_kernel<L, RPTC_CONTINUOUS>), dim3(row_blocks * ksplit), dim3(kTThreads),
                           lds_bytes, s, a_comp, a_cb, a_x, (int)m, cols, ksplit, out, sc.parts, sc.arrived);
    return t.end();
}

template <int L>
static int launch_t_dense(const int32_t *compressed, const uint16_t *codebook, uint16_t *W, int64_t m,
                          int64_t n, int carry_mode, hipStream_t s)
{
    auto a_comp = reinterpret_cast<const uint4 *>(compressed);
    auto a_w = reinterpret_cast<uint32_t *>(W);
    const dim3 grid((unsigned)((m + 255) / 256), (unsigned)(n / 64));
    if (carry_mode == RPTC_AS_WRITTEN)
        hipLaunchKernelGGL((matvec_t_dense_kernel<L, RPTC_AS_WRITTEN>), grid, dim3(256), 0, s, a_comp, codebook, a_w,
                           (int)m, (int)(n / 64));
    else
        hipLaunchKernelGGL((matvec_t_dense_kernel<L, RPTC_CONTINUOUS>), grid, dim3(256), 0, s, a_comp, codebook, a_w,
                           (int)m, (int)(n / 64));
    return 0;
}

void matvec_t_counters(int device, uint32_t **counters, int *count)
{
    *counters = g_t[device].arrived;
    *count = kTMaxParts;
}

int prepare_matvec_t(int device)
{
    // the device addresses of the static scratch arrays (the symbols themselves are not device addresses)
    int rc0 = (int)hipGetSymbolAddress(reinterpret_cast<void **>(&g_t[device].parts), HIP_SYMBOL(g_t_part));
    if (rc0) return rc0;
    rc0 = (int)hipGetSymbolAddress(reinterpret_cast<void **>(&g_t[device].arrived), HIP_SYMBOL(g_t_arrived));
    if (rc0) return rc0;
    const void *k[] = {
        reinterpret_cast<const void *>(matvec_t_kernel<16, RPTC_AS_WRITTEN>),
        reinterpret_cast<const void *>(matvec_t_kernel<16, RPTC_CONTINUOUS>),
        reinterpret_cast<const void *>(matvec_t_kernel<14, RPTC_AS_WRITTEN>),
        reinterpret_cast<const void *>(matvec_t_kernel<14, RPTC_CONTINUOUS>),
    };
    for (const void *f : k) {
        int rc = (int)hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_decompress_matvec_t_16(const int32_t *c, const uint16_t *cb, const uint16_t *x, uint16_t *out,
                                           int64_t m, int64_t n, int mode, void *stream, float *ms)
{
    return launch_matvec_t<16>(c, cb, x, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_t_14(const int32_t *c, const uint16_t *cb, const uint16_t *x, uint16_t *out,
                                           int64_t m, int64_t n, int mode, void *stream, float *ms)
{
    return launch_matvec_t<14>(c, cb, x, out, m, n, mode, stream, ms);
}

extern "C" int rptc_matvec_t_dense(const int32_t *compressed, const uint16_t *codebook, uint16_t *W, int64_t m,
                                   int64_t n, int L, int carry_mode, void *stream, float *ms)
{
    if (!compressed || !codebook || !W) return RPTC_ENULL;
    if (m < 1 || n < 64 || n % 64 != 0 || (L != 14 && L != 16)) return RPTC_ESHAPE;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(W)) return RPTC_EALIGN;
    if (m >= (1 << 24) || n / 64 >= 65536) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    if (L == 16) launch_t_dense<16>(compressed, codebook, W, m, n, carry_mode, s);
    else launch_t_dense<14>(compressed, codebook, W, m, n, carry_mode, s);
    return t.end();
}
