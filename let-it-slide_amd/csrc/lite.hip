// The general (L, S, R, V) hashed-codebook trellis of rptc_lite.py: dequantize.
//
// Semantics: rptc_lite.py:63-73 (dequantize: state = (state << R) | symbol on an int32 register that is never masked,
// output = alphabet[index_fn(state)]) with index_fn of rptc_lite.py:12-16 (x * (2x + 1) with int32 wraparound,
// x ^= x >> (L - S) with the arithmetic shift of a signed value, the low S bits).
//
// The register after step t is the OR of the last ceil(32 / R) symbols, symbol t - k shifted left by R k (bits that
// leave the 32-bit register are gone), so nothing is sequential: a thread rebuilds the register at its first step from
// the symbols in front of it and then walks kLiteSteps steps.  Symbols are used as the reference uses them, all 32
// bits, so a symbol outside [0, 2^R) spoils the steps behind it exactly as it does there.
//
// Bytes: 4 per symbol read, 4 V per symbol written (the reference's int32 symbols and float32 alphabet).
//   V == 2 (the reference's setting, rptc_lite.py:118): a workgroup takes 512 consecutive steps of a sequence at a time.
//     Its symbols and the 32 in front of them go through LDS (one coalesced request per wave), a thread folds the
//     history of its two steps from there, looks its two pairs up in an LDS copy of the alphabet (S <= 12; from the
//     caches above that) and writes them as one 16-byte store, so a wave writes 1 KiB contiguous.  A workgroup keeps
//     its copy of the alphabet while it walks over sequences.
//   other V: a thread reads its kLiteSteps symbols and the history in front of them (lines its neighbours read as
//     well) and writes kLiteSteps V consecutive floats.
#include "rptc_common.hpp"

namespace rptc {

constexpr int kLiteThreads = 256;
constexpr int kLiteSteps = 8;          // consecutive steps of one sequence per thread
constexpr int kLiteMaxV = 8;

__device__ __forceinline__ uint32_t lite_index(uint32_t state, int shift, uint32_t mask)
{
    const uint32_t p = state * (2u * state + 1u);
    const int32_t s = static_cast<int32_t>(p);
    return static_cast<uint32_t>(s ^ (s >> shift)) & mask;
}

__global__ __launch_bounds__(kLiteThreads) void lite_dequantize_kernel(
    const float *__restrict__ alphabet, const int32_t *__restrict__ symbols, float *__restrict__ out, int64_t length, int rows,
    uint32_t chunks_per_row, int R, int history, int shift, uint32_t mask, int vs)
{
    // grid: x over a sequence's chunks of kLiteSteps steps, y over sequences (strided when there are more than the grid has)
    const uint32_t chunk = blockIdx.x * kLiteThreads + threadIdx.x;
    if (chunk >= chunks_per_row) return;
    const int64_t t0 = (int64_t)chunk * kLiteSteps;
    const int steps = (int)(length - t0 < kLiteSteps ? length - t0 : kLiteSteps);
    for (int row = blockIdx.y; row < rows; row += gridDim.y) {
        const int32_t *sym = symbols + (int64_t)row * length;
        // this chunk's symbols, all requested before any is used (past the sequence's end: its last symbol, unused)
        uint32_t own[kLiteSteps];
#pragma unroll
        for (int i = 0; i < kLiteSteps; i++) own[i] = static_cast<uint32_t>(sym[t0 + (i < steps ? i : steps - 1)]);
        // the register in front of step t0: symbols t0 - history .. t0 - 1 (those that exist), oldest first
        uint32_t state = 0;
        for (int k = history; k >= 1; k--) {
            const int64_t t = t0 - k;
            if (t >= 0) state = (state << R) | static_cast<uint32_t>(sym[t]);
        }
        uint32_t idx[kLiteSteps];
#pragma unroll
        for (int i = 0; i < kLiteSteps; i++) {
            state = (state << R) | own[i];
            idx[i] = lite_index(state, shift, mask);
        }
        float *o = out + ((int64_t)row * length + t0) * vs;
#pragma unroll
        for (int i = 0; i < kLiteSteps; i++) {
            if (i >= steps) break;
            const float *a = alphabet + (size_t)idx[i] * vs;
            for (int v = 0; v < vs; v++) o[i * vs + v] = a[v];
        }
    }
}

constexpr int kLiteTile = 2 * kLiteThreads;    // steps of one sequence a workgroup takes at a time (V == 2)
constexpr int kLiteHalo = 32;                  // symbols in front of a tile that can still be in the register
constexpr int kLiteLdsAlphabetS = 12;          // the alphabet is copied to LDS up to 2^12 pairs (32 KiB)

template <bool ALPHABET_IN_LDS>
__global__ __launch_bounds__(kLiteThreads) void lite_dequantize_pairs_kernel(
    const float2 *__restrict__ alphabet, const int32_t *__restrict__ symbols, float *__restrict__ out, int64_t length, int rows,
    int R, int history, int shift, uint32_t mask)
{
    extern __shared__ uint32_t lite_lds[];
    uint32_t *tile = lite_lds;                                                  // [kLiteHalo + kLiteTile]
    float2 *table = reinterpret_cast<float2 *>(lite_lds + kLiteHalo + kLiteTile);   // [mask + 1] when ALPHABET_IN_LDS
    const int tid = threadIdx.x;
    if (ALPHABET_IN_LDS)
        for (uint32_t i = tid; i <= mask; i += kLiteThreads) table[i] = alphabet[i];
    const int64_t base = (int64_t)blockIdx.x * kLiteTile;      // the tile's first step
    const int64_t t0 = base + 2 * tid;                          // this thread's two steps
    for (int row = blockIdx.y; row < rows; row += gridDim.y) {
        const int32_t *sym = symbols + (int64_t)row * length;
        // own symbols and, from the first 32 threads, the halo; a step that does not exist counts as symbol 0,
        // which leaves the register as the missing step would
        const uint32_t s0 = t0 < length ? static_cast<uint32_t>(sym[t0]) : 0u;
        const uint32_t s1 = t0 + 1 < length ? static_cast<uint32_t>(sym[t0 + 1]) : 0u;
        uint32_t halo = 0u;
        if (tid < kLiteHalo) {
            const int64_t t = base - kLiteHalo + tid;
            if (t >= 0) halo = static_cast<uint32_t>(sym[t]);
        }
        __syncthreads();                     // the previous sequence's tile has been read (and the table is written)
        tile[kLiteHalo + 2 * tid] = s0;
        tile[kLiteHalo + 2 * tid + 1] = s1;
        if (tid < kLiteHalo) tile[tid] = halo;
        __syncthreads();
        uint32_t state = 0;
        for (int k = history; k >= 1; k--) state = (state << R) | tile[kLiteHalo + 2 * tid - k];
        state = (state << R) | s0;
        const uint32_t i0 = lite_index(state, shift, mask);
        state = (state << R) | s1;
        const uint32_t i1 = lite_index(state, shift, mask);
        const float2 w0 = ALPHABET_IN_LDS ? table[i0] : alphabet[i0];
        const float2 w1 = ALPHABET_IN_LDS ? table[i1] : alphabet[i1];
        float *o = out + ((int64_t)row * length + t0) * 2;
        if (t0 + 1 < length) {
            if ((reinterpret_cast<uintptr_t>(o) & 15u) == 0) {
                *reinterpret_cast<float4 *>(o) = make_float4(w0.x, w0.y, w1.x, w1.y);
            } else {
                reinterpret_cast<float2 *>(o)[0] = w0;
                reinterpret_cast<float2 *>(o)[1] = w1;
            }
        } else if (t0 < length) {
            reinterpret_cast<float2 *>(o)[0] = w0;
        }
    }
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_lite_dequantize(const float *alphabet, int L, int S, int R, int V, const int32_t *symbols, int64_t rows,
                                    int64_t length, float *out, void *stream, float *ms)
{
    if (!alphabet || !symbols || !out) return RPTC_ENULL;
    if (R < 1 || R > 16 || S < 1 || S > 16 || L < S || L > 31 || V < 1 || V > kLiteMaxV) return RPTC_ESHAPE;
    if (rows < 1 || length < 1 || rows > 0x7FFFFFFF) return RPTC_ESHAPE;
    const uintptr_t vec = V == 2 ? 7u : 3u;      // pairs are moved as one 8-byte value
    if ((reinterpret_cast<uintptr_t>(alphabet) & vec) || (reinterpret_cast<uintptr_t>(symbols) & 3u) ||
        (reinterpret_cast<uintptr_t>(out) & vec))
        return RPTC_EALIGN;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    const int64_t chunks_per_row = (length + kLiteSteps - 1) / kLiteSteps;
    const int64_t blocks = (chunks_per_row + kLiteThreads - 1) / kLiteThreads;
    if (chunks_per_row > 0xFFFFFFFFll || blocks > 0x7FFFFFFF) return RPTC_ELIMIT;
    const uint32_t grid_y = (uint32_t)(rows < 65535 ? rows : 65535);
    // every symbol whose bits are still in the 32-bit register: symbol t - k sits at bit R k
    const int history = (32 + R - 1) / R - 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    const uint32_t mask = (1u << S) - 1u;
    if (V == 2) {
        // 512 steps of a sequence per workgroup and turn; enough workgroups to fill the device, each walking over
        // sequences with its copy of the alphabet
        const int64_t tiles = (length + kLiteTile - 1) / kLiteTile;
        if (tiles > 0x7FFFFFFF) return RPTC_ELIMIT;
        int64_t want_y = ((int64_t)dev->cus * 8 + tiles - 1) / tiles;
        if (want_y > rows) want_y = rows;
        if (want_y > 65535) want_y = 65535;
        if (want_y < 1) want_y = 1;
        const bool in_lds = S <= kLiteLdsAlphabetS;
        const size_t lds = (size_t)(kLiteHalo + kLiteTile) * 4 + (in_lds ? ((size_t)8 << S) : 0);
        const float2 *pairs = reinterpret_cast<const float2 *>(alphabet);
        if (in_lds)
            hipLaunchKernelGGL(lite_dequantize_pairs_kernel<true>, dim3((uint32_t)tiles, (uint32_t)want_y), dim3(kLiteThreads), lds, s,
                               pairs, symbols, out, length, (int)rows, R, history, L - S, mask);
        else
            hipLaunchKernelGGL(lite_dequantize_pairs_kernel<false>, dim3((uint32_t)tiles, (uint32_t)want_y), dim3(kLiteThreads), lds, s,
                               pairs, symbols, out, length, (int)rows, R, history, L - S, mask);
    } else {
        hipLaunchKernelGGL(lite_dequantize_kernel, dim3((uint32_t)blocks, grid_y), dim3(kLiteThreads), 0, s, alphabet, symbols, out,
                           length, (int)rows, (uint32_t)chunks_per_row, R, history, L - S, mask, V);
    }
    return t.end();
}
