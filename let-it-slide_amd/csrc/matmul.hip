// Fused decode + small-batch mat-mat on the hashed pair stream: out[b][r] = sum_c W[r][c] x[b][c],
// batch 1..32, W the dense matrix the stream stands for (the same stream and codebook as the
// mat-vec: rptc_kernels/csrc/rptc_kernels/inference.cu:189-277 defines W; the reference has no
// batched kernel).
//
// gfx950 design: the products run on the matrix cores (v_mfma_f32_16x16x32_f16, fp32
// accumulate) and the decoder feeds them without ever materialising W:
//   * lanes are rows: lane (i = lane % 16, g = lane / 16) of wave c decodes stream element
//     (slab, row 16*rb + i, lane-of-row 4c + g).  Its 32 steps give 32 weight pairs; four pairs
//     are exactly the eight fp16 values lane (i, g) owes the MFMA's A operand, so eight MFMAs
//     consume the element.  The matching B operand is the activation pairs of the same steps for
//     batch column j = lane % 16, which depend only on (slab, 4c + g): a wave keeps them in 32
//     registers while it walks the row blocks.
//   * the decode is the mat-vec's (window pair per v_alignbit_b32, two hashes per v_pk_mad_u16,
//     one address op and one conflict-free LDS gather per pair) minus the per-pair dot product.
//   * a small pre-kernel writes the activations once in [slot][16 batch columns] order, the order
//     the B operand wants: a wave's read of one step's pairs is 256 consecutive bytes.  The image
//     (a few hundred KiB) stays in L2 and is read straight into registers one slab ahead; it lives
//     in a static device buffer (no allocation per call), so calls on different streams of one
//     device share it and must not overlap.
//   * a workgroup owns its rows for all slabs, keeps the 16x16 accumulators in registers and
//     adds the eight waves' tiles in a fixed order at the end: deterministic, no atomics.
#include "rptc_common.hpp"

namespace rptc {

constexpr int kMmThreads = 512;
constexpr int kMmWaves = kMmThreads / kWave;       // one wave per group of 4 lanes-of-row
constexpr int kMmTableBytes = 256 * 256;
constexpr int kMmMaxRowBlocks = 4;                 // 16-row blocks per workgroup
constexpr int kMmMaxN = 32768;
constexpr int kMmMaxBatch = 32;

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef uint32_t v4u32 __attribute__((ext_vector_type(4)));

// activations in [plane of 16 batch columns][slot][16] order, written by pack_x_kernel
static __device__ __align__(256) uint32_t g_xpack[(kMmMaxBatch / 16) * (kMmMaxN / 2) * 16];

// x: fp16 [batch][n] seen as dwords [batch][n/2]; slot P pairs x[8*idx + 2i], x[8*idx + 2i + 1]
// with i = P / (n/8), idx = P % (n/8) (inference.cu:215-221): dword 4*idx + i of the row.
__global__ __launch_bounds__(256) void pack_x_kernel(const uint32_t *__restrict__ x, uint32_t *__restrict__ xp,
                                                     int n, int batch, int planes)
{
    const int t = blockIdx.x * 256 + threadIdx.x;
    const int slots = n >> 1, n8 = n >> 3;
    if (t >= planes * slots * 16) return;
    const int j = t & 15, slot = (t >> 4) % slots, plane = (t >> 4) / slots;
    const int b = plane * 16 + j;
    const int i = slot / n8, idx = slot - i * n8;
    xp[t] = b < batch ? x[(size_t)b * slots + 4 * idx + i] : 0u;
}

template <int S>
__device__ __forceinline__ uint32_t mm_table_value(const uint32_t *__restrict__ codebook, int b)
{
    const uint32_t pair = codebook[b & ((1 << S) - 1)];
    return (pair & 0xFFFF7FFFu) | ((uint32_t)(b >> 7) << 15);
}

// four gathered pairs (steps q0..q3 of this lane's element) times the batch columns
__device__ __forceinline__ v4f32 mma4(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, uint32_t x0, uint32_t x1,
                                      uint32_t x2, uint32_t x3, v4f32 acc)
{
    const v4u32 a = {w0, w1, w2, w3};
    const v4u32 b = {x0, x1, x2, x3};
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, a), __builtin_bit_cast(v8f16, b), acc, 0,
                                                  0, 0);
}

// the two gathered pairs of one window register (high window first in the stream)
__device__ __forceinline__ void gather2(uint32_t g, uint32_t lane4, uint32_t &w_hi, uint32_t &w_lo)
{
    const uint32_t h = pk_hash16(g);
    w_hi = lds_read_abs(perm(h, lane4, 0x0C0C0700u));
    w_lo = lds_read_abs(and_or(h, 0xFF00u, lane4));
}

template <int S, int MODE>
__global__ __launch_bounds__(kMmThreads) void matmul_kernel(
    const uint4 *__restrict__ comp, const uint32_t *__restrict__ codebook, const uint4 *__restrict__ xp,
    uint16_t *__restrict__ out, int m, int n, int batch, int rows_per_block)
{
    extern __shared__ uint32_t lds[];
    float *part = reinterpret_cast<float *>(lds + kMmTableBytes / 4);   // [wave][rb][v][lane]

    const int tid = threadIdx.x, lane = tid & 63;
    const int c = __builtin_amdgcn_readfirstlane(tid >> 6);      // this wave's group of four lanes-of-row
    const int i = lane & 15, g = lane >> 4;
    // the table is the first thing in LDS and the kernel has no static LDS: it starts at address 0
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;
    const int T = n >> 11, Lt = (n & 2047) >> 6, slabs = T + (Lt ? 1 : 0);
    const int row0 = blockIdx.x * rows_per_block;
    const int row_blocks = rows_per_block >> 4;
    const uint32_t *comp32 = reinterpret_cast<const uint32_t *>(comp);

    for (int d = tid; d < kMmTableBytes / 4; d += kMmThreads) lds[d] = mm_table_value<S>(codebook, d >> 6);

    v4f32 acc[kMmMaxRowBlocks];
#pragma unroll
    for (int rb = 0; rb < kMmMaxRowBlocks; rb++) acc[rb] = v4f32{0.f, 0.f, 0.f, 0.f};

    // Everything a slab needs from memory is requested one slab ahead, straight into registers: this
    // lane's stream elements (one per row block) with their carry words, and the 32 activation pairs
    // of its batch column (lanes of one group read 64 consecutive bytes of the packed image, a wave
    // 256: coalesced, and the image stays in L2).  No LDS staging, so no barrier inside the loop.
    const uint32_t *xp32 = reinterpret_cast<const uint32_t *>(xp);
    uint4 e_next[kMmMaxRowBlocks];
    uint32_t carry_next[kMmMaxRowBlocks], xb_next[32];
    auto request = [&](int slab) {
        const int lanes = slab < T ? 32 : Lt;
        const size_t elem0 = slab < T ? (size_t)slab * m * 32 : (size_t)T * m * 32;
        const size_t slot0 = (size_t)(slab < T ? slab : T) * 1024;
        const int l = 4 * c + g;
        const bool has_l = l < lanes;
        // Activation pairs of step q for batch column i: slot 32q + l (full) or q*Lt + l (ragged).
        // Lanes past the end of a ragged row get zeros: whatever their (all-zero) element decodes
        // to is then multiplied by zero, so the decode needs no per-lane predicate.
        const uint32_t *xq = xp32 + (slot0 + (has_l ? l : 0)) * 16 + i;
#pragma unroll
        for (int q = 0; q < 32; q++) xb_next[q] = has_l ? xq[(size_t)q * lanes * 16] : 0u;
#pragma unroll
        for (int rb = 0; rb < kMmMaxRowBlocks; rb++) {
            const int row = row0 + 16 * rb + i;
            e_next[rb] = make_uint4(0, 0, 0, 0);
            carry_next[rb] = 0;
            if (rb < row_blocks && l < lanes && row < m) {
                const size_t ei = elem0 + (size_t)row * lanes + l;
                e_next[rb] = comp[ei];
                if (l > 0) carry_next[rb] = comp32[ei * 4 - 1];              // last word of the previous lane-of-row
                else if (MODE == RPTC_AS_WRITTEN) carry_next[rb] = e_next[rb].w;   // inference.cu:232: lane 0 keeps its own
                else if (slab > 0) carry_next[rb] = comp32[(((size_t)(slab - 1) * m + row) * 32 + 31) * 4 + 3];
            }
        }
    };
    request(0);
    __syncthreads();                                              // the table is complete

    for (int slab = 0; slab < slabs; slab++) {
        const int lanes = slab < T ? 32 : Lt;                     // elements per row in this slab
        uint4 e_cur[kMmMaxRowBlocks];
        uint32_t carry_cur[kMmMaxRowBlocks], xb[32];
#pragma unroll
        for (int rb = 0; rb < kMmMaxRowBlocks; rb++) {
            e_cur[rb] = e_next[rb];
            carry_cur[rb] = carry_next[rb];
        }
#pragma unroll
        for (int q = 0; q < 32; q++) xb[q] = xb_next[q];
        if (slab + 1 < slabs) request(slab + 1);
        if (4 * c >= lanes) continue;                             // nothing of this slab for this wave

#pragma unroll
        for (int rb = 0; rb < kMmMaxRowBlocks; rb++) {
            if (rb >= row_blocks) break;
            const uint4 e = e_cur[rb];
            const uint32_t carry = carry_cur[rb];
            // rows past m decode zeros into tile rows that are never stored
            v4f32 d0 = acc[rb], d1 = v4f32{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t sh = 12 - 4 * j;
                const uint32_t gc = j == 3 ? e.x : alignbit(carry, e.x, sh);   // steps (7,j) and (0,j)
                const uint32_t gx = j == 3 ? e.y : alignbit(e.x, e.y, sh);     // (4,j), (1,j)
                const uint32_t gy = j == 3 ? e.z : alignbit(e.y, e.z, sh);     // (5,j), (2,j)
                const uint32_t gz = j == 3 ? e.w : alignbit(e.z, e.w, sh);     // (6,j), (3,j)
                uint32_t w0, w1, w2, w3, w4, w5, w6, w7;
                gather2(gc, lane4, w0, w1);
                gather2(gx, lane4, w2, w3);
                gather2(gy, lane4, w4, w5);
                gather2(gz, lane4, w6, w7);
                d0 = mma4(w0, w1, w2, w3, xb[28 + j], xb[j], xb[16 + j], xb[4 + j], d0);
                d1 = mma4(w4, w5, w6, w7, xb[20 + j], xb[8 + j], xb[24 + j], xb[12 + j], d1);
            }
            acc[rb] = d0 + d1;
        }
    }

    // add the waves' 16x16 tiles in a fixed order.  Tile element (row 4*(lane/16) + v, batch lane%16)
    // sits in register v of lane `lane`.
    __syncthreads();
#pragma unroll
    for (int rb = 0; rb < kMmMaxRowBlocks; rb++) {
        if (rb < row_blocks) {
#pragma unroll
            for (int v = 0; v < 4; v++) part[((c * row_blocks + rb) * 4 + v) * 64 + lane] = acc[rb][v];
        }
    }
    __syncthreads();
    for (int t = tid; t < row_blocks * 256; t += kMmThreads) {
        const int ln = t & 63, v = (t >> 6) & 3, rb = t >> 8;
        float y = 0.f;
#pragma unroll
        for (int w = 0; w < kMmWaves; w++) y += part[((w * row_blocks + rb) * 4 + v) * 64 + ln];
        const int b = ln & 15, row = row0 + 16 * rb + 4 * (ln >> 4) + v;
        if (b < batch && row < m) out[(size_t)b * m + row] = float_to_half_bits(y);
    }
}

static uint32_t *g_xpack_ptr[64];   // per device: address of g_xpack

int prepare_matmul(int device)
{
    const void *k[] = {
        reinterpret_cast<const void *>(matmul_kernel<6, RPTC_AS_WRITTEN>),
        reinterpret_cast<const void *>(matmul_kernel<6, RPTC_CONTINUOUS>),
        reinterpret_cast<const void *>(matmul_kernel<8, RPTC_AS_WRITTEN>),
        reinterpret_cast<const void *>(matmul_kernel<8, RPTC_CONTINUOUS>),
    };
    for (const void *f : k) {
        int rc = (int)hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
        if (rc) return rc;
    }
    // the device address of the static scratch image (the symbol itself is not a device address)
    return (int)hipGetSymbolAddress(reinterpret_cast<void **>(&g_xpack_ptr[device]), HIP_SYMBOL(g_xpack));
}

template <int S>
static void launch_planes(const uint4 *comp, const uint32_t *cb, const uint32_t *x, uint32_t *xp, uint16_t *out,
                          int m, int n, int batch, int carry_mode, int cus, hipStream_t s)
{
    const int planes = (batch + 15) / 16;
    const int total = planes * (n / 2) * 16;
    hipLaunchKernelGGL(pack_x_kernel, dim3((total + 255) / 256), dim3(256), 0, s, x, xp, n, batch, planes);
    int row_blocks = (m + 16 * cus - 1) / (16 * cus);
    if (row_blocks > kMmMaxRowBlocks) row_blocks = kMmMaxRowBlocks;
    const int rows_per_block = 16 * row_blocks;
    const int grid = (m + rows_per_block - 1) / rows_per_block;
    const int lds_bytes = kMmTableBytes + kMmWaves * row_blocks * 4 * 64 * 4;
    for (int p = 0; p < planes; p++) {
        const uint4 *xp_plane = reinterpret_cast<const uint4 *>(xp + (size_t)p * (n / 2) * 16);
        uint16_t *out_plane = out + (size_t)p * 16 * m;
        const int b = batch - 16 * p < 16 ? batch - 16 * p : 16;
        if (carry_mode == RPTC_AS_WRITTEN)
            hipLaunchKernelGGL((matmul_kernel<S, RPTC_AS_WRITTEN>), dim3(grid), dim3(kMmThreads), lds_bytes, s, comp,
                               cb, xp_plane, out_plane, m, n, b, rows_per_block);
        else
            hipLaunchKernelGGL((matmul_kernel<S, RPTC_CONTINUOUS>), dim3(grid), dim3(kMmThreads), lds_bytes, s, comp,
                               cb, xp_plane, out_plane, m, n, b, rows_per_block);
    }
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_decompress_matmul(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                      uint16_t *out, int64_t m, int64_t n, int64_t batch, int S, int carry_mode,
                                      void *stream, float *ms)
{
    if (!compressed || !codebook || !x || !out) return RPTC_ENULL;
    if (m < 1 || n < 64 || n % 64 != 0 || batch < 1 || (S != 6 && S != 8)) return RPTC_ESHAPE;
    if (n > kMmMaxN || batch > kMmMaxBatch || m >= (1 << 24)) return RPTC_ELIMIT;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(x)) return RPTC_EALIGN;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_comp = reinterpret_cast<const uint4 *>(compressed);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    auto a_x = reinterpret_cast<const uint32_t *>(x);
    uint32_t *xp = g_xpack_ptr[dev->device];
    if (S == 6) launch_planes<6>(a_comp, a_cb, a_x, xp, out, (int)m, (int)n, (int)batch, carry_mode, dev->cus, s);
    else launch_planes<8>(a_comp, a_cb, a_x, xp, out, (int)m, (int)n, (int)batch, carry_mode, dev->cus, s);
    return t.end();
}
