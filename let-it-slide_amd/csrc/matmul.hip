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
//   * a workgroup owns one slab (2048 columns) of a group of up to 128 rows, so the activation pairs
//     a wave holds serve every row block of the group (a workgroup that owned whole rows would read
//     the complete activation image for as few as 16 rows: eight times the bytes of its stream).
//     Its eight waves' 16x16 tiles are added in LDS in a fixed order and go to a static scratch
//     buffer as fp32; the workgroup that finishes a row group last (a counter per group) adds the
//     slabs' partial tiles in slab order and writes fp16.  The order of every sum is fixed, so the
//     output is deterministic whichever workgroup comes last.
//   * batch 17..32 decodes once and feeds two sets of MFMAs (two planes of 16 batch columns).
#include "rptc_common.hpp"

namespace rptc {

constexpr int kMmThreads = 512;
constexpr int kMmWaves = kMmThreads / kWave;       // one wave per group of 4 lanes-of-row
constexpr int kMmTableBytes = 256 * 256;
constexpr int kMmMaxRowBlocks = 8;                 // 16-row blocks per workgroup (6 with two planes: registers)
constexpr int kMmScratchFloats = 8 << 20;          // 32 MiB of partial tiles
constexpr int kMmMaxGroups = 32768;
constexpr int kMmMaxN = 32768;
constexpr int kMmMaxBatch = 32;

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef uint32_t v4u32 __attribute__((ext_vector_type(4)));

// activations in [plane of 16 batch columns][slot][16] order, written by pack_x_kernel
static __device__ __align__(256) uint32_t g_xpack[(kMmMaxBatch / 16) * (kMmMaxN / 2) * 16];
// partial tiles [row group][slab][row block][plane][256] and one arrival counter per row group
static __device__ __align__(256) float g_partial[kMmScratchFloats];
static __device__ __align__(256) uint32_t g_arrived[kMmMaxGroups];

// x: fp16 [batch][n]; slot P pairs x[8*idx + 2i], x[8*idx + 2i + 1] with i = P / (n/8), idx = P % (n/8)
// (inference.cu:215-221).  Thread (plane, idx, j) reads the 16 bytes x[16*plane + j][8*idx .. 8*idx+7]
// (a wave: 16 rows x 64 contiguous bytes) and writes one dword to each of the slots i*(n/8) + idx,
// i = 0..3 (a wave: 256 contiguous bytes per i).
__global__ __launch_bounds__(256) void pack_x_kernel(const uint4 *__restrict__ x, uint32_t *__restrict__ xp,
                                                     uint32_t *__restrict__ arrived, int groups, int n, int batch,
                                                     int planes)
{
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t < groups) arrived[t] = 0;   // the counters start every call at zero, whatever an earlier call left
    const int n8 = n >> 3;
    if (t >= planes * n8 * 16) return;
    const int j = t & 15, idx = (t >> 4) % n8, plane = (t >> 4) / n8;
    const int b = plane * 16 + j;
    const uint4 v = b < batch ? x[(size_t)b * n8 + idx] : make_uint4(0, 0, 0, 0);
    uint32_t *dst = xp + (size_t)plane * (n >> 1) * 16 + (size_t)idx * 16 + j;
    dst[0] = v.x;
    dst[(size_t)n8 * 16] = v.y;
    dst[(size_t)n8 * 32] = v.z;
    dst[(size_t)n8 * 48] = v.w;
}

// The packed image of the row-owner kernel below: the four activation pairs that one MFMA's B operand takes from a lane
// are 16 consecutive bytes.  Step q = 4k + j of lane-of-row l in slab t (slot 1024 t + q * lanes + l, `lanes` elements a
// row in that slab) goes to dword ((((32 t + l) * 8 + 2 j + h) * 16 + b) * 4 + p) of its plane, b the batch column, with
// (h, p) = (0, 0..3) for k = 7, 0, 4, 1 and (1, 0..3) for k = 5, 2, 6, 3: the order in which the steps of an element meet
// the slots (inference.cu:237-250).  A ragged last slab is padded with zeros to a multiple of four lanes-of-row.
// Thread (idx, b) reads the 16 bytes x[b][8 idx .. 8 idx + 7] (slots i * (n/8) + idx, i = 0..3) as pack_x_kernel does;
// the threads behind them write the padding.
__device__ __forceinline__ size_t mm_tuple_position(int slot, int n, int b)
{
    const int T = n >> 11, Lt = (n & 2047) >> 6;
    const int t = slot >> 10 < T ? slot >> 10 : T;
    const int lanes = t < T ? 32 : Lt;
    const int r = slot - (t << 10), q = r / lanes, l = r - q * lanes;
    const int k = q >> 2, j = q & 3;
    // k:     0  1  2  3  4  5  6  7
    // half:  0  0  1  1  0  1  1  0
    // pos:   1  3  1  3  2  0  2  0
    const int h = (0x6C >> k) & 1, pos = (0x22DD >> (2 * k)) & 3;     // two bits of position per k, k = 0 lowest
    return ((((size_t)(32 * t + l) * 8 + 2 * j + h) * 16 + b) << 2) + pos;
}

__global__ __launch_bounds__(256) void pack_x_tuples_kernel(const uint4 *__restrict__ x, uint32_t *__restrict__ xp, int n, int batch)
{
    const int t = blockIdx.x * 256 + threadIdx.x;
    const int n8 = n >> 3, b = t & 15, idx = t >> 4;
    if (idx < n8) {
        const uint4 v = b < batch ? x[(size_t)b * n8 + idx] : make_uint4(0, 0, 0, 0);
        xp[mm_tuple_position(idx, n, b)] = v.x;
        xp[mm_tuple_position(n8 + idx, n, b)] = v.y;
        xp[mm_tuple_position(2 * n8 + idx, n, b)] = v.z;
        xp[mm_tuple_position(3 * n8 + idx, n, b)] = v.w;
        return;
    }
    // the lanes-of-row Lt .. 4 * ceil(Lt / 4) - 1 of the ragged slab: 512 dwords each
    const int T = n >> 11, Lt = (n & 2047) >> 6;
    const int pad = (t - n8 * 16) * 4;                                   // four dwords a thread
    if (pad < (((Lt + 3) & ~3) - Lt) * 512)
        *reinterpret_cast<uint4 *>(xp + (size_t)(32 * T + Lt) * 512 + pad) = make_uint4(0, 0, 0, 0);
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

// Row blocks a workgroup can hold in registers beside the activation pairs.
__host__ __device__ constexpr int mm_max_row_blocks(int planes, int bits)
{
    return bits == 2 ? (planes == 1 ? kMmMaxRowBlocks : 6) : (planes == 1 ? 6 : 3);   // even for one plane
}

// Step s of an element multiplies activation slot 4k + j with k = 7, 0, 4, 1, 5, 2, 6, 3 for
// s / 4 = 0..7 and j = s % 4 (inference.cu:237-250).
__device__ constexpr int mm_k_of_step_block(int sb)
{
    constexpr int k_of[8] = {7, 0, 4, 1, 5, 2, 6, 3};
    return k_of[sb];
}

// BITS: bits per weight.  2 is the reference stream (an element is 4 words, two windows per
// v_alignbit_b32); at 3 and 4 an element is 2 * BITS words, a step advances 2 * BITS stream bits, and
// the four windows of an MFMA's A operand are cut out one by one.
// four waves per SIMD = two workgroups per CU: at most 128 vector registers
// (arguments in the order of their first use: the first 14 dwords arrive preloaded in SGPRs)
template <int S, int MODE, int PLANES, int BITS>
__global__ __launch_bounds__(kMmThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void matmul_kernel(
    const uint32_t *__restrict__ comp32, const uint32_t *__restrict__ codebook, const uint32_t *__restrict__ xp32,
    int m, int n, int rb_quot, int rb_rem, int group_base, int max_rb, float *__restrict__ partial,
    uint32_t *__restrict__ arrived, uint16_t *__restrict__ out, int batch)
{
    extern __shared__ uint32_t lds[];
    // 64 KiB of table + 16 KiB of tiles: two workgroups share a CU's 160 KiB whatever the batch
    constexpr int kPartBuffers = PLANES == 1 ? 2 : 1;
    constexpr int WORDS = 2 * BITS;                               // words per stream element
    constexpr int kMaxRb = mm_max_row_blocks(PLANES, BITS);
    float *part = reinterpret_cast<float *>(lds + kMmTableBytes / 4);   // [buffer][wave][plane][v][lane]
    // the "came last" flag reuses the first word of the tiles once they are no longer read (all LDS
    // is dynamic, and 64 + 16 KiB lets two workgroups share a CU)
    uint32_t *s_last = lds + kMmTableBytes / 4;

    const int tid = threadIdx.x, lane = tid & 63;
    const int c = __builtin_amdgcn_readfirstlane(tid >> 6);      // this wave's group of four lanes-of-row
    const int i = lane & 15, g = lane >> 4;
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;
    const int T = n >> 11, Lt = (n & 2047) >> 6, slabs = T + (Lt ? 1 : 0);
    // grp counts the row groups of this launch (a very tall matrix takes several launches)
    const int grp = blockIdx.x / slabs, slab = blockIdx.x - grp * slabs;
    // the row blocks (16 rows each) are dealt to the groups as evenly as integers allow: rb_quot each,
    // one more for the first rb_rem groups (quotient and remainder of row blocks / groups, from the host:
    // a division here would be a loop of a few hundred instructions in front of the first request)
    const int g_all = group_base + grp;
    const int rb_begin = g_all * rb_quot + min(g_all, rb_rem);
    const int row_blocks = rb_quot + (g_all < rb_rem ? 1 : 0);
    const int row0 = rb_begin * 16;

    const int lanes = slab < T ? 32 : Lt;                        // elements per row in this slab
    const size_t elem0 = (size_t)(slab < T ? slab : T) * m * 32;
    const size_t slot0 = (size_t)(slab < T ? slab : T) * 1024;
    const int l = 4 * c + g;
    const bool has_l = l < lanes;
    const int waves_used = (lanes + 3) >> 2;

    // Table rows 32 * c .. 32 * c + 31 are this wave's to write.  A row is 64 copies of one value, so the
    // value is wave-uniform and comes through the scalar cache: these loads neither queue with the vector
    // loads below nor return in order with them.
    constexpr int kTableRowsPerWave = 256 / kMmWaves;
    uint32_t table_values[kTableRowsPerWave];
#pragma unroll
    for (int r = 0; r < kTableRowsPerWave; r++) table_values[r] = mm_table_value<S>(codebook, kTableRowsPerWave * c + r);

    // Everything comes straight into registers, all requests before the first use: the activation
    // pairs of this lane's 32 steps for its batch column(s) (lanes of one group read 64 consecutive
    // bytes of the packed image, a wave 256), and this lane's element of every row block with its
    // carry word.  Lanes past the end of a ragged row get zero activations: whatever their all-zero
    // element decodes to is multiplied by zero, so the decode needs no per-lane predicate.
    uint32_t xb[PLANES][32];
    {
        const uint32_t *xq = xp32 + (slot0 + (has_l ? l : 0)) * 16 + i;
#pragma unroll
        for (int p = 0; p < PLANES; p++)
#pragma unroll
            for (int q = 0; q < 32; q++) xb[p][q] = has_l ? xq[(size_t)p * (n >> 1) * 16 + (size_t)q * lanes * 16] : 0u;
    }
    // No branch around these loads and no use of their results before the row-block loop: a lane
    // with nothing to decode (row past m, lane past a ragged row, row block past the group) reads
    // element 0 instead, which is harmless: its products are multiplied by zero activations or land
    // in tile rows that are never stored.  Lane-of-row 0 reads its own last word as the carry
    // (inference.cu:232, as written) or lane 31 of the previous slab (continuous).
    uint32_t e_all[kMaxRb][WORDS];
    uint32_t carry_all[kMaxRb];
#pragma unroll
    for (int rb = 0; rb < kMaxRb; rb++) {
        const int row = row0 + 16 * rb + i;
        const bool valid = rb < row_blocks && has_l && row < m;
        const size_t ei = valid ? elem0 + (size_t)row * lanes + l : 0;
        size_t ci = ei * WORDS + WORDS - 1;
        if (l > 0 && valid) ci = ei * WORDS - 1;                         // last word of the previous lane-of-row
        else if (MODE == RPTC_CONTINUOUS && slab > 0 && valid) ci = (((size_t)(slab - 1) * m + row) * 32 + 31) * WORDS + WORDS - 1;
        if constexpr (WORDS % 4 == 0) {
#pragma unroll
            for (int q = 0; q < WORDS / 4; q++) {
                const uint4 v = reinterpret_cast<const uint4 *>(comp32 + ei * WORDS)[q];
                e_all[rb][4 * q] = v.x, e_all[rb][4 * q + 1] = v.y, e_all[rb][4 * q + 2] = v.z, e_all[rb][4 * q + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int q = 0; q < WORDS / 2; q++) {
                const uint2 v = reinterpret_cast<const uint2 *>(comp32 + ei * WORDS)[q];
                e_all[rb][2 * q] = v.x, e_all[rb][2 * q + 1] = v.y;
            }
        }
        carry_all[rb] = comp32[ci];
    }
    const bool no_carry = MODE == RPTC_CONTINUOUS && slab == 0 && l == 0;     // the stream starts here

    {
        // 64 lane copies of each of the wave's rows
#pragma unroll
        for (int r = 0; r < kTableRowsPerWave; r++) lds[(kTableRowsPerWave * c + r) * 64 + lane] = table_values[r];
    }
    __syncthreads();                                              // the table is complete

    float *my_partial = partial + ((size_t)blockIdx.x * max_rb) * (PLANES * 256);
#pragma unroll
    for (int rb = 0; rb < kMaxRb; rb++) {
        if (rb >= row_blocks) break;
        float *buf = part + (kPartBuffers == 2 ? (rb & 1) : 0) * (kMmWaves * PLANES * 256);
        if (c < waves_used) {
            const uint32_t carry = no_carry ? 0u : carry_all[rb];
            v4f32 d0[PLANES], d1[PLANES];
#pragma unroll
            for (int p = 0; p < PLANES; p++) d0[p] = d1[p] = v4f32{0.f, 0.f, 0.f, 0.f};
            if constexpr (BITS == 2) {
                const uint4 e = make_uint4(e_all[rb][0], e_all[rb][1], e_all[rb][2], e_all[rb][3]);
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
#pragma unroll
                    for (int p = 0; p < PLANES; p++) {
                        d0[p] = mma4(w0, w1, w2, w3, xb[p][28 + j], xb[p][j], xb[p][16 + j], xb[p][4 + j], d0[p]);
                        d1[p] = mma4(w4, w5, w6, w7, xb[p][20 + j], xb[p][8 + j], xb[p][24 + j], xb[p][12 + j], d1[p]);
                    }
                }
            } else {
                // four consecutive steps per MFMA: their slots are 4k .. 4k+3 of one k
                constexpr int SB = 2 * BITS;
#pragma unroll
                for (int sb = 0; sb < 8; sb++) {
                    uint32_t w[4];
                    if constexpr (BITS == 4) {
                        // a step is 8 bits: word sb as it is holds the windows of steps 4sb+1 and 4sb+3, and the
                        // 32 bits that start 8 bits before it those of steps 4sb and 4sb+2
                        const uint32_t front = sb == 0 ? carry : e_all[rb][sb > 0 ? sb - 1 : 0];
                        gather2(alignbit(front, e_all[rb][sb], 8), lane4, w[0], w[2]);
                        gather2(e_all[rb][sb], lane4, w[1], w[3]);
                    } else
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const int st = 4 * sb + u;
                        const int end = SB * (st + 1), start = end - 16;
                        uint32_t h;
                        if (start < 0) {
                            h = (carry << end) | (e_all[rb][0] >> (32 - end));
                        } else {
                            const int wi = start >> 5, o = start & 31;
                            h = o <= 16 ? e_all[rb][wi] >> (16 - o)
                                        : alignbit(e_all[rb][wi], e_all[rb][wi + 1 < WORDS ? wi + 1 : wi], 48 - o);
                        }
                        // hash of the low half (what sits in the high half is cut off by the address mask)
                        uint32_t prod;                                        // low 16 bits of h * (h + 1)
                        asm("v_pk_mad_u16 %0, %1, %1, %1" : "=v"(prod) : "v"(h));
                        w[u] = lds_read_abs(and_or(prod, 0xFF00u, lane4));
                    }
                    const int k = mm_k_of_step_block(sb);
#pragma unroll
                    for (int p = 0; p < PLANES; p++) {
                        v4f32 &d = (sb & 1) ? d1[p] : d0[p];
                        d = mma4(w[0], w[1], w[2], w[3], xb[p][4 * k], xb[p][4 * k + 1], xb[p][4 * k + 2], xb[p][4 * k + 3], d);
                    }
                }
            }
            // tile element (row 4*(lane/16) + v, batch column lane%16) sits in register v of lane `lane`
#pragma unroll
            for (int p = 0; p < PLANES; p++) {
                const v4f32 d = d0[p] + d1[p];
#pragma unroll
                for (int v = 0; v < 4; v++) buf[((c * PLANES + p) * 4 + v) * 64 + lane] = d[v];
            }
        }
        // With two buffers one barrier per row block is enough: the halves of `part` alternate, and a
        // wave can only reach the write of row block rb+2 after it passed the barrier of rb+1, which
        // every wave reaches after its sum of rb.
        __syncthreads();
        if (tid < PLANES * 256) {
            float y = 0.f;
            const int p = tid >> 8, vl = tid & 255;
            for (int w = 0; w < waves_used; w++) y += buf[(w * PLANES + p) * 256 + vl];
            // device-coherent store (written through the XCD's L2): visible to the workgroup on
            // another XCD that adds the slabs, without flushing a whole cache
            publishing();
            __hip_atomic_store(&my_partial[rb * (PLANES * 256) + tid], y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (kPartBuffers == 1) __syncthreads();                   // the one buffer is free again
    }

    // The workgroup that arrives last at its row group's counter adds the slabs' tiles, in slab order.
    // (the hand-off between workgroups: see published() / arrive() in rptc_common.hpp)
    published();
    __syncthreads();
    if (tid == 0) {
        const uint32_t prev = arrive(&arrived[grp]);
        const bool last = prev == (uint32_t)(slabs - 1);
        if (last) __hip_atomic_store(&arrived[grp], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        *s_last = last;
    }
    __syncthreads();
    if (!*s_last) return;
    const int tile_floats = row_blocks * PLANES * 256, tile_stride = max_rb * PLANES * 256;
    const float *grp_partial = partial + (size_t)grp * slabs * tile_stride;
    // every thread requests its share of four slabs' tiles before it adds any of them: the loads go
    // to memory, and one at a time they would cost a round trip each
    constexpr int kPerThread = kMaxRb * PLANES * 256 / kMmThreads;
    float y[kPerThread];
#pragma unroll
    for (int k = 0; k < kPerThread; k++) y[k] = 0.f;
    for (int sl0 = 0; sl0 < slabs; sl0 += 4) {
        float v[kPerThread][4];
        merging();
#pragma unroll
        for (int k = 0; k < kPerThread; k++)
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int t = tid + k * kMmThreads;
                v[k][u] = 0.f;
                if (t < tile_floats && sl0 + u < slabs)
                    v[k][u] = __hip_atomic_load(&grp_partial[(size_t)(sl0 + u) * tile_stride + t], __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
            }
        merged();
#pragma unroll
        for (int k = 0; k < kPerThread; k++)
#pragma unroll
            for (int u = 0; u < 4; u++) y[k] += v[k][u];          // slab order
    }
#pragma unroll
    for (int k = 0; k < kPerThread; k++) {
        const int t = tid + k * kMmThreads;
        if (t >= tile_floats) break;
        const int ln = t & 63, v = (t >> 6) & 3, p = (t >> 8) % PLANES, rb = t / (PLANES * 256);
        const int b = 16 * p + (ln & 15), row = row0 + 16 * rb + 4 * (ln >> 4) + v;
        if (b < batch && row < m) out[(size_t)b * m + row] = float_to_half_bits(y[k]);
    }
}

// ---------------------------------------------------------------- the row-owner form (2 bits, batch <= 16)
// A workgroup of 16 waves owns TILES blocks of 16 rows over the whole width, so nothing leaves the workgroup but the
// finished fp16 outputs: no partial tiles in memory, no arrival counters, no second pass.  The price is the one named
// above: every workgroup reads the whole packed activation image (from L2), 8 KiB for every 64 stream elements it
// decodes, so its first-level cache moves 352 KiB of activations for 44 KiB of stream on a 16 x 11008 share.
//   * a wave takes the (slab, group of four lanes-of-row) pairs w, w + 16, ... of the row; the 32 activation registers of
//     a pair serve its TILES row blocks.  They are refilled for the wave's next pair a quarter at a time, each quarter
//     as soon as the last row block has used it, so one set of 32 registers is enough.
//   * a wave's MFMA accumulators run over all its pairs; the 16 waves' tiles are added in LDS in wave order once.
constexpr int kMrThreads = 1024;
constexpr int kMrWaves = kMrThreads / kWave;
constexpr int kMrMaxTiles = 3;

template <int S, int MODE, int TILES>
__global__ __launch_bounds__(kMrThreads) void matmul_rows_kernel(const uint32_t *__restrict__ comp32,
                                                                 const uint32_t *__restrict__ codebook,
                                                                 const uint32_t *__restrict__ xp32, uint16_t *__restrict__ out,
                                                                 int m, int n, int batch)
{
    extern __shared__ uint32_t lds[];
    float *part = reinterpret_cast<float *>(lds + kMmTableBytes / 4);    // [wave][tile][v][lane]
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, g = lane >> 4;
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;
    const int T = n >> 11, Lt = (n & 2047) >> 6;
    const int pairs = 8 * T + ((Lt + 3) >> 2);                    // (slab, four lanes-of-row) pairs of a row
    const int row0 = blockIdx.x * (16 * TILES);

    constexpr int kTableRowsPerWave = 256 / kMrWaves;
    uint32_t table_values[kTableRowsPerWave];
#pragma unroll
    for (int r = 0; r < kTableRowsPerWave; r++) table_values[r] = mm_table_value<S>(codebook, kTableRowsPerWave * w + r);

    // what a pair's loads need: where its slab starts, how many elements a row has there, this lane's lane-of-row
    struct Pair {
        int slab, lanes, l;
        bool has_l;
    };
    auto pair_of = [&](int sq) {
        Pair p;
        p.slab = sq < 8 * T ? sq >> 3 : T;
        p.lanes = sq < 8 * T ? 32 : Lt;
        p.l = 4 * (sq - 8 * p.slab) + g;
        p.has_l = p.l < p.lanes;
        return p;
    };
    // this lane's element of row block t and the word in front of it (as in matmul_kernel: a lane with nothing to decode
    // reads element 0, and its products meet zero activations or land in rows that are never stored)
    auto load_element = [&](const Pair &p, int t, uint4 &e, uint32_t &carry) {
        const int row = row0 + 16 * t + i;
        const bool valid = p.has_l && row < m;
        const size_t ei = valid ? (size_t)p.slab * m * 32 + (size_t)row * p.lanes + p.l : 0;
        size_t ci = ei * 4 + 3;
        if (p.l > 0 && valid) ci = ei * 4 - 1;
        else if (MODE == RPTC_CONTINUOUS && p.slab > 0 && valid) ci = (((size_t)(p.slab - 1) * m + row) * 32 + 31) * 4 + 3;
        e = reinterpret_cast<const uint4 *>(comp32)[ei];
        carry = comp32[ci];
    };
    // the B operands of the two MFMAs of quarter j (steps 4k + j): 16 bytes each in the packed image, and zeros for a
    // lane past the end of a ragged row (pack_x_tuples_kernel pads), so no lane needs a predicate here
    auto load_quarter = [&](const Pair &p, int j, v4u32 (&xb)[8]) {
        const v4u32 *xq = reinterpret_cast<const v4u32 *>(xp32) + ((size_t)(32 * p.slab + p.l) * 8 + 2 * j) * 16 + i;
        xb[2 * j] = xq[0];
        xb[2 * j + 1] = xq[16];
    };
    // One pair's share of the product for every row block: quarter by quarter (the windows of a quarter come straight
    // from the element's words, so the order of the quarters is free), and behind each quarter the next pair's
    // activations for it when there is a next pair (`more` is a constant where this is expanded).
    auto consume = [&](const Pair &p, const Pair &next, bool more, v4u32 (&xb)[8], const uint4 (&e)[TILES],
                       const uint32_t (&carry)[TILES], v4f32 (&d)[TILES]) {
        const bool no_carry = MODE == RPTC_CONTINUOUS && p.slab == 0 && p.l == 0;    // the stream starts here
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t sh = 12 - 4 * j;
#pragma unroll
            for (int t = 0; t < TILES; t++) {
                const uint32_t cw = no_carry ? 0u : carry[t];
                const uint32_t gc = j == 3 ? e[t].x : alignbit(cw, e[t].x, sh);        // steps (7,j) and (0,j)
                const uint32_t gx = j == 3 ? e[t].y : alignbit(e[t].x, e[t].y, sh);    // (4,j), (1,j)
                const uint32_t gy = j == 3 ? e[t].z : alignbit(e[t].y, e[t].z, sh);    // (5,j), (2,j)
                const uint32_t gz = j == 3 ? e[t].w : alignbit(e[t].z, e[t].w, sh);    // (6,j), (3,j)
                // one accumulator: the second MFMA waits for the first, with the second half's decode between them
                uint32_t w0, w1, w2, w3, w4, w5, w6, w7;
                gather2(gc, lane4, w0, w1);
                gather2(gx, lane4, w2, w3);
                const v4u32 a0 = {w0, w1, w2, w3};
                d[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, a0), __builtin_bit_cast(v8f16, xb[2 * j]), d[t], 0, 0, 0);
                gather2(gy, lane4, w4, w5);
                gather2(gz, lane4, w6, w7);
                const v4u32 a1 = {w4, w5, w6, w7};
                d[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, a1), __builtin_bit_cast(v8f16, xb[2 * j + 1]), d[t], 0, 0, 0);
            }
            if (more) load_quarter(next, j, xb);                  // this quarter is free: the next pair's goes in
        }
    };

    int sq = w;
    Pair cur = pair_of(sq < pairs ? sq : 0);
    v4u32 xb[8];
    uint4 e[TILES];
    uint32_t carry[TILES];
    if (sq < pairs) {
#pragma unroll
        for (int t = 0; t < TILES; t++) load_element(cur, t, e[t], carry[t]);
#pragma unroll
        for (int j = 0; j < 4; j++) load_quarter(cur, j, xb);
    }
#pragma unroll
    for (int r = 0; r < kTableRowsPerWave; r++) lds[(kTableRowsPerWave * w + r) * 64 + lane] = table_values[r];
    __syncthreads();                                              // the table is complete

    v4f32 d[TILES];
#pragma unroll
    for (int t = 0; t < TILES; t++) d[t] = v4f32{0.f, 0.f, 0.f, 0.f};
    if (sq < pairs) {
        // every pair but the wave's last with the next pair's requests among the work, then the last without (one
        // loop with the requests under a condition would make every wait count as if they had not been made)
        while (sq + kMrWaves < pairs) {
            const Pair next = pair_of(sq + kMrWaves);
            uint4 en[TILES];
            uint32_t cn[TILES];
#pragma unroll
            for (int t = 0; t < TILES; t++) load_element(next, t, en[t], cn[t]);
            consume(cur, next, true, xb, e, carry, d);
#pragma unroll
            for (int t = 0; t < TILES; t++) e[t] = en[t], carry[t] = cn[t];
            cur = next;
            sq += kMrWaves;
        }
        consume(cur, cur, false, xb, e, carry, d);
    }

    // tile element (row 4*(lane/16) + v, batch column lane%16) sits in register v of lane `lane`
#pragma unroll
    for (int t = 0; t < TILES; t++)
#pragma unroll
        for (int v = 0; v < 4; v++) part[((w * TILES + t) * 4 + v) * 64 + lane] = d[t][v];
    __syncthreads();
    if (tid < TILES * 256) {
        const int t = tid >> 8, vl = tid & 255;
        float y = 0.f;
#pragma unroll
        for (int k = 0; k < kMrWaves; k++) y += part[(k * TILES + t) * 256 + vl];      // wave order
        const int ln = vl & 63, v = vl >> 6;
        const int b = ln & 15, row = row0 + 16 * t + 4 * (ln >> 4) + v;
        if (b < batch && row < m) out[(size_t)b * m + row] = float_to_half_bits(y);
    }
}

template <int S, int MODE>
static void launch_matmul_rows(const uint32_t *comp, const uint32_t *cb, const uint32_t *xpack, uint16_t *out, int m, int n,
                               int batch, int cus, hipStream_t s)
{
    const int total = (m + 15) / 16;
    int tiles = (total + cus - 1) / cus;                          // one workgroup per CU where the row blocks allow
    if (tiles > kMrMaxTiles) tiles = kMrMaxTiles;
    const int grid = (total + tiles - 1) / tiles;
    const int lds_bytes = kMmTableBytes + kMrWaves * tiles * 256 * 4;
    if (tiles == 1) hipLaunchKernelGGL((matmul_rows_kernel<S, MODE, 1>), dim3(grid), dim3(kMrThreads), lds_bytes, s, comp, cb, xpack, out, m, n, batch);
    else if (tiles == 2) hipLaunchKernelGGL((matmul_rows_kernel<S, MODE, 2>), dim3(grid), dim3(kMrThreads), lds_bytes, s, comp, cb, xpack, out, m, n, batch);
    else hipLaunchKernelGGL((matmul_rows_kernel<S, MODE, 3>), dim3(grid), dim3(kMrThreads), lds_bytes, s, comp, cb, xpack, out, m, n, batch);
}

struct MmScratch {
    uint32_t *xpack;
    float *partial;
    uint32_t *arrived;
    int64_t partial_floats;     // capacity of `partial`
};
static MmScratch g_mm[64];   // per device: addresses of the static scratch arrays

template <typename K>
static int mm_allow_lds(K kernel)
{
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    kMaxLds);
}

int prepare_matmul(int device)
{
    int rc;
#define RPTC_MM_ALLOW(PLANES, BITS)                                                          \
    if ((rc = mm_allow_lds(matmul_kernel<6, RPTC_AS_WRITTEN, PLANES, BITS>))) return rc;    \
    if ((rc = mm_allow_lds(matmul_kernel<6, RPTC_CONTINUOUS, PLANES, BITS>))) return rc;    \
    if ((rc = mm_allow_lds(matmul_kernel<8, RPTC_AS_WRITTEN, PLANES, BITS>))) return rc;    \
    if ((rc = mm_allow_lds(matmul_kernel<8, RPTC_CONTINUOUS, PLANES, BITS>))) return rc;
    RPTC_MM_ALLOW(1, 2)
    RPTC_MM_ALLOW(2, 2)
    RPTC_MM_ALLOW(1, 3)
    RPTC_MM_ALLOW(2, 3)
    RPTC_MM_ALLOW(1, 4)
    RPTC_MM_ALLOW(2, 4)
#undef RPTC_MM_ALLOW
#define RPTC_MR_ALLOW(TILES)                                                                \
    if ((rc = mm_allow_lds(matmul_rows_kernel<6, RPTC_AS_WRITTEN, TILES>))) return rc;     \
    if ((rc = mm_allow_lds(matmul_rows_kernel<6, RPTC_CONTINUOUS, TILES>))) return rc;     \
    if ((rc = mm_allow_lds(matmul_rows_kernel<8, RPTC_AS_WRITTEN, TILES>))) return rc;     \
    if ((rc = mm_allow_lds(matmul_rows_kernel<8, RPTC_CONTINUOUS, TILES>))) return rc;
    RPTC_MR_ALLOW(1)
    RPTC_MR_ALLOW(2)
    RPTC_MR_ALLOW(3)
#undef RPTC_MR_ALLOW
    // the device addresses of the static scratch arrays (the symbols themselves are not device addresses)
    MmScratch &sc = g_mm[device];
    if ((rc = (int)hipGetSymbolAddress(reinterpret_cast<void **>(&sc.xpack), HIP_SYMBOL(g_xpack)))) return rc;
    if ((rc = (int)hipGetSymbolAddress(reinterpret_cast<void **>(&sc.partial), HIP_SYMBOL(g_partial)))) return rc;
    sc.partial_floats = kMmScratchFloats;
    return (int)hipGetSymbolAddress(reinterpret_cast<void **>(&sc.arrived), HIP_SYMBOL(g_arrived));
}

void matmul_counters(int device, uint32_t **counters, int *count)
{
    *counters = g_mm[device].arrived;
    *count = kMmMaxGroups;
}

// Number of row groups: as many as keep every workgroup of the launch resident at once (two per
// CU), but no group larger than the kernel's register budget allows.
static int mm_groups(int m, int slabs, int cus, int planes, int bits)
{
    const int max_rb = mm_max_row_blocks(planes, bits);
    const int total = (m + 15) / 16;
    int groups = 2 * cus / slabs;
    if (groups < 1) groups = 1;
    if (groups > total) groups = total;
    const int least = (total + max_rb - 1) / max_rb;
    return groups < least ? least : groups;
}

template <int S, int PLANES, int BITS>
static void launch_matmul(const uint32_t *comp, const uint32_t *cb, const MmScratch &sc, uint16_t *out, int m, int n,
                          int batch, int carry_mode, int groups, int slabs, hipStream_t s)
{
    // sc.partial_floats: how many partial-tile floats the scratch holds (the static buffer, or the caller's)
    const int lds_bytes = kMmTableBytes + kMmWaves * 2 * 256 * 4;
    const int total = (m + 15) / 16;
    const int max_rb = (total + groups - 1) / groups;
    // as many row groups per launch as the scratch buffer holds partial tiles for
    int64_t per_launch = sc.partial_floats / ((int64_t)slabs * max_rb * PLANES * 256);
    if (per_launch > kMmMaxGroups) per_launch = kMmMaxGroups;
    for (int g0 = 0; g0 < groups; g0 += (int)per_launch) {
        const int g_n = groups - g0 < per_launch ? groups - g0 : (int)per_launch;
        if (carry_mode == RPTC_AS_WRITTEN)
            hipLaunchKernelGGL((matmul_kernel<S, RPTC_AS_WRITTEN, PLANES, BITS>), dim3(g_n * slabs), dim3(kMmThreads),
                               lds_bytes, s, comp, cb, sc.xpack, m, n, total / groups, total % groups, g0, max_rb,
                               sc.partial, sc.arrived, out, batch);
        else
            hipLaunchKernelGGL((matmul_kernel<S, RPTC_CONTINUOUS, PLANES, BITS>), dim3(g_n * slabs), dim3(kMmThreads),
                               lds_bytes, s, comp, cb, sc.xpack, m, n, total / groups, total % groups, g0, max_rb,
                               sc.partial, sc.arrived, out, batch);
    }
}

template <int S, int BITS>
static void launch_matmul_planes(const uint32_t *comp, const uint32_t *cb, const MmScratch &sc, uint16_t *out, int m,
                                 int n, int batch, int carry_mode, int cus, int slabs, hipStream_t s)
{
    if (batch <= 16) launch_matmul<S, 1, BITS>(comp, cb, sc, out, m, n, batch, carry_mode, mm_groups(m, slabs, cus, 1, BITS), slabs, s);
    else launch_matmul<S, 2, BITS>(comp, cb, sc, out, m, n, batch, carry_mode, mm_groups(m, slabs, cus, 2, BITS), slabs, s);
}

}  // namespace rptc

using namespace rptc;

namespace rptc {

struct MmPlan {
    int planes, slabs, groups, counters;
    int64_t xpack_words, partial_floats;      // what one launch over all row groups needs
};

static int plan_matmul(const void *compressed, const void *codebook, const void *x, const void *out, int64_t m, int64_t n,
                       int64_t batch, int S, int bits, int carry_mode, DeviceInfo **dev, MmPlan *p)
{
    if (!compressed || !codebook || !x || !out) return RPTC_ENULL;
    if (m < 1 || n < 64 || n % 64 != 0 || batch < 1 || (S != 6 && S != 8) || bits < 2 || bits > 4) return RPTC_ESHAPE;
    if (n > kMmMaxN || batch > kMmMaxBatch || m >= (1 << 24)) return RPTC_ELIMIT;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(x)) return RPTC_EALIGN;
    int rc = device_info(dev);
    if (rc) return rc;
    p->planes = batch > 16 ? 2 : 1;
    p->slabs = (int)(n / 2048) + (n % 2048 ? 1 : 0);
    p->groups = mm_groups((int)m, p->slabs, (*dev)->cus, p->planes, bits);
    p->counters = p->groups < kMmMaxGroups ? p->groups : kMmMaxGroups;
    const int total = ((int)m + 15) / 16;
    const int max_rb = (total + p->groups - 1) / p->groups;
    p->xpack_words = (int64_t)p->planes * (n / 2) * 16 + 3 * 512;     // and the padding of a ragged slab in the row-owner form's image
    p->partial_floats = (int64_t)p->groups * p->slabs * max_rb * p->planes * 256;
    return 0;
}

static int run_matmul(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x, uint16_t *out, int64_t m,
                      int64_t n, int64_t batch, int S, int bits, int carry_mode, const MmScratch &sc, const MmPlan &p,
                      DeviceInfo *dev, void *stream, float *ms)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    int rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_comp = reinterpret_cast<const uint32_t *>(compressed);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
#ifdef RPTC_MM_ROWS
    if (bits == 2 && batch <= 16) {
        // the row-owner form: its own packed image (B operands as 16-byte tuples, the ragged slab padded), no counters
        const int threads = (int)(n / 8) * 16 + 3 * 512 / 4;
        hipLaunchKernelGGL(pack_x_tuples_kernel, dim3((threads + 255) / 256), dim3(256), 0, s, reinterpret_cast<const uint4 *>(x), sc.xpack,
                           (int)n, (int)batch);
        if (S == 6 && carry_mode == RPTC_AS_WRITTEN) launch_matmul_rows<6, RPTC_AS_WRITTEN>(a_comp, a_cb, sc.xpack, out, (int)m, (int)n, (int)batch, dev->cus, s);
        if (S == 6 && carry_mode == RPTC_CONTINUOUS) launch_matmul_rows<6, RPTC_CONTINUOUS>(a_comp, a_cb, sc.xpack, out, (int)m, (int)n, (int)batch, dev->cus, s);
        if (S == 8 && carry_mode == RPTC_AS_WRITTEN) launch_matmul_rows<8, RPTC_AS_WRITTEN>(a_comp, a_cb, sc.xpack, out, (int)m, (int)n, (int)batch, dev->cus, s);
        if (S == 8 && carry_mode == RPTC_CONTINUOUS) launch_matmul_rows<8, RPTC_CONTINUOUS>(a_comp, a_cb, sc.xpack, out, (int)m, (int)n, (int)batch, dev->cus, s);
        return t.end();
    }
#endif
    const int total = p.planes * (int)(n / 8) * 16;
    const int pack_threads = total > p.counters ? total : p.counters;
    hipLaunchKernelGGL(pack_x_kernel, dim3((pack_threads + 255) / 256), dim3(256), 0, s, reinterpret_cast<const uint4 *>(x), sc.xpack, sc.arrived,
                       p.counters, (int)n, (int)batch, p.planes);
#define RPTC_MM_GO(SS, BB)                                                                                          \
    if (S == SS && bits == BB)                                                                                       \
        launch_matmul_planes<SS, BB>(a_comp, a_cb, sc, out, (int)m, (int)n, (int)batch, carry_mode, dev->cus, p.slabs, s);
    RPTC_MM_GO(6, 2) RPTC_MM_GO(6, 3) RPTC_MM_GO(6, 4) RPTC_MM_GO(8, 2) RPTC_MM_GO(8, 3) RPTC_MM_GO(8, 4)
#undef RPTC_MM_GO
    return t.end();
}

// layout of a caller's workspace: [packed activations | partial tiles | arrival counters], each 256-byte aligned
static int64_t ws_round(int64_t bytes) { return (bytes + 255) & ~(int64_t)255; }

}  // namespace rptc

extern "C" int rptc_decompress_matmul_bits(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                           uint16_t *out, int64_t m, int64_t n, int64_t batch, int S, int bits,
                                           int carry_mode, void *stream, float *ms)
{
    DeviceInfo *dev;
    MmPlan p;
    int rc = plan_matmul(compressed, codebook, x, out, m, n, batch, S, bits, carry_mode, &dev, &p);
    if (rc) return rc;
    return run_matmul(compressed, codebook, x, out, m, n, batch, S, bits, carry_mode, g_mm[dev->device], p, dev, stream, ms);
}

extern "C" int rptc_decompress_matmul(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                      uint16_t *out, int64_t m, int64_t n, int64_t batch, int S, int carry_mode,
                                      void *stream, float *ms)
{
    return rptc_decompress_matmul_bits(compressed, codebook, x, out, m, n, batch, S, 2, carry_mode, stream, ms);
}

extern "C" int64_t rptc_decompress_matmul_workspace_bytes(int64_t m, int64_t n, int64_t batch, int bits)
{
    if (m < 1 || n < 64 || n % 64 != 0 || batch < 1 || bits < 2 || bits > 4) return RPTC_ESHAPE;
    if (n > kMmMaxN || batch > kMmMaxBatch || m >= (1 << 24)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    MmPlan p;
    const void *any = reinterpret_cast<const void *>(16);      // the plan only tests pointers for NULL and alignment
    int rc = plan_matmul(any, any, any, any, m, n, batch, 8, bits, RPTC_AS_WRITTEN, &dev, &p);
    if (rc) return rc < 0 ? rc : RPTC_EDEVICE;
    return ws_round(p.xpack_words * 4) + ws_round(p.partial_floats * 4) + ws_round((int64_t)p.counters * 4);
}

extern "C" int rptc_decompress_matmul_ws(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                         uint16_t *out, int64_t m, int64_t n, int64_t batch, int S, int bits,
                                         int carry_mode, void *workspace, int64_t workspace_bytes, void *stream,
                                         float *ms)
{
    DeviceInfo *dev;
    MmPlan p;
    int rc = plan_matmul(compressed, codebook, x, out, m, n, batch, S, bits, carry_mode, &dev, &p);
    if (rc) return rc;
    if (!workspace) return RPTC_ENULL;
    if (reinterpret_cast<uintptr_t>(workspace) & 255u) return RPTC_EALIGN;
    const int64_t xb = ws_round(p.xpack_words * 4), pb = ws_round(p.partial_floats * 4), cb = ws_round((int64_t)p.counters * 4);
    if (workspace_bytes < xb + pb + cb) return RPTC_ELIMIT;
    char *base = static_cast<char *>(workspace);
    MmScratch sc;
    sc.xpack = reinterpret_cast<uint32_t *>(base);
    sc.partial = reinterpret_cast<float *>(base + xb);
    sc.arrived = reinterpret_cast<uint32_t *>(base + xb + pb);
    sc.partial_floats = p.partial_floats;
    return run_matmul(compressed, codebook, x, out, m, n, batch, S, bits, carry_mode, sc, p, dev, stream, ms);
}
