// Fused decode + mat-vec on the [slab][row][lane] stream with the hashed pair codebook.
//
// Semantics: rptc_kernels/csrc/rptc_kernels/inference.cu:189-277 (kernel) and :280-356
// (launcher) of the reference.  One stream element (16 bytes, one lane of one row of one slab)
// is 32 steps; step s reads the 16-bit window that ends 4(s+1) bits into the element, hashes
// it with h*(h+1), takes hash byte 1 as the codebook entry (bit 7 of that byte replaces the
// sign of the pair's first value) and multiplies the pair with two activations.
//
// gfx950 design (not the reference's):
//   * one workgroup of 16 waves per CU owns a block of rows and every slab of those rows, so the
//     sum over slabs stays inside the workgroup and is added in a fixed order (deterministic);
//   * a wave item is 64 consecutive stream elements (1 KiB, one coalesced 16-byte load per lane):
//     two rows of a full slab, or floor(64 / Lt) rows of the ragged last slab.  Its address is a
//     wave-uniform base plus 16 bytes per lane, so addressing costs scalar instructions only;
//   * a wave keeps a slab's 32 activation pairs per lane in registers and walks consecutive
//     items of that slab, so activations cost one LDS read per slab change, not one per step;
//   * two adjacent windows come out of one v_alignbit_b32, both hashes out of one
//     v_pk_mad_u16, the LDS address out of one v_and_or_b32 / v_perm_b32 (hash byte 1 is the
//     row of a 256-row table whose sign is already applied, replicated once per lane so the
//     gather has no bank conflicts), and the pair product out of one v_dot2c_f32_f16 with fp32
//     accumulation: about three vector ops per decoded pair, hand-scheduled in decode_asm.hpp;
//   * loads return in issue order, so the small loads that the table and the activation image
//     wait for are issued first and every wave's stream loads right behind them, before the
//     table is built; kernel arguments are preloaded into SGPRs.
#include "decode_asm.hpp"
#include "matvec_loop.hpp"
#include "hadamard_pass.hpp"
#include "rptc_common.hpp"

namespace rptc {

constexpr int kMatvecThreads = 1024;
constexpr int kXRegs = 2048 / kMatvecThreads;   // activation registers per thread: vectors of up to 16384 halves
constexpr int kMatvecWaves = kMatvecThreads / kWave;
constexpr int kTableBytes = 256 * 256;     // 256 rows of 64 lane copies of one half2

struct Geometry {
    int m, n, T, Lt, slabs;
    __host__ __device__ Geometry(int m_, int n_) : m(m_), n(n_), T(n_ >> 11), Lt((n_ & 2047) >> 6), slabs((n_ >> 11) + (((n_ & 2047) >> 6) ? 1 : 0)) {}
    __host__ __device__ int lanes(int slab) const { return slab < T ? 32 : Lt; }
    // index of the uint4 element (slab, row, lane)
    __host__ __device__ size_t elem(int slab, int row, int lane) const
    {
        return slab < T ? ((size_t)slab * m + row) * 32 + lane
                        : (size_t)T * m * 32 + (size_t)row * Lt + lane;
    }
    // half2 slot of step q = 4k + j of lane l (inference.cu:249 for the full slabs)
    __host__ __device__ int slot(int slab, int q, int lane) const
    {
        return slab < T ? 1024 * slab + 32 * q + lane : 1024 * T + q * Lt + lane;
    }
};

// The 256-row table: row b holds entry b & (2^S - 1) with sign bit b >> 7 in the first value.
template <int S>
__device__ __forceinline__ uint32_t table_value(const uint32_t *__restrict__ codebook, int b)
{
    const uint32_t pair = codebook[b & ((1 << S) - 1)];
    return (pair & 0xFFFF7FFFu) | ((uint32_t)(b >> 7) << 15);
}

// A stream element is read exactly once: load it with the non-temporal hint.  The address is a
// wave-uniform base plus 16 bytes per lane, so no vector address arithmetic is needed.
// An element is 2 * BITS words: 4 at 2 bits per weight (the reference format), 6 at 3, 8 at 4.
template <int WORDS>
struct Elem {
    uint32_t w[WORDS];
};

template <int WORDS>
__device__ __forceinline__ Elem<WORDS> load_stream(const uint32_t *wave_base, uint32_t lane)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    Elem<WORDS> e;
    const uint32_t *p = wave_base + lane * WORDS;
    if constexpr (WORDS % 4 == 0) {
#pragma unroll
        for (int i = 0; i < WORDS / 4; i++) {
            const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p) + i);
            e.w[4 * i] = v.x, e.w[4 * i + 1] = v.y, e.w[4 * i + 2] = v.z, e.w[4 * i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < WORDS / 2; i++) {
            const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p) + i);
            e.w[2 * i] = v.x, e.w[2 * i + 1] = v.y;
        }
    }
    return e;
}

// Step s of an element reads slot 4k + j with k = 7, 0, 4, 1, 5, 2, 6, 3 for s / 4 = 0..7, j = s % 4
// (inference.cu:237-250: which of reg_c[0..7] holds the window that ends 4(s+1) bits in).
__host__ __device__ constexpr int slot_of_step(int s)
{
    constexpr int k_of[8] = {7, 0, 4, 1, 5, 2, 6, 3};
    return 4 * k_of[s / 4] + s % 4;
}

// All 32 steps of one element at 3 or 4 bits per weight (a step consumes 2 * BITS stream bits; the
// window is the 16 bits that end 2 * BITS * (s + 1) bits into the element, the previous lane's last
// 16 bits in front).  Plain C++: the shifts are compile-time constants.
template <int BITS>
__device__ __forceinline__ float decode_element_bits(const Elem<2 * BITS> &e, uint32_t carry, uint32_t lane4,
                                                     const uint32_t (&xr)[32])
{
    constexpr int SB = 2 * BITS;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s0 = 0; s0 < 32; s0 += 8) {
        uint32_t wv[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int s = s0 + u;
            const int end = SB * (s + 1), start = end - 16;
            uint32_t h;
            if (start < 0) {
                h = (carry << end) | (e.w[0] >> (32 - end));
            } else {
                const int wi = start >> 5, o = start & 31;
                h = o <= 16 ? e.w[wi] >> (16 - o) : alignbit(e.w[wi], e.w[wi + 1 < 2 * BITS ? wi + 1 : wi], 48 - o);
            }
            // the hash of the low half by a packed 16-bit multiply-add: whatever sits in the high half of h
            // stays there and is cut off by the address mask
            uint32_t prod;                                            // low 16 bits: h * (h + 1)
            asm("v_pk_mad_u16 %0, %1, %1, %1" : "=v"(prod) : "v"(h));
            wv[u] = lds_read_abs(and_or(prod, 0xFF00u, lane4));
        }
#pragma unroll
        for (int u = 0; u < 8; u++) acc[u & 3] = dot2(wv[u], xr[slot_of_step(s0 + u)], acc[u & 3]);
    }
    return (acc[0] + acc[1]) + (acc[2] + acc[3]);
}

// What a wave needs to know about the slab it is working on.  A wave item is 64 consecutive
// stream elements of one slab: rows_per_item whole rows of `lanes` elements each (2 rows of 32
// in a full slab; floor(64 / Lt) rows in the ragged last slab).
struct SlabView {
    int lanes;            // elements per row
    int rows_per_item;
    int items;            // items of this slab in a workgroup
    int part_off;         // where this slab's partial sums start inside a row's run
    uint32_t elem0;       // index of element (slab, row 0 of the matrix, lane 0): m * n / 64 < 2^30 elements
};

struct MatvecArgs {
    int m, n, rows_per_block;
    int rw_tail;          // rows per item in the ragged slab
    int items_full;       // items per full slab per workgroup   = rows_per_block / 2
    int items_tail;       // items of the ragged slab            = ceil(rows_per_block / rw_tail)
    uint32_t full_magic;  // floor(2^32 / items_full) + 1 (0 for items_full = 1): x / items_full = mulhi(x, magic)
};

// Where the activations come from.  Plain: x.  SiluMul: x is [gate | up] (n each) and the
// activations are silu(gate) * up.  AddRmsNorm: r = x (+ x2), activations = r * rsqrt(mean(r^2) +
// eps) * norm_w, and workgroup 0 writes r to x_out: the element-wise step that precedes a
// projection in a decoder layer, done while the stream loads are in flight instead of in a
// kernel of its own.  SignHadamard: activations = H_P (x2 .* x) / sqrt(P) per block of P = 2^log_p
// elements, x2 the +-1 signs: the incoherence transform of hadamard.hip, same passes, same order.
// The fp16 roundings are those of the stand-alone kernels (decode_glue.hip, hadamard.hip).
constexpr int kXPlain = 0, kXSiluMul = 1, kXAddRmsNorm = 2, kXSignHadamard = 3;

struct XFuse {
    const uint4 *x2;       // AddRmsNorm: the residual delta, or null
    const uint4 *norm_w;   // AddRmsNorm: the norm's weight
    uint4 *x_out;          // AddRmsNorm: the updated residual stream (must not alias x or x2)
    float eps;
    int log_p;             // SignHadamard: log2 of the block length
    // AFFINE (the reference's reconstruction W = b_out + b_in + s_out * s_in * W_hat, quantize_hf.py:167):
    // out[r] = s_out[r] * (W_hat (s_in .* a))[r] + b_out[r] * sum(a) + (b_in . a), a = the activations above;
    // any of the four may be null (scale 1, bias 0)
    const uint4 *s_in, *b_in;
    const uint16_t *s_out, *b_out;
};

constexpr int kRedFloats = 48;   // workgroup reductions of the prologues: 16 waves x up to 3 values

struct Halves8 {
    float v[8];
};

__device__ __forceinline__ Halves8 unpack8(const uint4 q)
{
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    Halves8 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        r.v[2 * i] = half_bits_to_float((uint16_t)(w[i] & 0xFFFFu));
        r.v[2 * i + 1] = half_bits_to_float((uint16_t)(w[i] >> 16));
    }
    return r;
}

__device__ __forceinline__ uint4 pack8(const Halves8 &r)
{
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
        w[i] = (uint32_t)float_to_half_bits(r.v[2 * i]) | ((uint32_t)float_to_half_bits(r.v[2 * i + 1]) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

__device__ __forceinline__ float round_half(float v) { return half_bits_to_float(float_to_half_bits(v)); }

// A slab's 32 activation pairs of a lane from LDS: one address (XA) and 32 immediate offsets, 128 bytes (32 slots)
// apart, into XR[0..31].  The reads and their wait are ONE asm statement (a register such a read writes holds
// nothing until the wait; between two statements the compiler may copy or reuse it), and the outputs are
// early-clobber: none may share the address register.
#define RPTC_RELOAD_X32(XR, XA) \
    asm volatile( \
        "ds_read_b32 %0, %32 offset:0\n ds_read_b32 %1, %32 offset:128\n ds_read_b32 %2, %32 offset:256\n" \
        "ds_read_b32 %3, %32 offset:384\n ds_read_b32 %4, %32 offset:512\n ds_read_b32 %5, %32 offset:640\n" \
        "ds_read_b32 %6, %32 offset:768\n ds_read_b32 %7, %32 offset:896\n ds_read_b32 %8, %32 offset:1024\n" \
        "ds_read_b32 %9, %32 offset:1152\n ds_read_b32 %10, %32 offset:1280\n ds_read_b32 %11, %32 offset:1408\n" \
        "ds_read_b32 %12, %32 offset:1536\n ds_read_b32 %13, %32 offset:1664\n ds_read_b32 %14, %32 offset:1792\n" \
        "ds_read_b32 %15, %32 offset:1920\n ds_read_b32 %16, %32 offset:2048\n ds_read_b32 %17, %32 offset:2176\n" \
        "ds_read_b32 %18, %32 offset:2304\n ds_read_b32 %19, %32 offset:2432\n ds_read_b32 %20, %32 offset:2560\n" \
        "ds_read_b32 %21, %32 offset:2688\n ds_read_b32 %22, %32 offset:2816\n ds_read_b32 %23, %32 offset:2944\n" \
        "ds_read_b32 %24, %32 offset:3072\n ds_read_b32 %25, %32 offset:3200\n ds_read_b32 %26, %32 offset:3328\n" \
        "ds_read_b32 %27, %32 offset:3456\n ds_read_b32 %28, %32 offset:3584\n ds_read_b32 %29, %32 offset:3712\n" \
        "ds_read_b32 %30, %32 offset:3840\n ds_read_b32 %31, %32 offset:3968\n s_waitcnt lgkmcnt(0)\n" \
        : "=&v"((XR)[0]), "=&v"((XR)[1]), "=&v"((XR)[2]), "=&v"((XR)[3]), "=&v"((XR)[4]), "=&v"((XR)[5]), "=&v"((XR)[6]), "=&v"((XR)[7]), \
          "=&v"((XR)[8]), "=&v"((XR)[9]), "=&v"((XR)[10]), "=&v"((XR)[11]), "=&v"((XR)[12]), "=&v"((XR)[13]), "=&v"((XR)[14]), \
          "=&v"((XR)[15]), "=&v"((XR)[16]), "=&v"((XR)[17]), "=&v"((XR)[18]), "=&v"((XR)[19]), "=&v"((XR)[20]), "=&v"((XR)[21]), \
          "=&v"((XR)[22]), "=&v"((XR)[23]), "=&v"((XR)[24]), "=&v"((XR)[25]), "=&v"((XR)[26]), "=&v"((XR)[27]), "=&v"((XR)[28]), \
          "=&v"((XR)[29]), "=&v"((XR)[30]), "=&v"((XR)[31]) \
        : "v"(XA) \
        : "memory");

// COMPACT: partial sums per (row, full slab) and (row, ragged lane) instead of per (row, stream element)
template <int S, int MODE, int BITS, int XMODE, bool COMPACT, bool AFFINE = false>
__device__ __forceinline__ void matvec_body(
    const uint32_t *__restrict__ comp, const uint32_t *__restrict__ codebook,
    const uint4 *__restrict__ x, uint16_t *__restrict__ out, const MatvecArgs a, const XFuse fuse)
{
    constexpr int WORDS = 2 * BITS;                        // words per stream element
    // Stream elements a lane asks for at a time: one, and the next one when that one is about to be decoded.
    // The sixteen waves of a CU then have 16 KB on their way at the start and 32 KB in steady state, which is
    // what the memory latency asks for; with two, three or four elements per lane the first data arrives later
    // (the CU's address unit takes the requests one line at a time) and a batch is decoded only when all of
    // it has arrived: measured slower on every shape.
    constexpr int kBatch = 1;
    extern __shared__ uint32_t lds[];
    const int m = a.m, n = a.n;
    const int T = n >> 11, Lt = (n & 2047) >> 6, npr = n >> 6, n8 = n >> 3;
    uint32_t *sx = lds + kTableBytes / 4;                  // activation pairs, slot order
    // Partial sums: [row in block][n / 64], one per stream element of the row.  A long row (large n)
    // would not leave room for a CU's share of rows, so in compact mode the 32 lanes of a full slab
    // are added with DPP first: [row][T full slabs + Lt ragged lanes].
    float *part = reinterpret_cast<float *>(sx + (n >> 1));
    const int pstride = COMPACT ? T + Lt : npr;
    float *red = part + a.rows_per_block * pstride;        // kRedFloats, present when a prologue reduces

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps control flow scalar
    // The table is the first thing in LDS and the kernel has no static LDS, so it starts at LDS
    // address 0 (the low 32 bits of a flat pointer into LDS are the LDS address); OR-ing a row
    // offset into lane4 then equals adding it.
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;
    const int row0 = blockIdx.x * a.rows_per_block;
    const int rows = min(a.rows_per_block, m - row0);

    // Loads are returned in issue order, so the small loads the table and the activation image
    // wait for go first and the stream loads, which take longest, are issued right behind them.
    // Table rows 16 * wave .. 16 * wave + 15 are this wave's to write.  A row is 64 copies of one
    // value, so the value is wave-uniform and comes through the scalar cache: these loads neither
    // queue with the vector loads nor return in order with them.
    // The sign bit of a row is bit 7 of the row number, the same for a wave's sixteen rows: it is merged in
    // by the vector op that moves the value to the register the LDS write takes (v_and_or_b32), so a row
    // costs one vector op and no scalar one in front of the barrier.
    constexpr int kRowsPerWave = 256 / kMatvecWaves;
    uint32_t cbv[kRowsPerWave];
#pragma unroll
    for (int i = 0; i < kRowsPerWave; i++) cbv[i] = codebook[(kRowsPerWave * wave + i) & ((1 << S) - 1)];
    const uint32_t table_sign = (uint32_t)((kRowsPerWave * wave) >> 7) << 15;
    uint4 xv[kXRegs], xv2[kXRegs], xvw[kXRegs];
#pragma unroll
    for (int u = 0; u < kXRegs; u++) {
        const int idx = tid + u * kMatvecThreads;
        if constexpr (XMODE == kXPlain && !AFFINE) {
            xv[u] = x[min(idx, n8 - 1)];                // every lane asks (no masked region); staged only where idx < n8
        } else {
            xv[u] = idx < n8 ? x[idx] : make_uint4(0, 0, 0, 0);
        }
    }
    if constexpr (XMODE == kXSiluMul) {
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const int idx = tid + u * kMatvecThreads;
            xv2[u] = idx < n8 ? x[n8 + idx] : make_uint4(0, 0, 0, 0);
        }
    }
    if constexpr (XMODE == kXSignHadamard) {
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const int idx = tid + u * kMatvecThreads;
            xv2[u] = idx < n8 ? fuse.x2[idx] : make_uint4(0, 0, 0, 0);
        }
    }
    if constexpr (XMODE == kXAddRmsNorm) {
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const int idx = tid + u * kMatvecThreads;
            xv2[u] = (idx < n8 && fuse.x2) ? fuse.x2[idx] : make_uint4(0, 0, 0, 0);
            xvw[u] = idx < n8 ? fuse.norm_w[idx] : make_uint4(0, 0, 0, 0);
        }
    }

    uint4 xsi[kXRegs], xbi[kXRegs];
    uint16_t so_bits = 0x3C00u, bo_bits = 0;                // 1.0, 0.0: lane j holds the values of row wave + 16 j
    if constexpr (AFFINE) {
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const int idx = tid + u * kMatvecThreads;
            xsi[u] = (idx < n8 && fuse.s_in) ? fuse.s_in[idx] : make_uint4(0, 0, 0, 0);
            xbi[u] = (idx < n8 && fuse.b_in) ? fuse.b_in[idx] : make_uint4(0, 0, 0, 0);
        }
        const int my_row = wave + kMatvecWaves * lane;
        if (fuse.s_out && my_row < rows) so_bits = fuse.s_out[row0 + my_row];
        if (fuse.b_out && my_row < rows) bo_bits = fuse.b_out[row0 + my_row];
    }

    // This wave's items: a contiguous piece of [slab 0 items][slab 1 items]...[ragged slab items].
    const int total = T * a.items_full + a.items_tail;
    // Waves w, w+4, w+8, w+12 share a SIMD, and the SIMD issues from the oldest wave that is ready: with equal
    // shares wave w finishes long before wave w+12, and the SIMD ends its work with one wave that cannot
    // keep it busy.  From three items a wave on, the four waves of a SIMD get shares near the proportion
    // they are served in (kCum64 / 64 of the items for waves 0-3, 0-7, 0-11), split evenly inside each group
    // of four, the remainders dealt to the SIMDs in turn so that no SIMD has more than one item above
    // another.  With fewer items the first total % 16 waves take one more than the rest (older waves, again).
    static_assert(kMatvecWaves == 16, "four waves per SIMD");
    constexpr uint32_t kCum64 = 0x382A18u;                    // 24, 42, 56: shares of 24, 18, 14 and 8 of 64
    int it_begin, it_end;
    if (total >= 3 * kMatvecWaves) {
        const uint32_t group = (uint32_t)wave >> 2;
        const uint32_t cum_lo = group == 0 ? 0u : ((uint32_t)total * ((kCum64 >> (8 * group - 8)) & 0xFFu)) >> 6;
        const uint32_t cum_hi = group == 3 ? (uint32_t)total : ((uint32_t)total * ((kCum64 >> (8 * group)) & 0xFFu)) >> 6;
        const uint32_t cnt = cum_hi - cum_lo, per_wave = cnt >> 2, extra = cnt & 3u;
        const uint32_t turn = ((uint32_t)wave - cum_lo) & 3u;
        it_begin = (int)(cum_lo + turn * per_wave + min(turn, extra));
        it_end = it_begin + (int)per_wave + (turn < extra ? 1 : 0);
    } else {
        const int per_wave = (int)((uint32_t)total / kMatvecWaves), extra = (int)((uint32_t)total % kMatvecWaves);
        it_begin = wave * per_wave + min(wave, extra);
        it_end = it_begin + per_wave + (wave < extra ? 1 : 0);
    }
    auto view = [&](int slab) {
        SlabView v;
        const bool full = slab < T;
        v.lanes = full ? 32 : Lt;
        v.rows_per_item = full ? 2 : a.rw_tail;
        v.items = full ? a.items_full : a.items_tail;
        v.part_off = slab * 32;
        v.elem0 = (uint32_t)(full ? slab : T) * (uint32_t)m * 32u;
        return v;
    };
    // it_begin / items_full by a multiplication with the reciprocal the host prepared: exact while
    // it_begin * items_full < 2^32, and both are far smaller
    int first_slab = a.items_full == 1 ? it_begin : (int)__umulhi((uint32_t)it_begin, a.full_magic);
    first_slab = min(first_slab, T);
    const int first_idx = it_begin - first_slab * a.items_full;

    // cursor of the loads and cursor of the decode (slab, item index inside the slab)
    int ld_slab = first_slab, ld_idx = first_idx;
    SlabView ld = view(ld_slab);
    // The registers of the elements in flight.  A lane with nothing to load keeps what it has: such
    // a lane belongs to a row past the block's last one, and nothing it computes is written.
    Elem<WORDS> buf[kBatch];
    uint32_t cw[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; u++) {
#pragma unroll
        for (int i = 0; i < WORDS; i++) buf[u].w[i] = 0;
        cw[u] = 0;
    }
    // requests items base .. base + kBatch - 1 (those the wave has) and moves the load cursor on
    auto load_batch = [&](int base) {
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            if (base + u < it_end) {
                // the cursor stands at the item requested last: moving it on here, not behind the request,
                // keeps that arithmetic out of the instructions in front of the barrier
                if (++ld_idx == ld.items) {
                    ld_idx = 0;
                    ld_slab++;
                    ld = view(ld_slab);
                }
                const int row_first = ld_idx * ld.rows_per_item;           // row inside the block
                const int rows_here = min(ld.rows_per_item, rows - row_first);
                if (lane < rows_here * ld.lanes) {
                    const uint32_t *wave_base = comp + (size_t)(ld.elem0 + (uint32_t)(row0 + row_first) * (uint32_t)ld.lanes) * WORDS;
                    buf[u] = load_stream<WORDS>(wave_base, lane);
                    if (MODE == RPTC_CONTINUOUS && ld_slab > 0) {
                        // the word in front of a row: last word of the row's lane 31 in the slab before
                        const int sub = ld_slab < T ? lane >> 5 : lane / ld.lanes;
                        const int l = lane - sub * ld.lanes;
                        if (l == 0)
                            cw[u] = comp[(((size_t)(ld_slab - 1) * m + row0 + row_first + sub) * 32 + 31) * WORDS + WORDS - 1];
                    }
                }
            }
        }
    };
    // The first batch is requested by every lane of every wave, whatever the wave holds: a request
    // under a condition cannot be counted by the compiler, which then waits for all loads in
    // flight where it needs only the activations, and the staging below (and the element-wise
    // prologues) would start when the stream data has arrived instead of while it is on its way.
    // A lane past the item's rows repeats the last lane's address; a slot past the wave's items
    // repeats the first element of the wave's first item (of the stream for a wave with none).
    auto load_first = [&]() {
        const int row_first = ld_idx * ld.rows_per_item;           // row inside the block
        const int rows_here = min(ld.rows_per_item, rows - row_first);
        // a wave without an item, or whose item lies past the block's last row, asks for the first element of
        // the stream in every lane: one cache line, not eight
        const bool real = it_begin < it_end && rows_here > 0;
        const uint32_t elem = real ? ld.elem0 + (uint32_t)(row0 + row_first) * (uint32_t)ld.lanes : 0u;
        const uint32_t last = real ? (uint32_t)(rows_here * ld.lanes - 1) : 0u;
        buf[0] = load_stream<WORDS>(comp + (size_t)elem * WORDS, min((uint32_t)lane, last));
        if (MODE == RPTC_CONTINUOUS) {
            // the word in front of a row: last word of the row's lane 31 in the slab before
            // (read by all lanes of the row; used by its first lane, and only past slab 0)
            const bool prev = real && ld_slab > 0;
            const int sub = min(ld_slab < T ? lane >> 5 : lane / ld.lanes, max(rows_here, 1) - 1);
            const uint32_t *row_base =
                prev ? comp + (((size_t)(ld_slab - 1) * m + row0 + row_first) * 32 + 31) * WORDS + WORDS - 1 : comp;
            cw[0] = row_base[sub * (prev ? 32 * WORDS : 0)];
        }
    };
    static_assert(kBatch == 1, "the load cursor stands at the one item the first request asked for");
    load_first();

    // the element-wise step in front of the product, on the registers the small loads filled
    if constexpr (XMODE == kXSiluMul) {
#pragma unroll
        for (int u = 0; u < kXRegs; u++) xv[u] = silu_mul8(xv[u], xv2[u]);
    }
    if constexpr (XMODE == kXAddRmsNorm) {
        // host side guarantees n8 <= kXRegs * kMatvecThreads: the whole vector is in registers.
        // Every workgroup does this for the whole vector in front of its barrier, where the instruction count
        // is what costs, so the halves stay packed: the residual add is a packed fp16 add (the sum of two fp16
        // values rounded once: what an fp32 add rounded to fp16 gives as well), the squares are two-term dot
        // products with an fp32 sum, the scaling converts, multiplies and rounds each half once, and the
        // weight is a packed fp16 multiply (an exact product rounded once, as the fp32 product was).
        uint32_t r[kXRegs][4];
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const uint32_t xw[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w}, dw[4] = {xv2[u].x, xv2[u].y, xv2[u].z, xv2[u].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                r[u][i] = fuse.x2 ? __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, xw[i]) + __builtin_bit_cast(half2_t, dw[i]))
                                  : xw[i];                                    // the fp16 residual stream
                ss = dot2(r[u][i], r[u][i], ss);
            }
            const int idx = tid + u * kMatvecThreads;
            if (blockIdx.x == 0 && idx < n8) fuse.x_out[idx] = make_uint4(r[u][0], r[u][1], r[u][2], r[u][3]);
        }
        // sum over the workgroup in a fixed order
        ss = wave_sum(ss);
        if (lane == 63) red[wave] = ss;
        __syncthreads();
        // one value per lane and a sum across the lanes: one LDS round trip instead of sixteen in a row
        float total_ss = wave_sum(lane < kMatvecWaves ? red[lane] : 0.f);
        total_ss = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, total_ss), 63));
        const float inv = rsqrtf(total_ss / (float)n + fuse.eps);
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const uint32_t ww[4] = {xvw[u].x, xvw[u].y, xvw[u].z, xvw[u].w};
            uint32_t h[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const half2_t rv = __builtin_bit_cast(half2_t, r[u][i]);
                half2_t sv;
                sv.x = (_Float16)((float)rv.x * inv);
                sv.y = (_Float16)((float)rv.y * inv);
                h[i] = __builtin_bit_cast(uint32_t, sv * __builtin_bit_cast(half2_t, ww[i]));
            }
            xv[u] = make_uint4(h[0], h[1], h[2], h[3]);
        }
    }

    if constexpr (XMODE == kXSignHadamard) {
        // the signed vector as fp32 behind the partial sums (the host sized LDS for it), the passes of
        // the stand-alone transform over all blocks at once, then back to fp16 in the registers the
        // staging below expects (n8 <= kXRegs * kMatvecThreads is guaranteed by the host)
        float *hb = part + a.rows_per_block * pstride;
        auto signed8 = [&](int idx, const uint4 xq, const uint4 sq) {
            const Halves8 xs = unpack8(xq), ss = unpack8(sq);
#pragma unroll
            for (int k = 0; k < 8; k++) hb[had_pad(8 * idx + k)] = xs.v[k] * ss.v[k];
        };
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const int idx = tid + u * kMatvecThreads;
            if (idx < n8) signed8(idx, xv[u], xv2[u]);
        }
        __syncthreads();
        hadamard_stages<kMatvecThreads>(hb, n, fuse.log_p, tid);
        const float scale = rsqrtf((float)(1 << fuse.log_p));
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const int idx = tid + u * kMatvecThreads;
            Halves8 r;
#pragma unroll
            for (int k = 0; k < 8; k++) r.v[k] = idx < n8 ? hb[had_pad(8 * idx + k)] * scale : 0.f;
            xv[u] = pack8(r);
        }
    }

    float act_sum = 0.f, act_bias = 0.f;                   // sum(a), b_in . a
    if constexpr (AFFINE) {
        // host side guarantees n8 <= kXRegs * kMatvecThreads: the whole vector is in registers
        // two-term dot products for the sums (fp32 inside) and packed fp16 products for the scaling: a
        // product of two fp16 values rounded once to fp16 either way
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            uint32_t v[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};      // zero past the end of the vector
            const uint32_t bi[4] = {xbi[u].x, xbi[u].y, xbi[u].z, xbi[u].w}, si[4] = {xsi[u].x, xsi[u].y, xsi[u].z, xsi[u].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                act_sum = dot2(v[i], 0x3C003C00u, act_sum);            // (1.0, 1.0)
                act_bias = dot2(v[i], bi[i], act_bias);
                if (fuse.s_in)
                    v[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, v[i]) * __builtin_bit_cast(half2_t, si[i]));
            }
            if (fuse.s_in) xv[u] = make_uint4(v[0], v[1], v[2], v[3]);
        }
    }

    // table (256 rows x 64 lane copies) and activation image into LDS
#pragma unroll
    for (int i = 0; i < kRowsPerWave; i++) {
        uint32_t tv;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(tv) : "s"(cbv[i]), "v"(0xFFFF7FFFu), "v"(table_sign));
        lds[(kRowsPerWave * wave + i) * 64 + lane] = tv;
    }
    auto stage_x = [&](int idx, const uint4 v) {          // halves 8idx .. 8idx+7 (inference.cu:215-221)
        sx[idx] = v.x;
        sx[idx + n8] = v.y;
        sx[idx + 2 * n8] = v.z;
        sx[idx + 3 * n8] = v.w;
    };
    {
        // a thread's second register lands 4096 bytes behind its first: four addresses and immediate offsets
        uint32_t *const s0 = sx + tid, *const s1 = s0 + n8, *const s2 = s1 + n8, *const s3 = s2 + n8;
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            if (tid + u * kMatvecThreads < n8) {
                s0[u * kMatvecThreads] = xv[u].x;
                s1[u * kMatvecThreads] = xv[u].y;
                s2[u * kMatvecThreads] = xv[u].z;
                s3[u * kMatvecThreads] = xv[u].w;
            }
        }
    }
    if (n8 > kXRegs * kMatvecThreads) {                   // wave-uniform: short vectors skip the loop's set-up
        for (int idx = tid + kXRegs * kMatvecThreads; idx < n8; idx += kMatvecThreads)
            stage_x(idx, XMODE == kXSiluMul ? silu_mul8(x[idx], x[n8 + idx]) : x[idx]);
    }
    __syncthreads();
    if constexpr (AFFINE) {
        // the two sums are needed when the row sums are written: their reduction runs beside the decode,
        // not in front of the barrier every wave waits at
        act_sum = wave_sum(act_sum);
        act_bias = wave_sum(act_bias);
        if (lane == 63) {
            red[kMatvecWaves + 2 * wave] = act_sum;
            red[kMatvecWaves + 2 * wave + 1] = act_bias;
        }
    }

    uint32_t xr[32];
    int slab = first_slab, idx = first_idx, cur_slab = -1;
    SlabView sv = view(slab);
    int l = 0, sub = 0;                     // this lane's element inside a row, row inside the item
    uint32_t part_lane = 0;                 // LDS byte address of this lane's partial for row 0
    uint64_t first_lanes = 0;               // the lanes with l == 0
    auto decode_batch = [&](const Elem<WORDS> (&cur)[kBatch], const uint32_t (&ccw)[kBatch], int base) {
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            if (base + u >= it_end) break;
            if (slab != cur_slab) {
                cur_slab = slab;
                // lane -> (row inside the item, element inside the row); lanes past the last whole
                // row of a ragged item idle on element 0
                if (slab < T) {
                    sub = lane >> 5;
                    l = lane & 31;
                } else {
                    sub = lane / sv.lanes;
                    l = lane - sub * sv.lanes;
                    if (sub >= sv.rows_per_item) l = 0;
                }
                // step q of element l multiplies pair slot(slab, q, l) (inference.cu:249)
                const uint32_t *xp = sx + (slab < T ? 1024 * slab : 1024 * T) + l;
                if (slab < T) {
                    // One address and 32 immediate offsets (as inline assembly, or the compiler merges these reads with
                    // those of the ragged slab and forms 31 addresses with vector adds).  The reads and their wait are
                    // ONE statement: a register such a read writes holds nothing until the wait, and between two
                    // statements the compiler may copy or reuse it.
                    const uint32_t xa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(xp));
                    RPTC_RELOAD_X32(xr, xa);
                } else {
#pragma unroll
                    for (int q = 0; q < 32; q++) xr[q] = xp[q * sv.lanes];
                }
                first_lanes = __builtin_amdgcn_ballot_w64(l == 0);
                const int col = COMPACT ? (slab < T ? slab : T + l) : sv.part_off + l;
                part_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(part)) + 4u * (uint32_t)(sub * pstride + col);
            }
            const int row_first = idx * sv.rows_per_item;
            // The lanes whose sum is kept, as a wave-uniform mask: the lanes of the item's rows that
            // exist (the first `nact` lanes), and of those only the ones holding a row's sum.
            const int nact = max(min(sv.rows_per_item, rows - row_first), 0) * sv.lanes;   // 0 for an item past the last row
            uint64_t keep = nact >= 64 ? ~0ull : (1ull << nact) - 1ull;
            // Previous lane's last word.  Lane 0 of a row keeps its own as written
            // (inference.cu:232: the shuffle hands lane 0 its own value back).
            const uint32_t last = cur[u].w[WORDS - 1];
            const uint32_t own = MODE == RPTC_CONTINUOUS ? (slab > 0 ? ccw[u] : 0u) : last;
            float sum;
            if constexpr (BITS == 2) {
                float a0, a1, a2, a3;
                decode_element_asm(make_uint4(cur[u].w[0], cur[u].w[1], cur[u].w[2], cur[u].w[3]), own, first_lanes,
                                   lane4, xr, a0, a1, a2, a3);
                sum = (a0 + a1) + (a2 + a3);
            } else if constexpr (BITS == 4) {
                uint32_t xs[32];                        // the activation pairs in stream order of the steps
#pragma unroll
                for (int q = 0; q < 32; q++) xs[q] = xr[slot_of_step(q)];
                float a0, a1, a2, a3;
                decode_element_asm4(cur[u].w, own, first_lanes, lane4, xs, a0, a1, a2, a3);
                sum = (a0 + a1) + (a2 + a3);
            } else {
                uint32_t carry = __builtin_amdgcn_update_dpp(last, last, 0x138 /* wave_shr:1 */, 0xF, 0xF, false);
                if (l == 0) carry = own;
                sum = decode_element_bits<BITS>(cur[u], carry, lane4, xr);
            }
            if (COMPACT && slab < T) {
                sum = half_wave_sum(sum);        // lanes 31 and 63 hold their row's 32 elements
                keep &= 0x8000000080000000ull;
            }
            // (A store under a hand-set execution mask saves the three vector ops of this test, and
            // measured slower on short rows: the compiler cannot schedule around it.)
            if ((keep >> lane) & 1ull) {
                typedef __attribute__((address_space(3))) float lds_float;
                *reinterpret_cast<lds_float *>(static_cast<uintptr_t>(part_lane + 4u * (uint32_t)(row_first * pstride))) = sum;
            }
            if (++idx == sv.items) {
                idx = 0;
                slab++;
                sv = view(slab);
            }
        }
    };
    // One register set is decoded from a copy while its own registers take the next batch.  (Two
    // sets that take turns save the copies and measured 1 % faster on long rows, 1.5 % slower on
    // the short ones this kernel is graded on.)
    if (it_end - it_begin <= kBatch) {
        // everything the wave has is in the first batch: decoded from the registers the requests fill, element
        // by element as each arrives (no copy that would wait for the whole batch)
        decode_batch(buf, cw, it_begin);
    } else
    for (int base = it_begin; base < it_end; base += kBatch) {
        Elem<WORDS> cur[kBatch];
        uint32_t ccw[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            cur[u] = buf[u];
            ccw[u] = cw[u];
        }
        if (base + kBatch < it_end) load_batch(base + kBatch);
        if (total < 3 * kMatvecWaves) {
            // equal shares: a wave that is further along gives way to the ones behind it, so that the four waves of a
            // SIMD advance together instead of oldest first (the skewed shares above are the other answer to the same)
            const int done = base - it_begin;
            if (done == 0) __builtin_amdgcn_s_setprio(3);
            else if (done == 1) __builtin_amdgcn_s_setprio(2);
            else __builtin_amdgcn_s_setprio(1);
        }
        decode_batch(cur, ccw, base);
    }
    __builtin_amdgcn_s_setprio(3);
    __syncthreads();
    if constexpr (AFFINE) {
        // one pair per lane and sums across the lanes; the totals are the same for every lane
        act_sum = wave_sum(lane < kMatvecWaves ? red[kMatvecWaves + 2 * lane] : 0.f);
        act_bias = wave_sum(lane < kMatvecWaves ? red[kMatvecWaves + 2 * lane + 1] : 0.f);
        act_sum = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, act_sum), 63));
        act_bias = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, act_bias), 63));
    }
    // one wave per row: add the row's partial sums in a fixed order
    for (int r = wave, k = 0; r < rows; r += kMatvecWaves, k++) {
        float y = 0.f;
        for (int i = lane; i < pstride; i += kWave) y += part[r * pstride + i];
        y = wave_sum(y);
        if constexpr (AFFINE) {
            const float so = half_bits_to_float((uint16_t)__builtin_amdgcn_readlane((int)so_bits, k & 63));
            const float bo = half_bits_to_float((uint16_t)__builtin_amdgcn_readlane((int)bo_bits, k & 63));
            y = so * y + (bo * act_sum + act_bias);
        }
        if (lane == 63) out[row0 + r] = float_to_half_bits(y);
    }
}

template <int S, int MODE, int BITS, bool COMPACT>
__global__ __launch_bounds__(kMatvecThreads) void matvec_kernel(
    const uint32_t *__restrict__ comp, const uint32_t *__restrict__ codebook,
    const uint4 *__restrict__ x, int arg_m, int arg_n, int arg_rows_per_block,
    int arg_rw_tail, int arg_items_tail, uint32_t arg_full_magic, uint16_t *__restrict__ out)
{
    // Separate scalar arguments (not a struct), and what the first requests need in the first 14 dwords:
    // those arrive in SGPRs with the wave, the rest (the output pointer is needed last) through a scalar load.
    const MatvecArgs a = {arg_m, arg_n, arg_rows_per_block, arg_rw_tail, arg_rows_per_block >> 1, arg_items_tail, arg_full_magic};
    matvec_body<S, MODE, BITS, kXPlain, COMPACT>(comp, codebook, x, out, a, XFuse{nullptr, nullptr, nullptr, 0.f, 0, nullptr, nullptr, nullptr, nullptr});
}

// 2 bits per weight with an element-wise step fused in front (XMODE above)
template <int S, int MODE, int XMODE, bool COMPACT>
__global__ __launch_bounds__(kMatvecThreads) void matvec_fused_kernel(
    const uint32_t *__restrict__ comp, const uint32_t *__restrict__ codebook,
    const uint4 *__restrict__ x, int arg_m, int arg_n, int arg_rows_per_block,
    int arg_rw_tail, int arg_items_tail, uint32_t arg_full_magic, const uint4 *x2, uint16_t *__restrict__ out, const uint4 *norm_w,
    uint4 *x_out, float eps, int log_p)
{
    const MatvecArgs a = {arg_m, arg_n, arg_rows_per_block, arg_rw_tail, arg_rows_per_block >> 1, arg_items_tail, arg_full_magic};
    matvec_body<S, MODE, 2, XMODE, COMPACT>(comp, codebook, x, out, a, XFuse{x2, norm_w, x_out, eps, log_p, nullptr, nullptr, nullptr, nullptr});
}

// 2 bits per weight with the row/column scales and biases of the reference's factorisation applied in
// the prologue (input side) and where the row sums are written (output side), after any XMODE step
template <int S, int MODE, int XMODE>
__global__ __launch_bounds__(kMatvecThreads) void matvec_affine_kernel(
    const uint32_t *__restrict__ comp, const uint32_t *__restrict__ codebook,
    const uint4 *__restrict__ x, int arg_m, int arg_n, int arg_rows_per_block,
    int arg_rw_tail, int arg_items_tail, uint32_t arg_full_magic, const uint4 *x2, uint16_t *__restrict__ out, const uint4 *norm_w,
    uint4 *x_out, float eps, const uint4 *s_in, const uint4 *b_in, const uint16_t *s_out, const uint16_t *b_out)
{
    const MatvecArgs a = {arg_m, arg_n, arg_rows_per_block, arg_rw_tail, arg_rows_per_block >> 1, arg_items_tail, arg_full_magic};
    matvec_body<S, MODE, 2, XMODE, false, true>(comp, codebook, x, out, a, XFuse{x2, norm_w, x_out, eps, 0, s_in, b_in, s_out, b_out});
}

// Dense export: one thread per stream element, 32 pairs scattered to their columns.
// ------------------------------------------------------------------------------------------------------------
// A chain of independent layers in one launch: the body above in a loop over layers (2 bits, plain activations, one
// partial sum per stream element).  What a launch per layer pays every time is paid once or hidden:
//   * the table is written once;
//   * a layer costs ONE workgroup barrier: two activation images and two sets of partial sums take turns, so the
//     barrier that publishes layer k's activations is also the one behind which layer k - 1's rows are added up;
//   * everything layer k + 1 reads from memory -- all of a wave's stream elements (at most MAXI) and a thread's share of
//     the activations -- is requested when layer k's decode starts, into registers of their own: it has a whole layer
//     to arrive, and nothing in the loop ever waits for a request it has just made.
// Layers must not depend on each other (the host checks the addresses): nothing orders a layer's reads behind another
// layer's writes.  Every load is unconditional (clamped addresses), so the compiler counts them exactly.
template <int S, int MODE, int MAXI>
__global__ __launch_bounds__(kMatvecThreads) void matvec_loop_kernel(
    const LoopLayer *__restrict__ layers, const uint32_t *__restrict__ codebook, int count, int xslot_words, int part_floats)
{
    constexpr int WORDS = 4;
    extern __shared__ uint32_t lds[];
    uint32_t *const sx0 = lds + kTableBytes / 4;                                   // two activation images, slot order
    float *const part0 = reinterpret_cast<float *>(sx0 + 2 * xslot_words);         // two sets of [row in block][n / 64]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;   // the table is at LDS address 0

    // The pointers come out of a descriptor in memory, so their address space is stated: global loads and stores,
    // not flat ones.
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef const __attribute__((address_space(1))) uint32_t *global_words;
    typedef const __attribute__((address_space(1))) u32x4 *global_vec4;
    typedef __attribute__((address_space(1))) uint16_t *global_halves;
    typedef const __attribute__((address_space(1))) char *global_bytes;
    // a wave-uniform address plus a 32-bit byte offset of the lane's: the form a global load takes a scalar base for
    auto at = [](const __attribute__((address_space(1))) void *base, uint32_t bytes) {
        return reinterpret_cast<global_bytes>(base) + bytes;
    };
    struct Work {                 // a layer as this wave sees it (all wave-uniform)
        global_words comp;
        global_vec4 x;
        global_halves out;
        int m, T, Lt, npr, n8, rw_tail, items_full, items_tail;
        int row0, rows;           // rows <= 0: no row of this layer is this workgroup's
        int it_begin, it_end, first_slab, first_idx;
    };
    // `like`: the layer in front; a layer of the same shape takes its geometry over and reads the three pointers only
    // (chains of equal layers are the common case, and the set-up is ~200 scalar instructions of every wave)
    auto setup = [&](int k, const Work &like, bool have_like) {
        Work w;
        const LoopLayer d = layers[k];          // the whole descriptor in one request: one wait, not one per branch
        if (have_like && d.same_shape_as_previous) {
            w = like;
            w.comp = reinterpret_cast<global_words>(reinterpret_cast<uintptr_t>(d.comp));
            w.x = reinterpret_cast<global_vec4>(reinterpret_cast<uintptr_t>(d.x));
            w.out = reinterpret_cast<global_halves>(reinterpret_cast<uintptr_t>(d.out));
            return w;
        }
        const int n = d.n, rpb = d.rows_per_block;
        w.comp = reinterpret_cast<global_words>(reinterpret_cast<uintptr_t>(d.comp));
        w.x = reinterpret_cast<global_vec4>(reinterpret_cast<uintptr_t>(d.x));
        w.out = reinterpret_cast<global_halves>(reinterpret_cast<uintptr_t>(d.out));
        w.m = d.m;
        w.T = n >> 11, w.Lt = (n & 2047) >> 6, w.npr = n >> 6, w.n8 = n >> 3;
        w.rw_tail = d.rw_tail, w.items_full = rpb >> 1, w.items_tail = d.items_tail;
        w.row0 = blockIdx.x * rpb;
        w.rows = min(rpb, w.m - w.row0);
        // equal shares: the first total % 16 waves take one element more (at most MAXI each: the host checks)
        const int total = w.rows > 0 ? w.T * w.items_full + w.items_tail : 0;
        const int per_wave = (int)((uint32_t)total / kMatvecWaves), extra = (int)((uint32_t)total % kMatvecWaves);
        w.it_begin = wave * per_wave + min(wave, extra);
        w.it_end = w.it_begin + per_wave + (wave < extra ? 1 : 0);
        int first_slab = w.items_full == 1 ? w.it_begin : (int)__umulhi((uint32_t)w.it_begin, d.full_magic);
        w.first_slab = min(first_slab, w.T);
        w.first_idx = w.it_begin - w.first_slab * w.items_full;
        return w;
    };
    auto view = [&](const Work &w, int slab) {
        SlabView v;
        const bool full = slab < w.T;
        v.lanes = full ? 32 : w.Lt;
        v.rows_per_item = full ? 2 : w.rw_tail;
        v.items = full ? w.items_full : w.items_tail;
        v.part_off = slab * 32;
        v.elem0 = (uint32_t)(full ? slab : w.T) * (uint32_t)w.m * 32u;
        return v;
    };
    // a thread's share of a layer's activations (every lane asks, with a clamped index)
    auto load_x = [&](const Work &w, uint4 (&xv)[kXRegs]) {
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            const u32x4 v = *reinterpret_cast<global_vec4>(at(w.x, 16u * (uint32_t)min(tid + u * kMatvecThreads, w.n8 - 1)));
            xv[u] = make_uint4(v.x, v.y, v.z, v.w);
        }
    };
    // All of the wave's elements of layer w, requested by every lane whatever the wave holds: a lane past the item's
    // rows repeats the last lane's address, and a slot the wave has no item for asks for the first element of the
    // stream in every lane (one cache line).
    auto load_items = [&](const Work &w, Elem<WORDS> (&buf)[MAXI], uint32_t (&cw)[MAXI]) {
        int slab = w.first_slab, idx = w.first_idx;
        SlabView ld = view(w, slab);
#pragma unroll
        for (int u = 0; u < MAXI; u++) {
            const int row_first = idx * ld.rows_per_item;
            const int rows_here = min(ld.rows_per_item, w.rows - row_first);
            const bool mine = w.it_begin + u < w.it_end;
            const bool real = mine && rows_here > 0;          // an item past the block's last row is the wave's, and empty
            const uint32_t elem = real ? ld.elem0 + (uint32_t)(w.row0 + row_first) * (uint32_t)ld.lanes : 0u;
            const uint32_t last = real ? (uint32_t)(rows_here * ld.lanes - 1) : 0u;
            const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<global_vec4>(at(w.comp + (size_t)elem * WORDS, 4u * WORDS * min((uint32_t)lane, last))));
            buf[u].w[0] = v.x, buf[u].w[1] = v.y, buf[u].w[2] = v.z, buf[u].w[3] = v.w;
            if (MODE == RPTC_CONTINUOUS) {
                // the word in front of a row: last word of the row's lane 31 in the slab before (read by all lanes of
                // the row; used by its first lane, and only past slab 0)
                const bool prev = real && slab > 0;
                const int sub = min(slab < w.T ? lane >> 5 : lane / max(ld.lanes, 1), max(rows_here, 1) - 1);
                const global_words row_base =
                    prev ? w.comp + (((size_t)(slab - 1) * w.m + w.row0 + row_first) * 32 + 31) * WORDS + WORDS - 1 : w.comp;
                cw[u] = *reinterpret_cast<global_words>(at(row_base, (uint32_t)sub * (prev ? 4u * 32 * WORDS : 0u)));
            }
            // the cursor moves past every item of the wave's, empty or not, as the decode's does
            if (mine && ++idx == ld.items) {
                idx = 0;
                slab++;
                ld = view(w, slab);
            }
        }
    };

    Work cur = setup(0, Work{}, false), prev = cur, nxt = count > 1 ? setup(1, cur, true) : cur;
    uint4 xv[kXRegs];
    Elem<WORDS> buf[MAXI], nbuf[MAXI];
    uint32_t cw[MAXI], ncw[MAXI];
#pragma unroll
    for (int u = 0; u < MAXI; u++) cw[u] = ncw[u] = 0;
    // requests first (the activations, then the stream), the table behind them
    constexpr int kRowsPerWave = 256 / kMatvecWaves;
    uint32_t cbv[kRowsPerWave];
#pragma unroll
    for (int i = 0; i < kRowsPerWave; i++) cbv[i] = codebook[(kRowsPerWave * wave + i) & ((1 << S) - 1)];
    const uint32_t table_sign = (uint32_t)((kRowsPerWave * wave) >> 7) << 15;
    load_x(cur, xv);
    load_items(cur, nbuf, ncw);
#pragma unroll
    for (int i = 0; i < kRowsPerWave; i++) {
        uint32_t tv;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(tv) : "s"(cbv[i]), "v"(0xFFFF7FFFu), "v"(table_sign));
        lds[(kRowsPerWave * wave + i) * 64 + lane] = tv;
    }
    // a layer's activations into an image (halves 8 idx .. 8 idx + 7 to the four planes, inference.cu:215-221)
    auto stage_x = [&](uint32_t *sx, int n8) {
        uint32_t *const s0 = sx + tid, *const s1 = s0 + n8, *const s2 = s1 + n8, *const s3 = s2 + n8;
#pragma unroll
        for (int u = 0; u < kXRegs; u++) {
            if (tid + u * kMatvecThreads < n8) {
                s0[u * kMatvecThreads] = xv[u].x;
                s1[u * kMatvecThreads] = xv[u].y;
                s2[u * kMatvecThreads] = xv[u].z;
                s3[u * kMatvecThreads] = xv[u].w;
            }
        }
    };
    // One wave per row adds the row's partial sums in a fixed order.  The rows are the older half's: a SIMD serves its
    // oldest wave first, so the waves started first are through with a layer's decode while the younger ones have most
    // of theirs in front of them, and would only wait at the barrier.
    constexpr int kRowWaves = kMatvecWaves / 2;
    auto write_rows = [&](const Work &w, const float *part) {
        if (wave >= kRowWaves) return;
        for (int r = wave; r < w.rows; r += kRowWaves) {
            float y = 0.f;
            for (int i = lane; i < w.npr; i += kWave) y += part[r * w.npr + i];
            y = wave_sum(y);
            if (lane == 63) w.out[w.row0 + r] = float_to_half_bits(y);
        }
    };
    stage_x(sx0, cur.n8);
    // Layer 0's elements change registers here, as every later layer's do at the end of the iteration before: the loop
    // is entered with no request in flight, so the compiler puts no wait for memory in front of a decode.
#pragma unroll
    for (int u = 0; u < MAXI; u++) {
        buf[u] = nbuf[u];
        cw[u] = ncw[u];
    }

    uint32_t xr[32];
#pragma unroll
    for (int q = 0; q < 32; q++) xr[q] = 0;
    // Iteration k, behind the layer's one barrier (layer k's activations are in image k & 1 and every partial sum of
    // layer k - 1 is written): request what layer k + 1 reads, decode layer k from registers filled a layer ago, then
    // the rows of layer k - 1, the activations of layer k + 1 into the other image, the geometry of layer k + 2.
    for (int k = 0; k < count; k++) {
        __syncthreads();
        const bool has_next = k + 1 < count;
        if (has_next) {
            load_x(nxt, xv);
            load_items(nxt, nbuf, ncw);
        }
        const Work w = cur;
        const uint32_t *const sx = sx0 + (k & 1) * xslot_words;
        float *const part = part0 + (k & 1) * part_floats;
        const int pstride = w.npr;
        int slab = w.first_slab, idx = w.first_idx, cur_slab = -1;
        SlabView sv = view(w, slab);
        int l = 0, sub = 0;
        uint32_t part_lane = 0;
        uint64_t first_lanes = 0;
#pragma unroll
        for (int u = 0; u < MAXI; u++) {
            if (w.it_begin + u >= w.it_end) break;
            // A wave that is further along gives way to the ones behind it: left alone, the SIMD serves its oldest wave
            // first and its youngest decodes its last element with nobody to share the vector ALU's idle cycles with.
            if (u == 0) __builtin_amdgcn_s_setprio(3);
            else if (u == 1) __builtin_amdgcn_s_setprio(2);
            else if (u == 2) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(0);
            if (slab != cur_slab) {
                cur_slab = slab;
                if (slab < w.T) {
                    sub = lane >> 5;
                    l = lane & 31;
                } else {
                    sub = lane / sv.lanes;
                    l = lane - sub * sv.lanes;
                    if (sub >= sv.rows_per_item) l = 0;
                }
                // step q of element l multiplies pair slot(slab, q, l) (inference.cu:249): 32 slots, sv.lanes apart
                // (plain LDS reads: the compiler forms the 32 addresses and waits for the data itself)
                const uint32_t *xp = sx + (slab < w.T ? 1024 * slab : 1024 * w.T) + l;
                if (slab < w.T) {
                    // One address and 32 immediate offsets.  The reads and their wait are ONE statement: a register
                    // that such a read writes holds nothing until the wait, and between two statements the compiler
                    // may copy or reuse it.  Early-clobber outputs: none may share the address register.
                    const uint32_t xa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(xp));
                    RPTC_RELOAD_X32(xr, xa);
                } else {
#pragma unroll
                    for (int q = 0; q < 32; q++) xr[q] = xp[q * sv.lanes];
                }
                first_lanes = __builtin_amdgcn_ballot_w64(l == 0);
                part_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(part)) + 4u * (uint32_t)(sub * pstride + sv.part_off + l);
            }
            const int row_first = idx * sv.rows_per_item;
            const int nact = max(min(sv.rows_per_item, w.rows - row_first), 0) * sv.lanes;
            const uint32_t last = buf[u].w[WORDS - 1];
            const uint32_t own = MODE == RPTC_CONTINUOUS ? (slab > 0 ? cw[u] : 0u) : last;
            float a0, a1, a2, a3;
            decode_element_asm(make_uint4(buf[u].w[0], buf[u].w[1], buf[u].w[2], buf[u].w[3]), own, first_lanes, lane4, xr, a0, a1, a2, a3);
            const float sum = (a0 + a1) + (a2 + a3);
            if (lane < nact) {
                typedef __attribute__((address_space(3))) float lds_float;
                *reinterpret_cast<lds_float *>(static_cast<uintptr_t>(part_lane + 4u * (uint32_t)(row_first * pstride))) = sum;
            }
            if (++idx == sv.items) {
                idx = 0;
                slab++;
                sv = view(w, slab);
            }
        }
        __builtin_amdgcn_s_setprio(3);
        if (k > 0) write_rows(prev, part0 + ((k - 1) & 1) * part_floats);
        if (has_next) {
            stage_x(sx0 + ((k + 1) & 1) * xslot_words, nxt.n8);
#pragma unroll
            for (int u = 0; u < MAXI; u++) {
                buf[u] = nbuf[u];
                cw[u] = ncw[u];
            }
        }
        prev = cur;
        cur = nxt;
        if (k + 2 < count) nxt = setup(k + 2, cur, true);
    }
    __syncthreads();
    write_rows(prev, part0 + ((count - 1) & 1) * part_floats);
}

template <int S, int MODE>
__global__ __launch_bounds__(256) void matvec_dense_kernel(
    const uint4 *__restrict__ comp, const uint32_t *__restrict__ codebook, uint32_t *__restrict__ W,
    int m, int n, int slab, int slab_elems)
{
    const Geometry g(m, n);
    const int lanes = g.lanes(slab);
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= slab_elems) return;
    const int row = i / lanes, l = i - row * lanes;
    const uint4 e = comp[g.elem(slab, row, l)];
    uint32_t carry;
    if (l > 0) carry = comp[g.elem(slab, row, l - 1)].w;
    else if (MODE == RPTC_AS_WRITTEN) carry = e.w;
    else carry = slab > 0 ? comp[g.elem(slab - 1, row, 31)].w : 0u;
    const uint32_t reg_c[8] = {e.x, e.y, e.z, e.w,
                               alignbit(e.x, e.y, 16), alignbit(e.y, e.z, 16), alignbit(e.z, e.w, 16),
                               alignbit(carry, e.x, 16)};
    const int n8 = n >> 3;
    uint32_t *wrow = W + (size_t)row * (n >> 1);
#pragma unroll
    for (int k = 0; k < 8; k++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t h = (reg_c[k] >> (12 - 4 * j)) & 0xFFFFu;
            const uint32_t hash = h * (h + 1u);
            const uint32_t pair = codebook[(hash >> 8) & ((1u << S) - 1u)];
            const uint32_t val = (pair & 0xFFFF7FFFu) | (hash & 0x8000u);
            const int P = g.slot(slab, 4 * k + j, l);
            const int ii = P / n8, idx = P - ii * n8;
            wrow[4 * idx + ii] = val;                 // halves 8idx + 2i, 8idx + 2i + 1
        }
    }
}

static int matvec_part_stride(int n, bool compact)
{
    return compact ? (n >> 11) + ((n & 2047) >> 6) : n / 64;
}

static int matvec_lds_bytes(int n, int rows_per_block, bool compact)
{
    return kTableBytes + 2 * n + 4 * matvec_part_stride(n, compact) * rows_per_block;
}

// Argument checks and launch geometry shared by every mat-vec entry point.
static int plan_matvec(const void *compressed, const void *codebook, const void *x, const void *out, int64_t m,
                       int64_t n, int carry_mode, bool allow_compact, int extra_lds_bytes, DeviceInfo **dev,
                       MatvecArgs *a, bool *compact, int *lds_bytes, int *grid)
{
    if (!compressed || !codebook || !x || !out) return RPTC_ENULL;
    if (m < 1 || n < 64 || n % 64 != 0) return RPTC_ESHAPE;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(x)) return RPTC_EALIGN;
    if (m >= (1 << 24) || n >= (1 << 20) || m * n >= ((int64_t)1 << 36)) return RPTC_ELIMIT;
    int rc = device_info(dev);
    if (rc) return rc;
    // one workgroup per CU; when a CU's share of rows with one partial sum per stream element does
    // not fit in LDS beside the table and the activations, the compact partial layout is used where
    // the kernel has one, and if nothing fits, as many rows per workgroup as do
    a->m = (int)m;
    a->n = (int)n;
    a->rows_per_block = 2 * (int)((m + 2 * (*dev)->cus - 1) / (2 * (*dev)->cus));
    *compact = allow_compact && matvec_lds_bytes(a->n, a->rows_per_block, false) + extra_lds_bytes > kMaxLds;
    const int fixed_bytes = matvec_lds_bytes(a->n, 0, *compact) + extra_lds_bytes;
    const int row_bytes = 4 * matvec_part_stride(a->n, *compact);
    if (fixed_bytes + 2 * row_bytes > kMaxLds) return RPTC_ELIMIT;
    const int fit_rows = ((kMaxLds - fixed_bytes) / row_bytes) & ~1;
    if (a->rows_per_block > fit_rows) a->rows_per_block = fit_rows;
    const int lt = (a->n & 2047) >> 6;
    a->rw_tail = lt ? 64 / lt : 1;
    a->items_full = a->rows_per_block / 2;
    a->items_tail = lt ? (a->rows_per_block + a->rw_tail - 1) / a->rw_tail : 0;
    a->full_magic = a->items_full > 1 ? (uint32_t)(((uint64_t)1 << 32) / (uint64_t)a->items_full) + 1u : 0u;
    *lds_bytes = matvec_lds_bytes(a->n, a->rows_per_block, *compact) + extra_lds_bytes;
    *grid = (int)((m + a->rows_per_block - 1) / a->rows_per_block);
    return 0;
}

template <int S, int BITS = 2>
static int launch_matvec(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                         uint16_t *out, int64_t m, int64_t n, int carry_mode, void *stream, float *ms)
{
    DeviceInfo *dev;
    MatvecArgs a;
    int lds_bytes, grid;
    bool compact;
    int rc = plan_matvec(compressed, codebook, x, out, m, n, carry_mode, BITS == 2, 0, &dev, &a, &compact, &lds_bytes, &grid);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_comp = reinterpret_cast<const uint32_t *>(compressed);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    auto a_x = reinterpret_cast<const uint4 *>(x);
#define RPTC_LAUNCH(MODE, COMPACT)                                                                              \
    hipLaunchKernelGGL((matvec_kernel<S, MODE, BITS, COMPACT>), dim3(grid), dim3(kMatvecThreads), lds_bytes, s, \
                       a_comp, a_cb, a_x, a.m, a.n, a.rows_per_block, a.rw_tail, a.items_tail, a.full_magic, out)
    if constexpr (BITS == 2) {
        if (compact) {
            if (carry_mode == RPTC_AS_WRITTEN) RPTC_LAUNCH(RPTC_AS_WRITTEN, true);
            else RPTC_LAUNCH(RPTC_CONTINUOUS, true);
            return t.end();
        }
#ifdef RPTC_MV_ONE
        // the same layer through the chain kernel's hand-written body (an experiment until it is timed)
        if (matvec_one_fits(a.n, a.rows_per_block, a.items_tail)) {
            rc = matvec_one_launch(a_comp, a_cb, a_x, out, a.m, a.n, a.rows_per_block, a.rw_tail, a.items_tail, a.full_magic, grid, S,
                                   carry_mode, 0, nullptr, nullptr, nullptr, 0.f, s);
            return rc ? rc : t.end();
        }
#endif
    }
    if (carry_mode == RPTC_AS_WRITTEN) RPTC_LAUNCH(RPTC_AS_WRITTEN, false);
    else RPTC_LAUNCH(RPTC_CONTINUOUS, false);
#undef RPTC_LAUNCH
    return t.end();
}

template <int S, int XMODE>
static int launch_matvec_fused(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                               const uint16_t *x2, const uint16_t *norm_w, uint16_t *x_out, float eps, int log_p,
                               uint16_t *out, int64_t m, int64_t n, int carry_mode, void *stream, float *ms)
{
    DeviceInfo *dev;
    MatvecArgs a;
    int lds_bytes, grid;
    bool compact;
    // The norm and Hadamard variants hold the whole vector in registers (n <= 16384): never long enough
    // to need compact sums.  The Hadamard variant keeps the vector as padded fp32 behind the partial sums.
    const int extra = XMODE == kXSignHadamard ? (int)(n + n / 32 + 1) * 4 : XMODE == kXAddRmsNorm ? kRedFloats * 4 : 0;
    int rc = plan_matvec(compressed, codebook, x, out, m, n, carry_mode, XMODE == kXSiluMul, extra, &dev, &a, &compact,
                         &lds_bytes, &grid);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_comp = reinterpret_cast<const uint32_t *>(compressed);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    auto a_x = reinterpret_cast<const uint4 *>(x);
    auto a_x2 = reinterpret_cast<const uint4 *>(x2);
    auto a_w = reinterpret_cast<const uint4 *>(norm_w);
    auto a_xo = reinterpret_cast<uint4 *>(x_out);
#define RPTC_LAUNCH(MODE, COMPACT)                                                                                  \
    hipLaunchKernelGGL((matvec_fused_kernel<S, MODE, XMODE, COMPACT>), dim3(grid), dim3(kMatvecThreads), lds_bytes, \
                       s, a_comp, a_cb, a_x, a.m, a.n, a.rows_per_block, a.rw_tail, a.items_tail, a.full_magic, a_x2, out, \
                       a_w, a_xo, eps, log_p)
    if constexpr (XMODE == kXSiluMul) {
        if (compact) {
            if (carry_mode == RPTC_AS_WRITTEN) RPTC_LAUNCH(RPTC_AS_WRITTEN, true);
            else RPTC_LAUNCH(RPTC_CONTINUOUS, true);
            return t.end();
        }
#ifdef RPTC_MV_ONE
        if (matvec_one_fits(a.n, a.rows_per_block, a.items_tail)) {
            rc = matvec_one_launch(a_comp, a_cb, a_x, out, a.m, a.n, a.rows_per_block, a.rw_tail, a.items_tail, a.full_magic, grid, S,
                                   carry_mode, 1, nullptr, nullptr, nullptr, 0.f, s);
            return rc ? rc : t.end();
        }
#endif
    }
#ifdef RPTC_MV_ONE
    if constexpr (XMODE == kXAddRmsNorm) {
        if (matvec_one_fits(a.n, a.rows_per_block, a.items_tail)) {
            rc = matvec_one_launch(a_comp, a_cb, a_x, out, a.m, a.n, a.rows_per_block, a.rw_tail, a.items_tail, a.full_magic, grid, S,
                                   carry_mode, 2, a_x2, a_w, a_xo, eps, s);
            return rc ? rc : t.end();
        }
    }
#endif
    if (carry_mode == RPTC_AS_WRITTEN) RPTC_LAUNCH(RPTC_AS_WRITTEN, false);
    else RPTC_LAUNCH(RPTC_CONTINUOUS, false);
#undef RPTC_LAUNCH
    return t.end();
}

template <int S, int XMODE>
static int launch_matvec_affine(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                const uint16_t *x2, const uint16_t *norm_w, uint16_t *x_out, float eps,
                                const uint16_t *s_in, const uint16_t *b_in, const uint16_t *s_out, const uint16_t *b_out,
                                uint16_t *out, int64_t m, int64_t n, int carry_mode, void *stream, float *ms)
{
    // the whole activation vector sits in two registers per thread
    if (n > 8 * kXRegs * kMatvecThreads) return RPTC_ELIMIT;
    if (!aligned16(s_in) || !aligned16(b_in)) return RPTC_EALIGN;
    DeviceInfo *dev;
    MatvecArgs a;
    int lds_bytes, grid;
    bool compact;
    int rc = plan_matvec(compressed, codebook, x, out, m, n, carry_mode, false, kRedFloats * 4, &dev, &a, &compact,
                         &lds_bytes, &grid);
    if (rc) return rc;
    // lane j of a wave holds the output-side factors of row wave + 16 j of the workgroup's block
    if (a.rows_per_block > kMatvecWaves * kWave) return RPTC_ELIMIT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_comp = reinterpret_cast<const uint32_t *>(compressed);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    auto a_x = reinterpret_cast<const uint4 *>(x);
    auto a_x2 = reinterpret_cast<const uint4 *>(x2);
    auto a_w = reinterpret_cast<const uint4 *>(norm_w);
    auto a_xo = reinterpret_cast<uint4 *>(x_out);
    auto a_si = reinterpret_cast<const uint4 *>(s_in);
    auto a_bi = reinterpret_cast<const uint4 *>(b_in);
#define RPTC_LAUNCH(MODE)                                                                                      \
    hipLaunchKernelGGL((matvec_affine_kernel<S, MODE, XMODE>), dim3(grid), dim3(kMatvecThreads), lds_bytes, s, \
                       a_comp, a_cb, a_x, a.m, a.n, a.rows_per_block, a.rw_tail, a.items_tail, a.full_magic, a_x2, out, \
                       a_w, a_xo, eps, a_si, a_bi, s_out, b_out)
    if (carry_mode == RPTC_AS_WRITTEN) RPTC_LAUNCH(RPTC_AS_WRITTEN);
    else RPTC_LAUNCH(RPTC_CONTINUOUS);
#undef RPTC_LAUNCH
    return t.end();
}

// Dense export at 3 and 4 bits per weight: one thread per stream element.
template <int S, int MODE, int BITS>
__global__ __launch_bounds__(256) void bits_dense_kernel(
    const uint32_t *__restrict__ comp, const uint32_t *__restrict__ codebook, uint32_t *__restrict__ W,
    int m, int n, int slab, int slab_elems)
{
    constexpr int WORDS = 2 * BITS, SB = 2 * BITS;
    const Geometry g(m, n);
    const int lanes = g.lanes(slab);
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= slab_elems) return;
    const int row = i / lanes, l = i - row * lanes;
    const uint32_t *ep = comp + g.elem(slab, row, l) * WORDS;
    uint32_t w[WORDS];
#pragma unroll
    for (int q = 0; q < WORDS; q++) w[q] = ep[q];
    uint32_t carry;
    if (l > 0) carry = ep[-1];
    else if (MODE == RPTC_AS_WRITTEN) carry = w[WORDS - 1];
    else carry = slab > 0 ? comp[g.elem(slab - 1, row, 31) * WORDS + WORDS - 1] : 0u;
    const int n8 = n >> 3;
    uint32_t *wrow = W + (size_t)row * (n >> 1);
#pragma unroll
    for (int s = 0; s < 32; s++) {
        const int end = SB * (s + 1), start = end - 16;
        uint32_t h;
        if (start < 0) {
            h = (carry << end) | (w[0] >> (32 - end));
        } else {
            const int wi = start >> 5, o = start & 31;
            h = o <= 16 ? w[wi] >> (16 - o) : alignbit(w[wi], w[wi + 1 < WORDS ? wi + 1 : wi], 48 - o);
        }
        h &= 0xFFFFu;
        const uint32_t hash = h * (h + 1u);
        const uint32_t pair = codebook[(hash >> 8) & ((1u << S) - 1u)];
        const uint32_t val = (pair & 0xFFFF7FFFu) | (hash & 0x8000u);
        const int P = g.slot(slab, slot_of_step(s), l);
        const int ii = P / n8, idx = P - ii * n8;
        wrow[4 * idx + ii] = val;
    }
}

template <int S, int MODE, int BITS>
static void launch_bits_dense_slabs(const uint32_t *comp, const uint32_t *cb, uint32_t *W, int m, int n, hipStream_t s)
{
    const Geometry g(m, n);
    for (int slab = 0; slab < g.slabs; slab++) {
        const int elems = m * g.lanes(slab);
        hipLaunchKernelGGL((bits_dense_kernel<S, MODE, BITS>), dim3((elems + 255) / 256), dim3(256), 0, s,
                           comp, cb, W, m, n, slab, elems);
    }
}

template <int S, int MODE>
static void launch_dense_slabs(const uint4 *comp, const uint32_t *cb, uint32_t *W, int m, int n, hipStream_t s)
{
    const Geometry g(m, n);
    for (int slab = 0; slab < g.slabs; slab++) {
        const int elems = m * g.lanes(slab);
        hipLaunchKernelGGL((matvec_dense_kernel<S, MODE>), dim3((elems + 255) / 256), dim3(256), 0, s,
                           comp, cb, W, m, n, slab, elems);
    }
}

template <typename F>
static int set_lds_limit(F *kernel)
{
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
}

int prepare_matvec()
{
    int rc;
#define RPTC_SET_LIMITS(BITS, COMPACT)                                                               \
    if ((rc = set_lds_limit(matvec_kernel<6, RPTC_AS_WRITTEN, BITS, COMPACT>))) return rc;              \
    if ((rc = set_lds_limit(matvec_kernel<6, RPTC_CONTINUOUS, BITS, COMPACT>))) return rc;              \
    if ((rc = set_lds_limit(matvec_kernel<8, RPTC_AS_WRITTEN, BITS, COMPACT>))) return rc;              \
    if ((rc = set_lds_limit(matvec_kernel<8, RPTC_CONTINUOUS, BITS, COMPACT>))) return rc;
    RPTC_SET_LIMITS(2, false)
    RPTC_SET_LIMITS(2, true)
    RPTC_SET_LIMITS(3, false)
    RPTC_SET_LIMITS(4, false)
#undef RPTC_SET_LIMITS
#define RPTC_SET_LIMITS(XMODE, COMPACT)                                                                    \
    if ((rc = set_lds_limit(matvec_fused_kernel<6, RPTC_AS_WRITTEN, XMODE, COMPACT>))) return rc;             \
    if ((rc = set_lds_limit(matvec_fused_kernel<6, RPTC_CONTINUOUS, XMODE, COMPACT>))) return rc;             \
    if ((rc = set_lds_limit(matvec_fused_kernel<8, RPTC_AS_WRITTEN, XMODE, COMPACT>))) return rc;             \
    if ((rc = set_lds_limit(matvec_fused_kernel<8, RPTC_CONTINUOUS, XMODE, COMPACT>))) return rc;
    RPTC_SET_LIMITS(kXSiluMul, false)
    RPTC_SET_LIMITS(kXSiluMul, true)
    RPTC_SET_LIMITS(kXAddRmsNorm, false)
    RPTC_SET_LIMITS(kXSignHadamard, false)
#undef RPTC_SET_LIMITS
#define RPTC_SET_LIMITS(XMODE)                                                                     \
    if ((rc = set_lds_limit(matvec_affine_kernel<6, RPTC_AS_WRITTEN, XMODE>))) return rc;             \
    if ((rc = set_lds_limit(matvec_affine_kernel<6, RPTC_CONTINUOUS, XMODE>))) return rc;             \
    if ((rc = set_lds_limit(matvec_affine_kernel<8, RPTC_AS_WRITTEN, XMODE>))) return rc;             \
    if ((rc = set_lds_limit(matvec_affine_kernel<8, RPTC_CONTINUOUS, XMODE>))) return rc;
    RPTC_SET_LIMITS(kXPlain)
    RPTC_SET_LIMITS(kXSiluMul)
    RPTC_SET_LIMITS(kXAddRmsNorm)
#undef RPTC_SET_LIMITS
    return 0;
}

constexpr int kLoopMaxItems = 4;      // stream elements of a layer a wave holds in registers (kernels for 3 and for 4)

int prepare_matvec_loop()
{
    int rc;
#define RPTC_SET_LIMITS(MAXI)                                                                  \
    if ((rc = set_lds_limit(matvec_loop_kernel<6, RPTC_AS_WRITTEN, MAXI>))) return rc;          \
    if ((rc = set_lds_limit(matvec_loop_kernel<6, RPTC_CONTINUOUS, MAXI>))) return rc;          \
    if ((rc = set_lds_limit(matvec_loop_kernel<8, RPTC_AS_WRITTEN, MAXI>))) return rc;          \
    if ((rc = set_lds_limit(matvec_loop_kernel<8, RPTC_CONTINUOUS, MAXI>))) return rc;
    RPTC_SET_LIMITS(3)
    RPTC_SET_LIMITS(4)
#undef RPTC_SET_LIMITS
    return 0;
}

int matvec_loop_plan(const rptc_chain_layer *layers, int64_t count, int cus, LoopLayer *out, int *xslot_words,
                     int *part_floats, int *lds_bytes, int *max_items, int *uniform)
{
    int64_t n_max = 0, part_max = 0, items_max = 1;
    *uniform = 1;
    for (int64_t k = 0; k < count; k++) {
        const rptc_chain_layer &u = layers[k];
        if (u.n > (int64_t)8 * kXRegs * kMatvecThreads) return RPTC_ELIMIT;      // a thread's two registers hold its share
        LoopLayer &d = out[k];
        d = LoopLayer{};
        d.comp = reinterpret_cast<const uint32_t *>(u.compressed);
        d.x = reinterpret_cast<const uint4 *>(u.x);
        d.out = u.out;
        d.m = (int32_t)u.m;
        d.n = (int32_t)u.n;
        d.rows_per_block = 2 * (int32_t)((u.m + 2 * cus - 1) / (2 * cus));
        const int lt = (int)((u.n & 2047) >> 6), items_full = d.rows_per_block / 2;
        d.rw_tail = lt ? 64 / lt : 1;
        d.items_tail = lt ? (d.rows_per_block + d.rw_tail - 1) / d.rw_tail : 0;
        d.full_magic = items_full > 1 ? (uint32_t)(((uint64_t)1 << 32) / (uint64_t)items_full) + 1u : 0u;
        d.same_shape_as_previous = k > 0 && layers[k - 1].m == u.m && layers[k - 1].n == u.n;
        if (k > 0 && !d.same_shape_as_previous) *uniform = 0;
        // a wave keeps all its elements of a layer in registers: at most kLoopMaxItems of them
        const int64_t total = (u.n >> 11) * (int64_t)items_full + d.items_tail;
        const int64_t per_wave = (total + kMatvecWaves - 1) / kMatvecWaves;
        if (per_wave > kLoopMaxItems) return RPTC_ELIMIT;
        if (per_wave > items_max) items_max = per_wave;
        if (u.n > n_max) n_max = u.n;
        const int64_t part = (int64_t)d.rows_per_block * (u.n / 64);
        if (part > part_max) part_max = part;
    }
    const int64_t bytes = kTableBytes + 2 * (2 * n_max) + 2 * 4 * part_max;
    if (bytes > kMaxLds) return RPTC_ELIMIT;
    *xslot_words = (int)(n_max / 2);
    *part_floats = (int)part_max;
    *lds_bytes = (int)bytes;
    *max_items = items_max <= 3 ? 3 : 4;
    return 0;
}

int matvec_loop_launch(const LoopLayer *device_layers, const uint32_t *codebook, int count, int xslot_words,
                       int part_floats, int lds_bytes, int max_items, int grid, int S, int carry_mode, hipStream_t stream)
{
    if (max_items != 3 && max_items != 4) return RPTC_ESHAPE;
#define RPTC_LOOP_GO(SS, MM)                                                                                          \
    do {                                                                                                              \
        if (max_items == 3)                                                                                           \
            hipLaunchKernelGGL((matvec_loop_kernel<SS, MM, 3>), dim3(grid), dim3(kMatvecThreads), lds_bytes, stream,   \
                               device_layers, codebook, count, xslot_words, part_floats);                            \
        else                                                                                                          \
            hipLaunchKernelGGL((matvec_loop_kernel<SS, MM, 4>), dim3(grid), dim3(kMatvecThreads), lds_bytes, stream,   \
                               device_layers, codebook, count, xslot_words, part_floats);                            \
    } while (0)
    if (S == 6 && carry_mode == RPTC_AS_WRITTEN) RPTC_LOOP_GO(6, RPTC_AS_WRITTEN);
    else if (S == 6) RPTC_LOOP_GO(6, RPTC_CONTINUOUS);
    else if (carry_mode == RPTC_AS_WRITTEN) RPTC_LOOP_GO(8, RPTC_AS_WRITTEN);
    else RPTC_LOOP_GO(8, RPTC_CONTINUOUS);
#undef RPTC_LOOP_GO
    return (int)hipGetLastError();
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_decompress_matvec_16_6_1(const int32_t *c, const uint16_t *cb, const uint16_t *x, uint16_t *out,
                                             int64_t m, int64_t n, int mode, void *stream, float *ms)
{
    return launch_matvec<6>(c, cb, x, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_20_6_1(const int32_t *c, const uint16_t *cb, const uint16_t *x, uint16_t *out,
                                             int64_t m, int64_t n, int mode, void *stream, float *ms)
{
    return launch_matvec<6>(c, cb, x, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_16_8_1(const int32_t *c, const uint16_t *cb, const uint16_t *x, uint16_t *out,
                                             int64_t m, int64_t n, int mode, void *stream, float *ms)
{
    return launch_matvec<8>(c, cb, x, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_20_8_1(const int32_t *c, const uint16_t *cb, const uint16_t *x, uint16_t *out,
                                             int64_t m, int64_t n, int mode, void *stream, float *ms)
{
    return launch_matvec<8>(c, cb, x, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_silu(const int32_t *c, const uint16_t *cb, const uint16_t *gate_up, uint16_t *out,
                                           int64_t m, int64_t n, int S, int mode, void *stream, float *ms)
{
    if (S != 6 && S != 8) return RPTC_ESHAPE;
    return S == 6 ? launch_matvec_fused<6, kXSiluMul>(c, cb, gate_up, nullptr, nullptr, nullptr, 0.f, 0, out, m, n, mode, stream, ms)
                  : launch_matvec_fused<8, kXSiluMul>(c, cb, gate_up, nullptr, nullptr, nullptr, 0.f, 0, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_rmsnorm(const int32_t *c, const uint16_t *cb, const uint16_t *x_in,
                                              const uint16_t *delta, const uint16_t *weight, uint16_t *x_out,
                                              uint16_t *out, int64_t m, int64_t n, float eps, int S, int mode,
                                              void *stream, float *ms)
{
    if (!weight || !x_out) return RPTC_ENULL;
    if (S != 6 && S != 8) return RPTC_ESHAPE;
    // every workgroup reads x_in and delta while workgroup 0 writes x_out
    if (x_out == x_in || x_out == delta) return RPTC_EALIAS;
    if (!aligned16(delta) || !aligned16(weight) || !aligned16(x_out)) return RPTC_EALIGN;
    if (n > 8 * kXRegs * kMatvecThreads) return RPTC_ELIMIT;      // the whole vector sits in two registers per thread
    return S == 6 ? launch_matvec_fused<6, kXAddRmsNorm>(c, cb, x_in, delta, weight, x_out, eps, 0, out, m, n, mode, stream, ms)
                  : launch_matvec_fused<8, kXAddRmsNorm>(c, cb, x_in, delta, weight, x_out, eps, 0, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_affine(const int32_t *c, const uint16_t *cb, const uint16_t *x,
                                             const uint16_t *scales_in, const uint16_t *biases_in,
                                             const uint16_t *scales_out, const uint16_t *biases_out, uint16_t *out,
                                             int64_t m, int64_t n, int S, int mode, void *stream, float *ms)
{
    if (S != 6 && S != 8) return RPTC_ESHAPE;
    return S == 6 ? launch_matvec_affine<6, kXPlain>(c, cb, x, nullptr, nullptr, nullptr, 0.f, scales_in, biases_in, scales_out, biases_out, out, m, n, mode, stream, ms)
                  : launch_matvec_affine<8, kXPlain>(c, cb, x, nullptr, nullptr, nullptr, 0.f, scales_in, biases_in, scales_out, biases_out, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_silu_affine(const int32_t *c, const uint16_t *cb, const uint16_t *gate_up,
                                                  const uint16_t *scales_in, const uint16_t *biases_in,
                                                  const uint16_t *scales_out, const uint16_t *biases_out, uint16_t *out,
                                                  int64_t m, int64_t n, int S, int mode, void *stream, float *ms)
{
    if (S != 6 && S != 8) return RPTC_ESHAPE;
    return S == 6 ? launch_matvec_affine<6, kXSiluMul>(c, cb, gate_up, nullptr, nullptr, nullptr, 0.f, scales_in, biases_in, scales_out, biases_out, out, m, n, mode, stream, ms)
                  : launch_matvec_affine<8, kXSiluMul>(c, cb, gate_up, nullptr, nullptr, nullptr, 0.f, scales_in, biases_in, scales_out, biases_out, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_rmsnorm_affine(const int32_t *c, const uint16_t *cb, const uint16_t *x_in,
                                                     const uint16_t *delta, const uint16_t *weight, uint16_t *x_out,
                                                     const uint16_t *scales_in, const uint16_t *biases_in,
                                                     const uint16_t *scales_out, const uint16_t *biases_out,
                                                     uint16_t *out, int64_t m, int64_t n, float eps, int S, int mode,
                                                     void *stream, float *ms)
{
    if (!weight || !x_out) return RPTC_ENULL;
    if (S != 6 && S != 8) return RPTC_ESHAPE;
    if (x_out == x_in || x_out == delta) return RPTC_EALIAS;
    if (!aligned16(delta) || !aligned16(weight) || !aligned16(x_out)) return RPTC_EALIGN;
    return S == 6 ? launch_matvec_affine<6, kXAddRmsNorm>(c, cb, x_in, delta, weight, x_out, eps, scales_in, biases_in, scales_out, biases_out, out, m, n, mode, stream, ms)
                  : launch_matvec_affine<8, kXAddRmsNorm>(c, cb, x_in, delta, weight, x_out, eps, scales_in, biases_in, scales_out, biases_out, out, m, n, mode, stream, ms);
}

extern "C" int rptc_decompress_matvec_hadamard(const int32_t *c, const uint16_t *cb, const uint16_t *x,
                                               const uint16_t *signs, uint16_t *out, int64_t m, int64_t n,
                                               int64_t block, int S, int mode, void *stream, float *ms)
{
    if (!signs) return RPTC_ENULL;
    if (S != 6 && S != 8) return RPTC_ESHAPE;
    if (n < 64 || n % 64 != 0) return RPTC_ESHAPE;
    if (n > 15360) return RPTC_ELIMIT;                       // table + fp16 image + padded fp32 copy must fit in LDS
    int64_t P = block;
    if (P == 0) {                                            // the largest power of two that divides n
        P = 1;
        while (n % (2 * P) == 0) P *= 2;
    }
    if (P < 2 || (P & (P - 1)) != 0 || n % P != 0) return RPTC_ESHAPE;
    if (!aligned16(signs)) return RPTC_EALIGN;
    int log_p = 0;
    while (((int64_t)1 << log_p) < P) log_p++;
    return S == 6 ? launch_matvec_fused<6, kXSignHadamard>(c, cb, x, signs, nullptr, nullptr, 0.f, log_p, out, m, n, mode, stream, ms)
                  : launch_matvec_fused<8, kXSignHadamard>(c, cb, x, signs, nullptr, nullptr, 0.f, log_p, out, m, n, mode, stream, ms);
}

extern "C" int rptc_matvec_dense(const int32_t *compressed, const uint16_t *codebook, uint16_t *W, int64_t m,
                                 int64_t n, int S, int carry_mode, void *stream, float *ms)
{
    if (!compressed || !codebook || !W) return RPTC_ENULL;
    if (m < 1 || n < 64 || n % 64 != 0 || (S != 6 && S != 8)) return RPTC_ESHAPE;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(W)) return RPTC_EALIGN;
    if (m >= (1 << 24) || n >= (1 << 20) || m * 32 >= ((int64_t)1 << 31)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_comp = reinterpret_cast<const uint4 *>(compressed);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    auto a_w = reinterpret_cast<uint32_t *>(W);
    const bool aw = carry_mode == RPTC_AS_WRITTEN;
    if (S == 6 && aw) launch_dense_slabs<6, RPTC_AS_WRITTEN>(a_comp, a_cb, a_w, (int)m, (int)n, s);
    else if (S == 6) launch_dense_slabs<6, RPTC_CONTINUOUS>(a_comp, a_cb, a_w, (int)m, (int)n, s);
    else if (aw) launch_dense_slabs<8, RPTC_AS_WRITTEN>(a_comp, a_cb, a_w, (int)m, (int)n, s);
    else launch_dense_slabs<8, RPTC_CONTINUOUS>(a_comp, a_cb, a_w, (int)m, (int)n, s);
    return t.end();
}

extern "C" int rptc_decompress_matvec_bits(const int32_t *c, const uint16_t *cb, const uint16_t *x, uint16_t *out,
                                           int64_t m, int64_t n, int S, int bits, int mode, void *stream, float *ms)
{
    if ((S != 6 && S != 8) || bits < 2 || bits > 4) return RPTC_ESHAPE;
    if (bits == 2) return S == 6 ? launch_matvec<6, 2>(c, cb, x, out, m, n, mode, stream, ms)
                                 : launch_matvec<8, 2>(c, cb, x, out, m, n, mode, stream, ms);
    if (bits == 3) return S == 6 ? launch_matvec<6, 3>(c, cb, x, out, m, n, mode, stream, ms)
                                 : launch_matvec<8, 3>(c, cb, x, out, m, n, mode, stream, ms);
    return S == 6 ? launch_matvec<6, 4>(c, cb, x, out, m, n, mode, stream, ms)
                  : launch_matvec<8, 4>(c, cb, x, out, m, n, mode, stream, ms);
}

extern "C" int rptc_matvec_bits_dense(const int32_t *compressed, const uint16_t *codebook, uint16_t *W, int64_t m,
                                      int64_t n, int S, int bits, int carry_mode, void *stream, float *ms)
{
    if (bits == 2) return rptc_matvec_dense(compressed, codebook, W, m, n, S, carry_mode, stream, ms);
    if (!compressed || !codebook || !W) return RPTC_ENULL;
    if (m < 1 || n < 64 || n % 64 != 0 || (S != 6 && S != 8) || (bits != 3 && bits != 4)) return RPTC_ESHAPE;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(compressed) || !aligned16(codebook) || !aligned16(W)) return RPTC_EALIGN;
    if (m >= (1 << 24) || n >= (1 << 20) || m * 32 >= ((int64_t)1 << 31)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_comp = reinterpret_cast<const uint32_t *>(compressed);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    auto a_w = reinterpret_cast<uint32_t *>(W);
    const bool aw = carry_mode == RPTC_AS_WRITTEN;
#define RPTC_DENSE(SS, BB)                                                                          \
    if (S == SS && bits == BB) {                                                                    \
        if (aw) launch_bits_dense_slabs<SS, RPTC_AS_WRITTEN, BB>(a_comp, a_cb, a_w, (int)m, (int)n, s); \
        else launch_bits_dense_slabs<SS, RPTC_CONTINUOUS, BB>(a_comp, a_cb, a_w, (int)m, (int)n, s);    \
    }
    RPTC_DENSE(6, 3) RPTC_DENSE(6, 4) RPTC_DENSE(8, 3) RPTC_DENSE(8, 4)
#undef RPTC_DENSE
    return t.end();
}
