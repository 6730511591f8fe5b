// A chain of fused decode + mat-vecs (the op of matvec.hip: rptc_kernels/csrc/rptc_kernels/inference.cu:189-277)
// in ONE launch: layer k of the chain is out_k = W_k x_k on its own stream, activations and output.
//
// Why: a mat-vec of a few megabytes lasts a few microseconds, and a launch per layer spends about half of
// that on things that are not the layer: the dispatch of the grid, the table build and staging in front of
// the first decode, and a tail in which most waves have run out of work.  Here the grid is launched once and
// stays (one 16-wave workgroup per CU), the LDS table is built once, and a wave that has finished its share
// of layer k goes on with layer k + 1 while others still work on k:
//   * stream elements are requested kDepth items ahead of the decode, across layer boundaries (weights never
//     depend on activations, so this also runs ahead of a dependency);
//   * activations are staged in three LDS slots: x_{k+1} is staged when a wave STARTS layer k (its loads were
//     issued a layer earlier), so a fast wave may finish k and enter k + 1 as soon as every wave has started k;
//   * partial sums (one per row and slab) have two LDS buffers; the wave that finishes a layer last in its
//     workgroup adds them in a fixed order and writes the rows.  No workgroup barrier after the prologue:
//     the hand-offs are LDS counters (release / acquire at workgroup scope);
//   * a layer whose activations (or output) overlap an earlier layer's output (or activations) starts behind a
//     grid-wide arrival counter (release / acquire at agent scope): all workgroups have finished everything in
//     front of it.  Every wait, in LDS or in memory, is bounded: a wave that gives up raises an abort flag
//     that ends its workgroup, sets a status word, and every other workgroup then times out the same way, so
//     the kernel always exits.
// The arithmetic per stream element is the mat-vec's (decode_asm.hpp); sums over a row have a fixed order,
// so the output does not depend on which wave came last.
#include <string.h>

#include <vector>

#include "decode_asm.hpp"
#include "rptc_common.hpp"

namespace rptc {

constexpr int kChainThreads = 1024;
constexpr int kChainWaves = kChainThreads / kWave;
constexpr int kChainXRegs = 2;                                    // 16-byte activation registers per thread
constexpr int kChainMaxN = 8 * kChainXRegs * kChainThreads;       // 16384: a thread's share is two registers
constexpr int kChainTableWords = 256 * 64;
constexpr int kChainCtlWords = 16 + 64;                          // control words, then a word per lane for writes that go nowhere
constexpr int kChainSyncBytes = 256;                              // behind the descriptors: grid counter, exit counter, status
constexpr uint64_t kChainMagic = 0x5250544343484E31ull;           // "RPTCCHN1"

// flags of a layer
constexpr int kChLate = 1;       // activations staged when every wave has finished the layer in front (not a layer ahead)
constexpr int kChWaitGrid = 2;   // ... and every workgroup of the grid has (a dependency)
constexpr int kChSignal = 4;     // the workgroup counts its arrival when the layer's rows are written
constexpr int kChFence = 8;      // the rows are released to the device when written (some later layer waits)

struct ChainDesc {               // 64 bytes, device memory, read through the scalar cache
    const uint32_t *comp;
    const uint4 *x;
    uint16_t *out;
    int32_t m, n;
    int32_t rows_per_block;      // even
    int32_t rw_tail;             // rows per item in the ragged slab
    int32_t items_tail;          // items of the ragged slab per workgroup
    uint32_t full_magic;         // floor(2^32 / items_full) + 1 (0 for items_full = 1)
    int32_t flags;
    int32_t wait_signals;        // arrivals every workgroup has counted before this layer (kChWaitGrid)
    int32_t pad[2];
};
static_assert(sizeof(ChainDesc) == 64, "descriptor layout");

// The descriptors do not change while the kernel runs.  Reading them through the constant address space makes
// every read a scalar load (the compiler cannot prove that for a global pointer once the kernel contains
// atomics and hand-written memory instructions, and would use vector loads that its own wait logic then
// serialises with everything in flight).
typedef const __attribute__((address_space(4))) ChainDesc *ChainDescPtr;

// control words in LDS (uint32 each)
constexpr int kCtlXReady = 0;    // [3]: arrivals of the waves that have staged their share of a slot
constexpr int kCtlDone = 4;      // [2]: arrivals of the waves that have finished a layer
constexpr int kCtlAbort = 6;
constexpr int kCtlGrid = 7;      // arrivals per workgroup wave 0 has seen the whole grid reach

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// Waits until *word >= target; false when the abort flag is up or the spin limit is reached.
__device__ __forceinline__ bool lds_wait_ge(uint32_t *word, uint32_t target, uint32_t *abort_word, uint32_t spin_limit)
{
    for (uint32_t spin = 0;; spin++) {
        const uint32_t v = uniform(__hip_atomic_load(word, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP));
        if (v >= target) return true;
        const uint32_t ab = uniform(__hip_atomic_load(abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
        if (ab != 0u || spin >= spin_limit) return false;
        __builtin_amdgcn_s_sleep(1);
    }
}

// one arrival of this wave at an LDS counter (lane 0 adds); returns the count before it, the same in every lane
__device__ __forceinline__ uint32_t lds_arrive(uint32_t *word, int lane)
{
    uint32_t prev = 0;
    if (lane == 0) prev = __hip_atomic_fetch_add(word, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
    return uniform(prev);
}

// The items of one wave in one layer, walked in order: [slab 0 items][slab 1 items]...[ragged slab items] of the
// workgroup's rows, a contiguous share per wave.  All fields are wave-uniform.
struct ChainCursor {
    int layer, count;
    int it, it_end;              // position in the workgroup's items of the layer, end of this wave's share
    int slab, idx;               // slab, and item inside the slab
    // the layer
    const uint32_t *comp;
    int m, T, Lt, rows, row0, rw_tail, items_full, items_tail;

    __device__ __forceinline__ int lanes() const { return slab < T ? 32 : Lt; }
    __device__ __forceinline__ int rows_per_item() const { return slab < T ? 2 : rw_tail; }
    __device__ __forceinline__ int items() const { return slab < T ? items_full : items_tail; }

    // Positions the cursor on the wave's first item of layer l; false when the wave has none there.
    __device__ __forceinline__ bool enter(ChainDescPtr desc, int l, int wave, int block)
    {
        layer = l;
        const auto &d = desc[l];
        comp = d.comp;
        m = d.m;
        const int n = d.n;
        T = n >> 11;
        Lt = (n & 2047) >> 6;
        row0 = block * d.rows_per_block;
        rows = min(d.rows_per_block, m - row0);
        rw_tail = d.rw_tail;
        items_full = d.rows_per_block >> 1;
        items_tail = d.items_tail;
        if (rows <= 0) {
            it = it_end = 0;
            return false;
        }
        // equal shares; the waves that take one item more change from layer to layer
        const int total = T * items_full + items_tail;
        const int v = (wave + l) & (kChainWaves - 1);
        const int per_wave = (int)((uint32_t)total / kChainWaves), extra = (int)((uint32_t)total % kChainWaves);
        it = v * per_wave + min(v, extra);
        it_end = it + per_wave + (v < extra ? 1 : 0);
        int first_slab = items_full == 1 ? it : (int)__umulhi((uint32_t)it, d.full_magic);
        first_slab = min(first_slab, T);
        slab = first_slab;
        idx = it - first_slab * items_full;
        return it < it_end;
    }

    // the next item of the wave, in this layer or a later one; false at the end of the chain
    __device__ __forceinline__ bool next(ChainDescPtr desc, int wave, int block)
    {
        if (++it < it_end) {
            if (++idx == items()) {
                idx = 0;
                slab++;
            }
            return true;
        }
        for (int l = layer + 1; l < count; l++)
            if (enter(desc, l, wave, block)) return true;
        layer = count;
        return false;
    }

    __device__ __forceinline__ int row_first() const { return idx * rows_per_item(); }
    __device__ __forceinline__ int rows_here() const { return max(min(rows_per_item(), rows - row_first()), 0); }
};

typedef uint32_t chain_u32x4 __attribute__((ext_vector_type(4)));
// Pointers that come out of a descriptor are generic to the compiler, and loads through them would be flat
// instructions (counted with the LDS operations as well as with the memory operations): say they are global.
typedef const __attribute__((address_space(1))) chain_u32x4 *global_u32x4_ptr;
typedef const __attribute__((address_space(1))) uint32_t *global_u32_ptr;
typedef __attribute__((address_space(1))) uint16_t *global_u16_out_ptr;
template <typename G, typename P>
__device__ __forceinline__ G as_global(P *p)
{
    return reinterpret_cast<G>(reinterpret_cast<uintptr_t>(p));
}

// The stream and the look-ahead activation loads are issued and waited for by hand: with requests in flight
// across layer changes the compiler falls back to waiting for every outstanding load before each use, which
// would hold a decode until the request issued one item earlier has arrived.  Loads return in issue order, so
// "at most N outstanding" (s_waitcnt vmcnt(N)) means everything but the N youngest has arrived; whatever else
// is in flight at that moment (stores of finished rows, loads the compiler issued) only makes the wait stricter.
__device__ __forceinline__ void issue_load_b128(chain_u32x4 &dst, const void *uniform_base, uint32_t byte_offset)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(dst) : "v"(byte_offset), "s"(uniform_base) : "memory");
}
__device__ __forceinline__ void issue_load_b128_cached(chain_u32x4 &dst, const void *uniform_base, uint32_t byte_offset)
{
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(byte_offset), "s"(uniform_base) : "memory");
}
__device__ __forceinline__ void issue_load_b32(uint32_t &dst, const void *uniform_base, uint32_t byte_offset)
{
    asm volatile("global_load_dword %0, %1, %2" : "=v"(dst) : "v"(byte_offset), "s"(uniform_base) : "memory");
}
// Registers with a load in flight must not be read by anything but a block that waits first: the compiler does
// not know about the load and is free to copy such a register (for an in/out operand it does, in front of the
// block).  So a hand-issued load is either waited for in the same block that issues it (load_now_b128), or its
// registers are input-only operands of a block that starts with the wait (decode_element_asm<N>, stage_after_wait).
__device__ __forceinline__ void load_now_b128(chain_u32x4 &d0, chain_u32x4 &d1, const void *uniform_base, uint32_t off0, uint32_t off1)
{
    asm volatile("global_load_dwordx4 %0, %2, %4\n\tglobal_load_dwordx4 %1, %3, %4\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(d0), "=&v"(d1) : "v"(off0), "v"(off1), "s"(uniform_base) : "memory");
}
// waits until at most N loads are outstanding, then writes the four words of v to the LDS byte addresses a0..a3
template <int N>
__device__ __forceinline__ void stage_after_wait(const chain_u32x4 &v, uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3)
{
    asm volatile("s_waitcnt vmcnt(%8)\n\tds_write_b32 %4, %0\n\tds_write_b32 %5, %1\n\tds_write_b32 %6, %2\n\tds_write_b32 %7, %3"
                 :: "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w), "v"(a0), "v"(a1), "v"(a2), "v"(a3), "n"(N) : "memory");
}

template <int S, int MODE, int DEPTH>
__global__ __launch_bounds__(kChainThreads) void matvec_chain_kernel(
    const ChainDesc *__restrict__ desc_global, const uint32_t *__restrict__ codebook, int count, int nb, int xslot_words,
    int part_floats, uint32_t arrivals, uint32_t spin_limit, uint32_t *__restrict__ sync, int uses_grid)
{
    extern __shared__ uint32_t lds[];
    const ChainDescPtr desc = reinterpret_cast<ChainDescPtr>(reinterpret_cast<uintptr_t>(desc_global));
    uint32_t *ctl = lds + kChainTableWords;
    uint32_t *xbuf = ctl + kChainCtlWords;
    float *part = reinterpret_cast<float *>(xbuf + nb * xslot_words);     // [2][part_floats]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int block = blockIdx.x;
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 4;   // the table starts at LDS address 0

    // ---------------------------------------------------------------- prologue: table and control words
    constexpr int kRowsPerWave = 256 / kChainWaves;
    uint32_t cbv[kRowsPerWave];
#pragma unroll
    for (int i = 0; i < kRowsPerWave; i++) cbv[i] = codebook[(kRowsPerWave * wave + i) & ((1 << S) - 1)];
    const uint32_t table_sign = (uint32_t)((kRowsPerWave * wave) >> 7) << 15;
    if (tid < kChainCtlWords) ctl[tid] = 0u;
#pragma unroll
    for (int i = 0; i < kRowsPerWave; i++) {
        uint32_t tv;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(tv) : "s"(cbv[i]), "v"(0xFFFF7FFFu), "v"(table_sign));
        lds[(kRowsPerWave * wave + i) * 64 + lane] = tv;
    }
    __syncthreads();                       // the only workgroup barrier: table and control words are in place

    uint32_t *const abort_word = ctl + kCtlAbort;
    bool failed = false;
    auto give_up = [&]() {
        // this wave stops; its workgroup follows through the abort flag, the other workgroups through their own
        // bounded waits, and the status word tells the host
        if (lane == 0) {
            __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __hip_atomic_store(&sync[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        failed = true;
    };

    // ---------------------------------------------------------------- stream requests
    // The load cursor runs DEPTH items ahead of the decode.  Each ring position has ONE place in the code that
    // issues its load and ONE that decodes it (a block that waits first): registers with a load in flight then
    // have one definition and one use, and the compiler has no reason to copy them.
    ChainCursor lc;
    lc.count = count;
    lc.layer = -1;
    lc.it = lc.it_end = 0;
    bool lc_live = lc.next(desc, wave, block);
    constexpr int kLoadsPerRequest = MODE == RPTC_CONTINUOUS ? 2 : 1;
    int loads_since_x = 0;                 // stream loads issued after the look-ahead activation loads
    auto request = [&](chain_u32x4 &dst, uint32_t &cw) {
        // Every lane of every wave asks, whatever is left: a lane past the item's rows repeats the item's last
        // element, a request past the end of the chain the chain's first element (the counting of loads in
        // flight relies on one request per decoded item).
        const int rh = lc_live ? lc.rows_here() : 0;
        const bool real = rh > 0;
        const int ln = lc.lanes();
        const uint32_t elem0 = (uint32_t)(lc.slab < lc.T ? lc.slab : lc.T) * (uint32_t)lc.m * 32u;
        const uint32_t elem = real ? elem0 + (uint32_t)(lc.row0 + lc.row_first()) * (uint32_t)ln : 0u;
        const uint32_t last = real ? (uint32_t)(rh * ln - 1) : 0u;
        const uint32_t *base = (real ? lc.comp : desc[0].comp) + (size_t)elem * 4;
        issue_load_b128(dst, base, min((uint32_t)lane, last) * 16u);
        if (MODE == RPTC_CONTINUOUS) {
            // the word in front of a row: last word of the row's lane 31 in the slab before (read by all lanes
            // of the row; used by its first lane).  In slab 0 the word is zero: read from a word of the sync
            // area that always is, so that nothing outside the decode block has to look at the register.
            const bool prev = real && lc.slab > 0;
            const int sub = min(lc.slab < lc.T ? lane >> 5 : lane / max(ln, 1), max(rh, 1) - 1);
            const uint32_t *row_base =
                prev ? lc.comp + (((size_t)(lc.slab - 1) * lc.m + lc.row0 + lc.row_first()) * 32 + 31) * 4 + 3 : sync + 3;
            issue_load_b32(cw, row_base, (uint32_t)(sub * (prev ? 512 : 0)));
        }
        loads_since_x += kLoadsPerRequest;
        if (lc_live) lc_live = lc.next(desc, wave, block);
    };

    // ---------------------------------------------------------------- activations
    // a thread's share of a layer's activations: 16-byte pieces tid and tid + 1024 (n <= 16384)
    chain_u32x4 xe[kChainXRegs];           // the share of the layer after next, on its way while this layer is decoded
    // loaded and waited for in one block (a layer behind a dependency, and the first two layers)
    auto load_x = [&](const auto &d, chain_u32x4 (&dst)[kChainXRegs]) {
        const int n8 = d.n >> 3;
        static_assert(kChainXRegs == 2, "two registers per thread");
        load_now_b128(dst[0], dst[1], d.x, (uint32_t)min(tid, n8 - 1) * 16u, (uint32_t)min(tid + kChainThreads, n8 - 1) * 16u);
    };
    auto stage_x = [&](const auto &d, int slot, const chain_u32x4 (&src)[kChainXRegs]) {
        // halves 8 idx .. 8 idx + 7 go to the four planes of the slot order (inference.cu:215-221)
        const int n8 = d.n >> 3;
        uint32_t *sx = xbuf + slot * xslot_words;
#pragma unroll
        for (int u = 0; u < kChainXRegs; u++) {
            const int idx = tid + u * kChainThreads;
            if (idx < n8) {
                sx[idx] = src[u].x;
                sx[idx + n8] = src[u].y;
                sx[idx + 2 * n8] = src[u].z;
                sx[idx + 3 * n8] = src[u].w;
            }
        }
    };
    // the look-ahead share: requested here ...
    auto load_x_ahead = [&](const auto &d) {
        const int n8 = d.n >> 3;
#pragma unroll
        for (int u = 0; u < kChainXRegs; u++) issue_load_b128_cached(xe[u], d.x, (uint32_t)min(tid + u * kChainThreads, n8 - 1) * 16u);
        loads_since_x = 0;
    };
    // ... and staged a layer later by blocks that wait first: for everything but the stream loads issued since
    // (all loads when fewer than a ring's worth were issued).  A lane with nothing to stage writes to a word of
    // its own that nobody reads.
    auto stage_x_ahead = [&](const auto &d, int slot) {
        constexpr int kRing = DEPTH * kLoadsPerRequest;
        const int n8 = d.n >> 3;
        const uint32_t sx = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(xbuf + slot * xslot_words));
        const uint32_t dump = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(ctl + 16)) + 4u * (uint32_t)lane;
#pragma unroll
        for (int u = 0; u < kChainXRegs; u++) {
            const int idx = tid + u * kChainThreads;
            const bool live = idx < n8;
            const uint32_t a0 = live ? sx + 4u * (uint32_t)idx : dump;
            const uint32_t a1 = live ? a0 + 4u * (uint32_t)n8 : dump, a2 = live ? a1 + 4u * (uint32_t)n8 : dump,
                           a3 = live ? a2 + 4u * (uint32_t)n8 : dump;
            if (loads_since_x >= kRing) stage_after_wait<kRing>(xe[u], a0, a1, a2, a3);
            else stage_after_wait<0>(xe[u], a0, a1, a2, a3);
        }
    };
    auto slot_of = [&](int l) { return nb == 3 ? l % 3 : 0; };
    auto xready_target = [&](int l) { return (uint32_t)kChainWaves * (uint32_t)((nb == 3 ? l / 3 : l) + 1); };
    auto early = [&](int l) { return l < count && !(desc[l].flags & kChLate); };

    // ---------------------------------------------------------------- per-layer protocol
    // Start of layer l for this wave: its activations are complete in their slot; the next layer's share is staged.
    auto start_layer = [&](int l) {
        const auto &d = desc[l];
        const bool late = l == 0 || (d.flags & kChLate);
        if (late) {
            if (l > 0) {
                // every wave of the workgroup has finished the layer in front (and so has stopped reading the slot)
                if (!lds_wait_ge(ctl + kCtlDone + ((l - 1) & 1), (uint32_t)kChainWaves * (uint32_t)(((l - 1) >> 1) + 1), abort_word, spin_limit)) {
                    give_up();
                    return;
                }
            }
            if (l > 0 && (d.flags & kChWaitGrid)) {
                const uint32_t need = (uint32_t)d.wait_signals;
                if (wave == 0) {
                    bool ok = false;
                    for (uint32_t spin = 0; spin < spin_limit; spin++) {
                        // a device-coherent load of the counter (by hand, like every load of this kernel)
                        uint32_t seen;
                        asm volatile("global_load_dword %0, %1, %2 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(seen) : "v"(0u), "s"(sync) : "memory");
                        if (uniform(seen) >= need * arrivals) {
                            ok = true;
                            break;
                        }
                        if (uniform(__hip_atomic_load(abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) != 0u) break;
                        __builtin_amdgcn_s_sleep(2);
                    }
                    if (!ok) {
                        give_up();
                        return;
                    }
                    if (lane == 0) __hip_atomic_store(ctl + kCtlGrid, need, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
                } else if (!lds_wait_ge(ctl + kCtlGrid, need, abort_word, spin_limit)) {
                    give_up();
                    return;
                }
                // what the other workgroups wrote is visible to the loads below
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            }
            chain_u32x4 xl[kChainXRegs];
            load_x(d, xl);
            stage_x(d, slot_of(l), xl);
            lds_arrive(ctl + kCtlXReady + slot_of(l), lane);
        }
        if (!lds_wait_ge(ctl + kCtlXReady + slot_of(l), xready_target(l), abort_word, spin_limit)) {
            give_up();
            return;
        }
        // Every wave has finished layer l - 2, so the slot of layer l + 1 is free: stage it now, before this layer
        // is decoded, so that a wave that finishes this layer early finds it complete.  (Its loads went out when
        // the layer in front was started; for layer 1 there was none: loaded here.)
        if (early(l + 1)) {
            if (l == 0) {
                chain_u32x4 x1[kChainXRegs];
                load_x(desc[1], x1);
                stage_x(desc[1], slot_of(1), x1);
            } else {
                stage_x_ahead(desc[l + 1], slot_of(l + 1));
            }
            lds_arrive(ctl + kCtlXReady + slot_of(l + 1), lane);
        }
        if (early(l + 2)) load_x_ahead(desc[l + 2]);
    };

    // End of layer l for this wave; the wave that arrives last adds the partial sums and writes the rows.
    bool wrote_last_layer = false;
    auto finish_layer = [&](int l) {
        const auto &d = desc[l];
        const uint32_t prev = lds_arrive(ctl + kCtlDone + (l & 1), lane);
        if (prev + 1u != (uint32_t)kChainWaves * (uint32_t)((l >> 1) + 1)) return;
        wrote_last_layer = l == count - 1;
        const int row0 = block * d.rows_per_block;
        const int rows = min(d.rows_per_block, d.m - row0);
        const int pstride = (d.n >> 11) + ((d.n & 2047) >> 6);
        const float *pl = part + (l & 1) * part_floats;
        // four lanes per row: each adds every fourth partial in rising order, then the four are added
        for (int r = lane >> 2; r < rows; r += 16) {
            float s = 0.f;
            for (int i = lane & 3; i < pstride; i += 4) s += pl[r * pstride + i];
            s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(uint32_t, s), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
            s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(uint32_t, s), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
            if ((lane & 3) == 0) as_global<global_u16_out_ptr>(d.out)[row0 + r] = float_to_half_bits(s);
        }
        if (d.flags & kChFence) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        if ((d.flags & kChSignal) && lane == 0) __hip_atomic_fetch_add(&sync[0], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    };

    // ---------------------------------------------------------------- the decode
    ChainCursor dc;
    dc.count = count;
    dc.layer = -1;
    dc.it = dc.it_end = 0;
    bool dc_live = dc.next(desc, wave, block);
    int cur_layer = -1;                     // the layer this wave has started and not yet finished

    uint32_t xr[32];
    int xr_layer = -1, xr_slab = -1;
    int l = 0, sub = 0;
    uint32_t part_lane = 0;
    uint64_t first_lanes = 0;
    int pstride = 0;
    int primed = 0;                         // ring positions that hold a request

    // one ring position: its item is decoded (once the ring is primed), then its registers take the item DEPTH ahead
    auto step = [&](chain_u32x4 &e_reg, uint32_t &cw_reg) {
        if (primed >= DEPTH) {
            if (dc.layer != xr_layer || dc.slab != xr_slab) {
                xr_layer = dc.layer;
                xr_slab = dc.slab;
                const int ln = dc.lanes();
                if (dc.slab < dc.T) {
                    sub = lane >> 5;
                    l = lane & 31;
                } else {
                    sub = lane / ln;
                    l = lane - sub * ln;
                    if (sub >= dc.rw_tail) l = 0;
                }
                const uint32_t *xp = xbuf + slot_of(dc.layer) * xslot_words + (dc.slab < dc.T ? 1024 * dc.slab : 1024 * dc.T) + l;
                if (dc.slab < dc.T) {
                    const uint32_t xa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(xp));
#pragma unroll
                    for (int q = 0; q < 32; q++)
                        asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(xr[q]) : "v"(xa), "n"(128 * q));
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                } else {
#pragma unroll
                    for (int q = 0; q < 32; q++) xr[q] = xp[q * ln];
                }
                first_lanes = __builtin_amdgcn_ballot_w64(l == 0);
                pstride = dc.T + dc.Lt;
                const int col = dc.slab < dc.T ? dc.slab : dc.T + l;
                part_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(part + (dc.layer & 1) * part_floats)) +
                            4u * (uint32_t)(sub * pstride + col);
            }
            const int row_first = dc.row_first();
            const int nact = dc.rows_here() * dc.lanes();
            uint64_t keep = nact >= 64 ? ~0ull : (1ull << nact) - 1ull;
            // the block waits for this element (and its carry word) itself: everything but the requests issued after it
            float a0, a1, a2, a3;
            decode_element_asm<(DEPTH - 1) * kLoadsPerRequest>(e_reg, MODE == RPTC_CONTINUOUS ? cw_reg : e_reg.w, first_lanes, lane4,
                                                               xr, a0, a1, a2, a3);
            float sum = (a0 + a1) + (a2 + a3);
            if (dc.slab < dc.T) {
                sum = half_wave_sum(sum);           // lanes 31 and 63 hold their row's 32 elements
                keep &= 0x8000000080000000ull;
            }
            if ((keep >> lane) & 1ull) {
                typedef __attribute__((address_space(3))) float lds_float;
                *reinterpret_cast<lds_float *>(static_cast<uintptr_t>(part_lane + 4u * (uint32_t)(row_first * pstride))) = sum;
            }
            dc_live = dc.next(desc, wave, block);
        } else {
            primed++;
        }
        // the registers are free: the item DEPTH ahead takes them
        request(e_reg, cw_reg);
    };

    chain_u32x4 ring[DEPTH];
    uint32_t ring_cw[DEPTH];
    static_assert(DEPTH >= 1 && DEPTH <= 4, "ring positions are spelled out below");
    int pos = 0;
    while (true) {
        // Layer changes happen here and nowhere else (one place in the code): the wave finishes and starts every
        // layer between the one it is in and the one its next item belongs to, also those in which it has nothing
        // to decode; at the end of the chain it finishes the last one.
        // (Not before the ring holds its first requests: those go out in front of everything else.)
        if (primed >= DEPTH) {
            const int target = dc_live ? dc.layer : count;
            while (cur_layer < target) {
                if (cur_layer >= 0) finish_layer(cur_layer);
                cur_layer++;
                if (cur_layer < count) {
                    start_layer(cur_layer);
                    if (failed) break;
                }
            }
            if (failed || !dc_live) break;
        }
        // ring positions in turn, until the next item belongs to another layer (or there is none)
        if (pos == 0) {
            step(ring[0], ring_cw[0]);
            pos = DEPTH > 1 ? 1 : 0;
            if (primed >= DEPTH && (!dc_live || dc.layer != cur_layer)) continue;
        }
        if constexpr (DEPTH > 1) {
            if (pos == 1) {
                step(ring[1], ring_cw[1]);
                pos = DEPTH > 2 ? 2 : 0;
                if (primed >= DEPTH && (!dc_live || dc.layer != cur_layer)) continue;
            }
        }
        if constexpr (DEPTH > 2) {
            if (pos == 2) {
                step(ring[2], ring_cw[2]);
                pos = DEPTH > 3 ? 3 : 0;
                if (primed >= DEPTH && (!dc_live || dc.layer != cur_layer)) continue;
            }
        }
        if constexpr (DEPTH > 3) {
            if (pos == 3) {
                step(ring[3], ring_cw[3]);
                pos = 0;
            }
        }
    }
    // the ring's last requests are still in flight: they must have landed before the registers are given up
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // After the chain's last layer: the workgroup that leaves last puts the grid counters back for the next launch
    // (nobody waits on them any more).
    if (!failed && wrote_last_layer && uses_grid) {
        uint32_t left = 0;
        if (lane == 0) left = __hip_atomic_fetch_add(&sync[1], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if (uniform(left) + 1u == arrivals && lane == 0) {
            __hip_atomic_store(&sync[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&sync[1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------------------------- host side

struct ChainPlanHost {            // what rptc_chain_t holds (see the header): written by rptc_chain_plan
    uint64_t magic;
    void *device_desc;
    int32_t count, grid, lds_bytes, nb, xslot_words, part_floats, uses_grid;
    uint32_t arrivals, spin_limit;
    int32_t device;
    int32_t reserved[3];
};
static_assert(sizeof(ChainPlanHost) <= sizeof(rptc_chain_t), "the public struct holds the plan");

static bool overlaps(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes)
{
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + (uintptr_t)b_bytes && b0 < a0 + (uintptr_t)a_bytes;
}

template <typename K>
static int chain_allow_lds(K kernel)
{
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
}

constexpr int kChainDepth = 3;

int prepare_matvec_chain()
{
    int rc;
    if ((rc = chain_allow_lds(matvec_chain_kernel<6, RPTC_AS_WRITTEN, kChainDepth>))) return rc;
    if ((rc = chain_allow_lds(matvec_chain_kernel<6, RPTC_CONTINUOUS, kChainDepth>))) return rc;
    if ((rc = chain_allow_lds(matvec_chain_kernel<8, RPTC_AS_WRITTEN, kChainDepth>))) return rc;
    return chain_allow_lds(matvec_chain_kernel<8, RPTC_CONTINUOUS, kChainDepth>);
}

}  // namespace rptc

using namespace rptc;

extern "C" int64_t rptc_chain_desc_bytes(int64_t count)
{
    if (count < 1 || count > (1 << 20)) return RPTC_ESHAPE;
    return count * (int64_t)sizeof(ChainDesc) + kChainSyncBytes;
}

extern "C" int rptc_chain_plan(const rptc_chain_layer *layers, int64_t count, void *device_desc, int64_t device_desc_bytes,
                               rptc_chain_t *plan, void *stream)
{
    if (!layers || !device_desc || !plan) return RPTC_ENULL;
    if (count < 1 || count > (1 << 20)) return RPTC_ESHAPE;
    if (device_desc_bytes < rptc_chain_desc_bytes(count)) return RPTC_ELIMIT;
    if (reinterpret_cast<uintptr_t>(device_desc) & 255u) return RPTC_EALIGN;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    const int grid = dev->cus;
    std::vector<ChainDesc> descs((size_t)count + kChainSyncBytes / sizeof(ChainDesc));
    memset(descs.data(), 0, descs.size() * sizeof(ChainDesc));
    int n_max = 0, part_max = 0;
    for (int64_t k = 0; k < count; k++) {
        const rptc_chain_layer &u = layers[k];
        if (!u.compressed || !u.x || !u.out) return RPTC_ENULL;
        if (u.m < 1 || u.n < 64 || u.n % 64 != 0) return RPTC_ESHAPE;
        if (u.n > kChainMaxN || u.m >= (1 << 24) || u.m * u.n >= ((int64_t)1 << 36)) return RPTC_ELIMIT;
        if (!aligned16(u.compressed) || !aligned16(u.x)) return RPTC_EALIGN;
        ChainDesc &d = descs[(size_t)k];
        d.comp = reinterpret_cast<const uint32_t *>(u.compressed);
        d.x = reinterpret_cast<const uint4 *>(u.x);
        d.out = u.out;
        d.m = (int)u.m;
        d.n = (int)u.n;
        d.rows_per_block = 2 * (int)((u.m + 2 * grid - 1) / (2 * grid));
        const int lt = (d.n & 2047) >> 6;
        d.rw_tail = lt ? 64 / lt : 1;
        const int items_full = d.rows_per_block / 2;
        d.items_tail = lt ? (d.rows_per_block + d.rw_tail - 1) / d.rw_tail : 0;
        d.full_magic = items_full > 1 ? (uint32_t)(((uint64_t)1 << 32) / (uint64_t)items_full) + 1u : 0u;
        const int pstride = (d.n >> 11) + lt;
        if (d.n > n_max) n_max = d.n;
        if (d.rows_per_block * pstride > part_max) part_max = d.rows_per_block * pstride;
    }
    // LDS: table, control words, the activation slots (three when they fit, so that waves can run a layer ahead;
    // else one), two buffers of partial sums
    const int xslot_words = n_max / 2;
    const int fixed = (kChainTableWords + kChainCtlWords) * 4 + 2 * part_max * 4;
    int nb = 3;
    if (fixed + 3 * xslot_words * 4 > kMaxLds) nb = 1;
    if (fixed + nb * xslot_words * 4 > kMaxLds) return RPTC_ELIMIT;
    // Hazards: a layer starts behind the grid-wide counter when its activations overlap an earlier output (read
    // after write), or its output overlaps earlier activations or outputs (write after read / write).  Everything
    // in front of a counter-guarded layer is complete when that layer starts, so "earlier" need not reach past one.
    // The loads of a layer that is not behind the counter go out two layers ahead, so for such a layer "earlier"
    // reaches back to the last counter-guarded layer at or before k - 2.
    std::vector<int64_t> barrier_at_or_before((size_t)count, 0);      // last guarded layer <= k (0: the start)
    int signals = 0;
    bool any = false;
    for (int64_t k = 1; k < count; k++) {
        const rptc_chain_layer &a = layers[k];
        const int64_t from = barrier_at_or_before[(size_t)(k >= 2 ? k - 2 : 0)];
        bool dep = false;
        for (int64_t j = from; j < k && !dep; j++) {
            const rptc_chain_layer &b = layers[j];
            dep = overlaps(a.x, 2 * a.n, b.out, 2 * b.m) || overlaps(a.out, 2 * a.m, b.x, 2 * b.n) ||
                  overlaps(a.out, 2 * a.m, b.out, 2 * b.m);
        }
        barrier_at_or_before[(size_t)k] = dep ? k : barrier_at_or_before[(size_t)k - 1];
        if (dep) {
            descs[(size_t)k - 1].flags |= kChSignal;
            signals++;
            descs[(size_t)k].flags |= kChLate | kChWaitGrid;
            descs[(size_t)k].wait_signals = signals;
            any = true;
        } else if (nb == 1) {
            descs[(size_t)k].flags |= kChLate;
        }
    }
    if (any)
        for (int64_t k = 0; k < count; k++) descs[(size_t)k].flags |= kChFence;
    // the sync words behind the descriptors start at zero
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((rc = (int)hipMemcpyAsync(device_desc, descs.data(), (size_t)rptc_chain_desc_bytes(count), hipMemcpyHostToDevice, s))) return rc;
    if ((rc = (int)hipStreamSynchronize(s))) return rc;
    ChainPlanHost p;
    memset(&p, 0, sizeof(p));
    p.magic = kChainMagic;
    p.device_desc = device_desc;
    p.count = (int)count;
    p.grid = grid;
    p.nb = nb;
    p.xslot_words = xslot_words;
    p.part_floats = part_max;
    p.lds_bytes = fixed + nb * xslot_words * 4;
    p.uses_grid = any ? 1 : 0;
    p.arrivals = (uint32_t)grid;
    p.spin_limit = 1u << 22;
    p.device = dev->device;
    memset(plan, 0, sizeof(*plan));
    memcpy(plan, &p, sizeof(p));
    return 0;
}

extern "C" int rptc_decompress_matvec_chain(const rptc_chain_t *plan, const uint16_t *codebook, int S, int carry_mode,
                                            void *stream, float *ms)
{
    if (!plan || !codebook) return RPTC_ENULL;
    ChainPlanHost p;
    memcpy(&p, plan, sizeof(p));
    if (p.magic != kChainMagic || !p.device_desc || p.count < 1) return RPTC_ESHAPE;
    if (S != 6 && S != 8) return RPTC_ESHAPE;
    if (carry_mode != RPTC_AS_WRITTEN && carry_mode != RPTC_CONTINUOUS) return RPTC_EMODE;
    if (!aligned16(codebook)) return RPTC_EALIGN;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    if (dev->device != p.device || p.grid != dev->cus || p.lds_bytes > kMaxLds) return RPTC_EDEVICE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    rc = t.begin(dev, s, ms);
    if (rc) return rc;
    auto a_desc = reinterpret_cast<const ChainDesc *>(p.device_desc);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    auto a_sync = reinterpret_cast<uint32_t *>(static_cast<char *>(p.device_desc) + (size_t)p.count * sizeof(ChainDesc));
#define RPTC_CHAIN_GO(SS, MM)                                                                                              \
    hipLaunchKernelGGL((matvec_chain_kernel<SS, MM, kChainDepth>), dim3(p.grid), dim3(kChainThreads), p.lds_bytes, s, a_desc, \
                       a_cb, p.count, p.nb, p.xslot_words, p.part_floats, p.arrivals, p.spin_limit, a_sync, p.uses_grid)
    if (S == 6 && carry_mode == RPTC_AS_WRITTEN) RPTC_CHAIN_GO(6, RPTC_AS_WRITTEN);
    else if (S == 6) RPTC_CHAIN_GO(6, RPTC_CONTINUOUS);
    else if (carry_mode == RPTC_AS_WRITTEN) RPTC_CHAIN_GO(8, RPTC_AS_WRITTEN);
    else RPTC_CHAIN_GO(8, RPTC_CONTINUOUS);
#undef RPTC_CHAIN_GO
    return t.end();
}

extern "C" int rptc_chain_status(const rptc_chain_t *plan, int *status, void *stream)
{
    if (!plan || !status) return RPTC_ENULL;
    ChainPlanHost p;
    memcpy(&p, plan, sizeof(p));
    if (p.magic != kChainMagic || !p.device_desc || p.count < 1) return RPTC_ESHAPE;
    uint32_t words[3] = {0, 0, 0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const char *sync = static_cast<const char *>(p.device_desc) + (size_t)p.count * sizeof(ChainDesc);
    int rc = (int)hipMemcpyAsync(words, sync, sizeof(words), hipMemcpyDeviceToHost, s);
    if (rc) return rc;
    if ((rc = (int)hipStreamSynchronize(s))) return rc;
    *status = (words[2] != 0u ? 1 : 0) | (words[0] != 0u || words[1] != 0u ? 2 : 0);
    return 0;
}
