// A chain of fused decode + mat-vecs (the op of matvec.hip: rptc_kernels/csrc/rptc_kernels/inference.cu:189-277)
// in ONE launch: layer k of the chain is out_k = W_k x_k on its own stream, activations and output.
//
// Why: a mat-vec of a few megabytes lasts a few microseconds, and a launch per layer spends about half of
// that on things that are not the layer: the dispatch of the grid, the table build and staging in front of
// the first decode, and a tail in which most waves have run out of work.  Here the grid is launched once and
// stays (one 16-wave workgroup per CU), the LDS table is built once, and the waves of a workgroup have two jobs:
//   * fifteen DECODE waves do nothing but stream and decode.  A wave walks its share of a layer's stream elements
//     item by item (an item = 64 consecutive elements, as in the mat-vec), requests them kChainDepth items ahead of
//     the decode, across layer boundaries (weights never depend on activations, so this also runs ahead of a
//     dependency), and leaves one partial sum per row and slab in LDS.  Its loads are issued and waited for by
//     hand, and nothing else of the wave uses memory, so "all but the newest kChainDepth - 1 requests have
//     arrived" is exact.  When it has finished its share of layer k it goes on with layer k + 1 while others still
//     work on k; it may enter a layer once that layer's activations are staged and the partial sums of the layer
//     before last have been added up (one LDS counter, `go`, tells both);
//   * one SERVICE wave does everything else, one layer after the other: it stages a layer's activations in one of
//     three LDS slots (two layers ahead of the decode, unless the layer waits for another one's output), adds a
//     finished layer's partial sums in a fixed order, writes the rows, and counts the workgroup's arrival at the
//     grid-wide counter behind which dependent layers start.
// No workgroup barrier after the prologue: the hand-offs are LDS counters (release / acquire at workgroup scope).
// A layer whose activations (or output) overlap an earlier layer's output (or activations) starts behind a
// grid-wide arrival counter: all workgroups have finished everything in front of it.  Every wait, in LDS or in
// memory, is bounded: a wave that gives up raises an abort flag that ends its workgroup and sets a status word,
// and every other workgroup then runs out of patience the same way, so the kernel always exits.
// The arithmetic per stream element is the mat-vec's (decode_asm.hpp); sums over a row have a fixed order, so
// the output does not depend on timing.
#include <string.h>

#include <vector>

#include "decode_asm.hpp"
#include "matvec_loop.hpp"
#include "rptc_common.hpp"

namespace rptc {

constexpr int kChainThreads = 1024;
constexpr int kChainWaves = kChainThreads / kWave;
constexpr int kChainDecodeWaves = kChainWaves - 1;                // wave 15 is the service wave
constexpr int kChainMaxN = 16384;
constexpr int kChainTableWords = 256 * 64;
constexpr int kChainCtlWords = 16;
constexpr int kChainSyncBytes = 256;                              // behind the descriptors: grid counter, exit counter, status, a zero
constexpr uint64_t kChainMagic = 0x5250544343484E32ull;           // "RPTCCHN2"

// flags of a layer
constexpr int kChLate = 1;       // activations staged when the layer in front has been written (not two layers ahead)
constexpr int kChWaitGrid = 2;   // ... and every workgroup of the grid has written it (a dependency)
constexpr int kChSignal = 4;     // the workgroup counts its arrival when the layer's rows are written
constexpr int kChFence = 8;      // the rows are written through to device-coherent memory (some layer depends on another)

struct ChainDesc {               // 64 bytes, device memory, read through the scalar cache
    const uint32_t *comp;
    const uint32_t *x;
    uint16_t *out;
    const uint32_t *items;       // the item table of the layer's shape (ChainTable)
    int32_t m, n;
    int32_t rows_per_block;      // even
    int32_t rw_tail;             // rows per item in the ragged slab
    int32_t flags;
    int32_t wait_signals;        // arrivals every workgroup has counted before this layer (kChWaitGrid)
    int32_t pad[2];
};
static_assert(sizeof(ChainDesc) == 64, "descriptor layout");

// The descriptors do not change while the kernel runs.  Reading them through the constant address space makes
// every read a scalar load (the compiler cannot prove that for a global pointer once the kernel contains
// atomics and hand-written memory instructions).
typedef const __attribute__((address_space(4))) ChainDesc *ChainDescPtr;

// control words in LDS (uint32 each)
constexpr int kCtlGo = 0;        // layers below this number may be entered by the decode waves
constexpr int kCtlDone = 2;      // [2]: arrivals of the decode waves that have finished a layer (even / odd layers)
constexpr int kCtlAbort = 4;

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
// by value (a min that returns a reference to one of two struct fields makes the compiler keep both in memory)
__device__ __forceinline__ int imin(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ uint32_t umin(uint32_t a, uint32_t b) { return a < b ? a : b; }

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

typedef uint32_t chain_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) uint16_t *global_u16_out_ptr;
typedef const __attribute__((address_space(1))) chain_u32x4 *global_u32x4_ptr;
template <typename G, typename P>
__device__ __forceinline__ G as_global(P *p)
{
    return reinterpret_cast<G>(reinterpret_cast<uintptr_t>(p));
}

// The stream loads are issued and waited for by hand.  With requests in flight across layer changes the compiler
// falls back to waiting for every outstanding load before each use, which would hold a decode until the request
// issued one item earlier has arrived.  Loads return in issue order, so "at most N outstanding" (s_waitcnt
// vmcnt(N)) means everything but the N youngest has arrived.
// Registers with a load in flight must not be read by anything but a block that comes behind such a wait: the
// compiler does not know about the load and is free to copy such a register when it has two definitions to merge
// or an in/out operand to tie.  So every ring position has ONE place in the code that issues its load and ONE
// that decodes it, and the registers are input-only operands there.
__device__ __forceinline__ void issue_load_b128(chain_u32x4 &dst, const void *uniform_base, uint32_t byte_offset)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(dst) : "v"(byte_offset), "s"(uniform_base) : "memory");
}
__device__ __forceinline__ void issue_load_b32(uint32_t &dst, const void *uniform_base, uint32_t byte_offset)
{
    asm volatile("global_load_dword %0, %1, %2" : "=v"(dst) : "v"(byte_offset), "s"(uniform_base) : "memory");
}

// ---------------------------------------------------------------------------------------------- decode waves

// The items of a workgroup in a layer of a given shape (m, n), in the order [slab 0 items][slab 1 items] ... [ragged slab
// items], are the same for every workgroup but for the rows it starts at, so the host writes them down once per shape:
// the index arithmetic of the walk is then a table read and a handful of scalar operations per item.
//   ChainTable: begin[16] (the share of decode wave w is items begin[w] .. begin[w + 1] - 1; begin[15] = all), then
//   one ChainItem per item.
// Waves w, w + 4, w + 8, w + 12 share a SIMD, and the SIMD of the service wave has three decode waves where the others
// have four: a wave there takes 4 units of work, the others 3 (48 units in all), so that every SIMD decodes a quarter
// of the items.
struct ChainItem {               // 16 bytes
    uint32_t offset;             // byte offset of the item's first element in the stream of a workgroup whose rows start at 0
    uint32_t row_first;          // the item's first row inside the workgroup's block
    uint32_t geom;               // slab | rows per item << 8 | elements per row << 16
    uint32_t poff;               // byte offset of the item's first partial sum: 4 * row_first * (partial sums per row)
};
constexpr int kChainTableHeaderWords = 16;
typedef const __attribute__((address_space(4))) uint32_t *ChainTablePtr;
typedef uint32_t chain_table_u32x4 __attribute__((ext_vector_type(4)));

// Where the next item to REQUEST is (all fields wave-uniform).
struct ChainWalker {
    int layer, count;
    int it, it_end;              // position in the layer's item table, end of this wave's share
    ChainTablePtr items;         // the layer's table
    const uint32_t *comp;        // the layer's stream
    uint32_t row0x16;            // 16 * first row of the workgroup's block
    int rows;                    // rows of the block that exist
    uint32_t parity_off;         // byte offset of the layer's partial-sum buffer

    // positions the walker on the wave's first item of the first layer >= l in which it has one; false: none left
    __device__ __forceinline__ bool enter(ChainDescPtr desc, int l, int wave, int block, int part_floats)
    {
#pragma clang loop vectorize(disable) interleave(disable) unroll(disable)
        for (; l < count; l++) {
            const auto &d = desc[l];
            const int row0 = block * d.rows_per_block;
            rows = d.m - row0 < d.rows_per_block ? d.m - row0 : d.rows_per_block;
            if (rows <= 0) continue;
            items = reinterpret_cast<ChainTablePtr>(reinterpret_cast<uintptr_t>(d.items));
            it = (int)items[wave];
            it_end = (int)items[wave + 1];
            if (it >= it_end) continue;
            layer = l;
            comp = d.comp;
            row0x16 = (uint32_t)row0 * 16u;
            parity_off = 4u * (uint32_t)((l & 1) * part_floats);
            return true;
        }
        layer = count;
        return false;
    }
};

// what the decode is told about an item: layer, slab and number of live lanes in one word, the byte offset of the
// item's first partial sum inside the partial-sum area in the other
constexpr uint32_t kItemEnd = 0xFFFFFFFFu;

template <int S, int MODE, int DEPTH>
__device__ __forceinline__ void chain_decode_wave(ChainDescPtr desc, int count, uint32_t *ctl, const uint32_t *xbuf, int nb,
                                                  int xslot_words, float *part, int part_floats, uint32_t spin_limit,
                                                  uint32_t *sync, int wave, int lane, int block, uint32_t lane4)
{
    constexpr int kLoadsPerRequest = MODE == RPTC_CONTINUOUS ? 2 : 1;
    uint32_t *const abort_word = ctl + kCtlAbort;
    ChainWalker wk;
    wk.count = count;
    bool live = wk.enter(desc, 0, wave, block, part_floats);
    auto request = [&](chain_u32x4 &dst, uint32_t &cw, uint32_t &info, uint32_t &poff) {
        // Every lane asks, whatever is left: a lane past the item's rows repeats the item's last element, a request
        // past the end of the chain (or for an item whose rows do not exist) the chain's first element: one request
        // per decoded item keeps the count of loads in flight exact.
        const void *src = desc[0].comp;
        uint32_t voff = 0u;
        const uint32_t *cw_src = sync + 3;
        uint32_t cw_off = 0u;
        info = kItemEnd;
        poff = 0u;
        if (live) {
            const chain_table_u32x4 e = *reinterpret_cast<const __attribute__((address_space(4))) chain_table_u32x4 *>(
                wk.items + kChainTableHeaderWords + 4 * wk.it);
            const uint32_t slab = e.z & 0xFFu, rpi = (e.z >> 8) & 0xFFu, lanes = e.z >> 16;
            const int rows_left = wk.rows - (int)e.y;
            const uint32_t rows_here = rows_left <= 0 ? 0u : ((uint32_t)rows_left < rpi ? (uint32_t)rows_left : rpi);
            const uint32_t nact = rows_here * lanes;
            info = (uint32_t)wk.layer | (slab << 16) | (nact << 24);
            poff = wk.parity_off + e.w;
            if (nact != 0u) {
                src = wk.comp;
                const uint32_t off = e.x + wk.row0x16 * lanes;
                voff = off + umin((uint32_t)lane, nact - 1u) * 16u;
                if (MODE == RPTC_CONTINUOUS && slab > 0u) {
                    // the word in front of a row: last word of the row's lane 31 in the slab before (read by all lanes
                    // of the row; used by its first lane).  In slab 0 the word is zero: read from a word of the sync
                    // area that always is, so that nothing outside the decode block has to look at the register.
                    // (The slab before a ragged slab is a full one, and an item's rows are as far apart there.)
                    const uint32_t sub = umin(lanes == 32u ? (uint32_t)lane >> 5 : (uint32_t)lane / lanes, rows_here - 1u);
                    const uint32_t m32 = (uint32_t)desc[wk.layer].m * 32u;
                    const uint32_t elem_prev = (slab - 1u) * m32 + ((wk.row0x16 >> 4) + e.y) * 32u + 31u;
                    cw_src = wk.comp;
                    cw_off = (elem_prev << 4) + 12u + sub * 512u;
                }
            }
            if (++wk.it == wk.it_end) live = wk.enter(desc, wk.layer + 1, wave, block, part_floats);
        }
        issue_load_b128(dst, src, voff);
        if (MODE == RPTC_CONTINUOUS) issue_load_b32(cw, cw_src, cw_off);
    };

    // the layer this wave is in (it has entered it and not yet counted its arrival behind it)
    int cur_layer = -1;
    bool failed = false;
    auto give_up = [&]() {
        if (lane == 0) {
            __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __hip_atomic_store(&sync[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        failed = true;
    };
    // leaves the current layer and enters `target` (or, target == count, leaves the chain): the wave counts its
    // arrival behind every layer on the way, also those in which it had nothing to decode, and enters none before
    // the service wave allows it
    auto move_to = [&](int target) {
        while (cur_layer < target) {
            if (cur_layer >= 0 && lane == 0)
                __hip_atomic_fetch_add(ctl + kCtlDone + (cur_layer & 1), 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            cur_layer++;
            if (cur_layer < count && !lds_wait_ge(ctl + kCtlGo, (uint32_t)cur_layer + 1u, abort_word, spin_limit)) {
                give_up();
                return;
            }
        }
    };

    uint32_t xr[32];
    uint32_t xr_key = 0xFFFFFFFFu;          // layer and slab the activation registers hold
    uint32_t part_lane = 0;                 // LDS byte address of this lane's partial sum for the item's first row
    uint64_t first_lanes = 0;               // the lanes that hold the first element of a row
    bool full_slab = true;
    // one ring position: decode what it holds, then let it take the item DEPTH ahead
    auto step = [&](chain_u32x4 &e_reg, uint32_t &cw_reg, uint32_t &info, uint32_t &poff, bool primed) -> bool {
        if (primed) {
            if (info == kItemEnd) return false;
            const int layer = (int)(info & 0xFFFFu);
            if (layer != cur_layer) {
                move_to(layer);
                if (failed) return false;
            }
            const uint32_t nact = info >> 24;
            const uint32_t key = info & 0xFFFFFFu;
            if (nact != 0u && key != xr_key) {
                xr_key = key;
                const auto &d = desc[layer];
                const int n = d.n, T = n >> 11, Lt = (n & 2047) >> 6, slab = (int)(key >> 16);
                full_slab = slab < T;
                int sub, l;
                if (full_slab) {
                    sub = lane >> 5;
                    l = lane & 31;
                } else {
                    sub = (int)((uint32_t)lane / (uint32_t)Lt);
                    l = lane - sub * Lt;
                    if (sub >= d.rw_tail) l = 0;
                }
                const uint32_t *xp = xbuf + (nb == 3 ? layer % 3 : 0) * xslot_words + (full_slab ? 1024 * slab : 1024 * T) + l;
                if (full_slab) {
                    const uint32_t xa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(xp));
#pragma unroll
                    for (int q = 0; q < 32; q++)
                        asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(xr[q]) : "v"(xa), "n"(128 * q));
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                } else {
#pragma unroll
                    for (int q = 0; q < 32; q++) xr[q] = xp[q * Lt];
                }
                first_lanes = __builtin_amdgcn_ballot_w64(l == 0);
                const int pstride = T + Lt;
                part_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(part)) + 4u * (uint32_t)(sub * pstride + (full_slab ? slab : T + l));
            }
            if (nact != 0u) {                       // (an item whose rows do not exist in this workgroup's block: nothing to do)
                uint64_t keep = nact >= 64u ? ~0ull : (1ull << nact) - 1ull;
                // everything but the DEPTH - 1 requests issued after this one has arrived: exact, this wave issues nothing else
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * kLoadsPerRequest) : "memory");
                float a0, a1, a2, a3;
                decode_element_asm(e_reg, MODE == RPTC_CONTINUOUS ? cw_reg : e_reg.w, first_lanes, lane4, xr, a0, a1, a2, a3);
                float sum = (a0 + a1) + (a2 + a3);
                if (full_slab) {
                    sum = half_wave_sum(sum);       // lanes 31 and 63 hold their row's 32 elements
                    keep &= 0x8000000080000000ull;
                }
                if ((keep >> lane) & 1ull) {
                    typedef __attribute__((address_space(3))) float lds_float;
                    *reinterpret_cast<lds_float *>(static_cast<uintptr_t>(part_lane + poff)) = sum;
                }
            }
        }
        request(e_reg, cw_reg, info, poff);
        return true;
    };

    chain_u32x4 ring[DEPTH];
    uint32_t ring_cw[DEPTH], ring_info[DEPTH], ring_poff[DEPTH];
    static_assert(DEPTH >= 1 && DEPTH <= 4, "ring positions are spelled out below");
    bool primed = false;
    while (true) {
        if (!step(ring[0], ring_cw[0], ring_info[0], ring_poff[0], primed)) break;
        if constexpr (DEPTH > 1) {
            if (!step(ring[1], ring_cw[1], ring_info[1], ring_poff[1], primed)) break;
        }
        if constexpr (DEPTH > 2) {
            if (!step(ring[2], ring_cw[2], ring_info[2], ring_poff[2], primed)) break;
        }
        if constexpr (DEPTH > 3) {
            if (!step(ring[3], ring_cw[3], ring_info[3], ring_poff[3], primed)) break;
        }
        primed = true;
    }
    // the ring's last requests are still in flight: they must have landed before the registers are given up
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (!failed) move_to(count);
}

// ---------------------------------------------------------------------------------------------- service wave

template <int DEPTH>
__device__ __forceinline__ void chain_service_wave(ChainDescPtr desc, int count, uint32_t *ctl, uint32_t *xbuf, int nb, int xslot_words,
                                                   const float *part, int part_floats, uint32_t arrivals, uint32_t spin_limit,
                                                   uint32_t *sync, int uses_grid, int lane, int block)
{
    uint32_t *const abort_word = ctl + kCtlAbort;
    // fifteen waves wait for what this one does: it goes first when it has something to issue
    __builtin_amdgcn_s_setprio(3);
    bool failed = false;
    auto give_up = [&]() {
        if (lane == 0) {
            __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __hip_atomic_store(&sync[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        failed = true;
    };
    // Stages layer l's activations.  Halves 8 idx .. 8 idx + 7 (dwords 4 idx .. 4 idx + 3) go to the four planes of the
    // slot order (inference.cu:215-221): plane i holds the dwords 4 idx + i, idx = 0 .. n/8 - 1.  A load that writes
    // LDS directly puts lane j's dword at the instruction's LDS address + 4 j, so with lane j reading dword
    // 4 (base + j) + i one instruction fills 64 consecutive slots of plane i: the transposition costs nothing, no
    // register holds the data, and all of a layer's requests (88 for n = 11008) are in flight at once.
    auto stage = [&](int l) {
        const auto &d = desc[l];
        const int n8 = d.n >> 3;
        uint32_t *sx = xbuf + (nb == 3 ? l % 3 : 0) * xslot_words;
        typedef const __attribute__((address_space(1))) uint32_t *global_words;
        typedef __attribute__((address_space(3))) uint32_t *lds_words;
        const global_words x = as_global<global_words>(d.x);
        for (int base = 0; base < n8; base += kWave) {
            if (base + lane < n8) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    __builtin_amdgcn_global_load_lds(x + 4 * (base + lane) + i, (lds_words)(sx + i * n8 + base), 4, 0, 0);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    auto done_full = [&](int l) {
        return lds_wait_ge(ctl + kCtlDone + (l & 1), (uint32_t)kChainDecodeWaves * (uint32_t)((l >> 1) + 1), abort_word, spin_limit);
    };
    auto allow = [&](int layers) {           // decode waves may enter every layer below `layers`
        if (lane == 0) __hip_atomic_store(ctl + kCtlGo, (uint32_t)layers, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    auto late = [&](int l) { return l < count && (desc[l].flags & kChLate) != 0; };

    // layers 0 and 1 (1 unless it waits for layer 0)
    stage(0);
    if (count > 1 && !late(1)) stage(1);
    allow(count > 1 && !late(1) ? 2 : 1);

    for (int l = 0; l < count; l++) {
        // the slot of layer l + 2 held layer l - 1: free when every decode wave has left that layer
        if (l + 2 < count && !late(l + 2)) {
            if (l > 0 && !done_full(l - 1)) {
                give_up();
                return;
            }
            stage(l + 2);
        }
        // layer l: all partial sums are in; add them in a fixed order and write the rows
        if (!done_full(l)) {
            give_up();
            return;
        }
        const auto &d = desc[l];
        const int row0 = block * d.rows_per_block;
        const int rows = imin(d.rows_per_block, d.m - row0);
        const int pstride = (d.n >> 11) + ((d.n & 2047) >> 6);
        const float *pl = part + (l & 1) * part_floats;
        const bool coherent = (d.flags & kChFence) != 0;
        // four lanes per row: each adds every fourth partial in rising order, then the four are added
        for (int r = lane >> 2; r < rows; r += 16) {
            float s = 0.f;
            for (int i = lane & 3; i < pstride; i += 4) s += pl[r * pstride + i];
            s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(uint32_t, s), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
            s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(uint32_t, s), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
            if ((lane & 3) == 0) {
                // In a chain with dependencies the rows are written through to device-coherent memory (agent-scope
                // stores): another XCD reads them behind the counter, and two layers that write one buffer reach
                // memory in the order of the chain.  A release fence per layer instead would write back the whole
                // L2 of the XCD (buffer_wbl2) once per layer and workgroup: measured at 10 us per layer.
                if (coherent) __hip_atomic_store(as_global<global_u16_out_ptr>(d.out) + row0 + r, float_to_half_bits(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else as_global<global_u16_out_ptr>(d.out)[row0 + r] = float_to_half_bits(s);
            }
        }
        if (d.flags & kChSignal) {
            // The arrival is counted when this wave's stores (of this and of earlier layers) have completed: a store
            // is acknowledged when it has reached the level its scope names, so everything the other workgroups
            // need is then in device-coherent memory.  They read it behind an acquire that drops what their caches
            // hold, so no cache write-back is part of the hand-over.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_fetch_add(&sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // the next layer, when it had to wait for this one
        if (late(l + 1)) {
            const auto &dn = desc[l + 1];
            if (dn.flags & kChWaitGrid) {
                const uint32_t need = (uint32_t)dn.wait_signals * arrivals;
                bool ok = false;
                for (uint32_t spin = 0; spin < spin_limit; spin++) {
                    if (uniform(__hip_atomic_load(&sync[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >= need) {
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
                // What the other workgroups wrote is visible to every load from here on: the acquire invalidates the
                // CU's vector cache and the L2 lines another XCD may have overwritten in memory.  One wave per
                // workgroup does this, once per dependent layer.
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            }
            stage(l + 1);
        }
        // layer l + 1 is staged by now; layer l + 2 as well unless it waits for layer l + 1
        allow(l + 2 < count && !late(l + 2) ? l + 3 : l + 2);
    }
    // After the chain's last layer: the workgroup that leaves last puts the grid counters back for the next launch
    // (nobody waits on them any more).
    if (!failed && uses_grid) {
        uint32_t left = 0;
        if (lane == 0) left = __hip_atomic_fetch_add(&sync[1], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if (uniform(left) + 1u == arrivals && lane == 0) {
            __hip_atomic_store(&sync[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&sync[1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
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

    // table (256 rows of 64 lane copies, the sign of a row's first value in place) and control words
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

    if (wave == kChainDecodeWaves)
        chain_service_wave<DEPTH>(desc, count, ctl, xbuf, nb, xslot_words, part, part_floats, arrivals, spin_limit, sync, uses_grid,
                                  lane, block);
    else
        chain_decode_wave<S, MODE, DEPTH>(desc, count, ctl, xbuf, nb, xslot_words, part, part_floats, spin_limit, sync, wave, lane,
                                          block, lane4);
}

// ---------------------------------------------------------------------------------------------- host side

struct ChainPlanHost {            // what rptc_chain_t holds (see the header): written by rptc_chain_plan
    uint64_t magic;
    void *device_desc;
    int32_t count, grid, lds_bytes, nb, xslot_words, part_floats, uses_grid;
    uint32_t arrivals, spin_limit;
    int32_t device;
    // a chain without dependencies runs in the per-launch kernel's loop form (matvec.hip) when that fits:
    int32_t loop_at_256;          // its descriptors start 256 * this many bytes into the descriptor area (0: not used)
    int32_t loop_lds_bytes, loop_part_floats, loop_max_items;
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
constexpr int kChainMaxItems = 1 << 16;      // items of a workgroup in one layer (a table of 1 MiB)

int prepare_matvec_chain()
{
    int rc;
    if ((rc = chain_allow_lds(matvec_chain_kernel<6, RPTC_AS_WRITTEN, kChainDepth>))) return rc;
    if ((rc = chain_allow_lds(matvec_chain_kernel<6, RPTC_CONTINUOUS, kChainDepth>))) return rc;
    if ((rc = chain_allow_lds(matvec_chain_kernel<8, RPTC_AS_WRITTEN, kChainDepth>))) return rc;
    return chain_allow_lds(matvec_chain_kernel<8, RPTC_CONTINUOUS, kChainDepth>);
}

struct ChainShape {
    int64_t m, n;
    int rows_per_block, rw_tail, items;
    int64_t table_offset;        // bytes from the start of the descriptor area
};

static int chain_rows_per_block(int64_t m, int grid) { return 2 * (int)((m + 2 * grid - 1) / (2 * grid)); }

static int chain_shape_items(int64_t n, int rows_per_block)
{
    const int T = (int)(n >> 11), lt = (int)((n & 2047) >> 6), rw_tail = lt ? 64 / lt : 1;
    return T * (rows_per_block / 2) + (lt ? (rows_per_block + rw_tail - 1) / rw_tail : 0);
}

static int64_t chain_table_bytes(int items) { return (((int64_t)kChainTableHeaderWords + 4 * (int64_t)items) * 4 + 255) & ~(int64_t)255; }

// the item table of a shape: begin[16], then the items in the order [slab 0][slab 1] ... [ragged slab]
static void chain_build_table(const ChainShape &sh, uint32_t *words)
{
    const int64_t m = sh.m, n = sh.n;
    const int R = sh.rows_per_block, T = (int)(n >> 11), lt = (int)((n & 2047) >> 6), pstride = T + lt;
    const int items_full = R / 2, items_tail = lt ? (R + sh.rw_tail - 1) / sh.rw_tail : 0;
    const int total = T * items_full + items_tail;
    for (int w = 0; w < 16; w++) {
        const int64_t cum = 3 * w + (w >> 2);          // units of work in front of decode wave w: 48 for w = 15
        words[w] = (uint32_t)((int64_t)total * cum / 48);
    }
    ChainItem *it = reinterpret_cast<ChainItem *>(words + kChainTableHeaderWords);
    for (int t = 0; t < T; t++)
        for (int idx = 0; idx < items_full; idx++, it++) {
            it->row_first = (uint32_t)(2 * idx);
            it->offset = (uint32_t)(((int64_t)t * m * 32 + (int64_t)it->row_first * 32) * 16);
            it->geom = (uint32_t)t | (2u << 8) | (32u << 16);
            it->poff = 4u * it->row_first * (uint32_t)pstride;
        }
    for (int idx = 0; idx < items_tail; idx++, it++) {
        it->row_first = (uint32_t)(idx * sh.rw_tail);
        it->offset = (uint32_t)(((int64_t)T * m * 32 + (int64_t)it->row_first * lt) * 16);
        it->geom = (uint32_t)T | ((uint32_t)sh.rw_tail << 8) | ((uint32_t)lt << 16);
        it->poff = 4u * it->row_first * (uint32_t)pstride;
    }
}

// checks the layers and finds the distinct shapes; the layout of the descriptor area is
// [descriptors][sync words][one item table per shape]
static int chain_layout(const rptc_chain_layer *layers, int64_t count, int grid, std::vector<ChainShape> *shapes,
                        std::vector<int> *shape_of, int64_t *total_bytes, int64_t *loop_at = nullptr)
{
    if (!layers) return RPTC_ENULL;
    if (count < 1 || count > 65535) return RPTC_ESHAPE;
    int64_t at = count * (int64_t)sizeof(ChainDesc) + kChainSyncBytes;
    at = (at + 255) & ~(int64_t)255;
    shape_of->assign((size_t)count, -1);
    for (int64_t k = 0; k < count; k++) {
        const rptc_chain_layer &u = layers[k];
        if (!u.compressed || !u.x || !u.out) return RPTC_ENULL;
        if (u.m < 1 || u.n < 64 || u.n % 64 != 0) return RPTC_ESHAPE;
        if (u.n > kChainMaxN || u.m >= (1 << 24) || u.m * u.n >= ((int64_t)1 << 34)) return RPTC_ELIMIT;     // stream < 4 GiB
        if (!aligned16(u.compressed) || !aligned16(u.x)) return RPTC_EALIGN;
        int found = -1;
        for (size_t i = 0; i < shapes->size(); i++)
            if ((*shapes)[i].m == u.m && (*shapes)[i].n == u.n) found = (int)i;
        if (found < 0) {
            ChainShape sh;
            sh.m = u.m;
            sh.n = u.n;
            sh.rows_per_block = chain_rows_per_block(u.m, grid);
            const int lt = (int)((u.n & 2047) >> 6);
            sh.rw_tail = lt ? 64 / lt : 1;
            sh.items = chain_shape_items(u.n, sh.rows_per_block);
            if (sh.items > kChainMaxItems || sh.rows_per_block > 255 * 2 * 128) return RPTC_ELIMIT;
            sh.table_offset = at;
            at += chain_table_bytes(sh.items);
            found = (int)shapes->size();
            shapes->push_back(sh);
        }
        (*shape_of)[(size_t)k] = found;
    }
    // the descriptors of the loop form (one 64-byte line a layer), used when no layer depends on another
    if (loop_at) *loop_at = at;
    at += (count * (int64_t)sizeof(LoopLayer) + 255) & ~(int64_t)255;
    *total_bytes = at;
    return 0;
}

}  // namespace rptc

using namespace rptc;

extern "C" int64_t rptc_chain_desc_bytes(const rptc_chain_layer *layers, int64_t count)
{
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc < 0 ? rc : RPTC_EDEVICE;
    std::vector<ChainShape> shapes;
    std::vector<int> shape_of;
    int64_t total = 0;
    rc = chain_layout(layers, count, dev->cus, &shapes, &shape_of, &total);
    return rc ? rc : total;
}

extern "C" int rptc_chain_plan(const rptc_chain_layer *layers, int64_t count, void *device_desc, int64_t device_desc_bytes,
                               rptc_chain_t *plan, void *stream)
{
    if (!layers || !device_desc || !plan) return RPTC_ENULL;
    if (reinterpret_cast<uintptr_t>(device_desc) & 255u) return RPTC_EALIGN;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    const int grid = dev->cus;
    std::vector<ChainShape> shapes;
    std::vector<int> shape_of;
    int64_t total_bytes = 0, loop_at = 0;
    if ((rc = chain_layout(layers, count, grid, &shapes, &shape_of, &total_bytes, &loop_at))) return rc;
    if (device_desc_bytes < total_bytes) return RPTC_ELIMIT;
    std::vector<uint32_t> image((size_t)total_bytes / 4, 0u);
    ChainDesc *descs = reinterpret_cast<ChainDesc *>(image.data());
    int n_max = 0, part_max = 0;
    for (int64_t k = 0; k < count; k++) {
        const rptc_chain_layer &u = layers[k];
        const ChainShape &sh = shapes[(size_t)shape_of[(size_t)k]];
        ChainDesc &d = descs[k];
        d.comp = reinterpret_cast<const uint32_t *>(u.compressed);
        d.x = reinterpret_cast<const uint32_t *>(u.x);
        d.out = u.out;
        d.items = reinterpret_cast<const uint32_t *>(static_cast<const char *>(device_desc) + sh.table_offset);
        d.m = (int)u.m;
        d.n = (int)u.n;
        d.rows_per_block = sh.rows_per_block;
        d.rw_tail = sh.rw_tail;
        const int pstride = (d.n >> 11) + ((d.n & 2047) >> 6);
        if (d.n > n_max) n_max = d.n;
        if (d.rows_per_block * pstride > part_max) part_max = d.rows_per_block * pstride;
    }
    for (const ChainShape &sh : shapes) chain_build_table(sh, image.data() + sh.table_offset / 4);
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
    // The activations of a layer that is not behind the counter are read two layers ahead, so for such a layer
    // "earlier" reaches back to the last counter-guarded layer at or before k - 2.
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
            descs[k - 1].flags |= kChSignal;
            signals++;
            descs[k].flags |= kChLate | kChWaitGrid;
            descs[k].wait_signals = signals;
            any = true;
        } else if (nb == 1) {
            descs[k].flags |= kChLate;
        }
    }
    if (any)
        for (int64_t k = 0; k < count; k++) descs[k].flags |= kChFence;
    // No layer reads or writes what another writes (every pair was looked at: without a guarded layer "earlier"
    // reaches back to the start): the loop form of the per-launch kernel runs the chain when it fits.
    int loop_xslot_words = 0, loop_part_floats = 0, loop_lds_bytes = 0, loop_max_items = 0;
    const bool loop = !any && (loop_at >> 8) < (int64_t)1 << 31 &&
                      matvec_loop_plan(layers, count, grid, reinterpret_cast<LoopLayer *>(image.data() + loop_at / 4),
                                       &loop_xslot_words, &loop_part_floats, &loop_lds_bytes, &loop_max_items) == 0;
    // the sync words behind the descriptors start at zero
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((rc = (int)hipMemcpyAsync(device_desc, image.data(), (size_t)total_bytes, hipMemcpyHostToDevice, s))) return rc;
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
    if (loop) {
        p.loop_at_256 = (int32_t)(loop_at >> 8);
        p.loop_lds_bytes = loop_lds_bytes;
        p.loop_part_floats = loop_part_floats;       // (the activation image is xslot_words long in both forms)
        p.loop_max_items = loop_max_items;
    }
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
    if (p.loop_at_256 > 0) {
        if (p.loop_lds_bytes > kMaxLds) return RPTC_EDEVICE;
        auto a_loop = reinterpret_cast<const LoopLayer *>(static_cast<const char *>(p.device_desc) + ((int64_t)p.loop_at_256 << 8));
        rc = matvec_loop_launch(a_loop, a_cb, p.count, p.xslot_words, p.loop_part_floats, p.loop_lds_bytes, p.loop_max_items, p.grid, S, carry_mode, s);
        if (rc) return rc;
        return t.end();
    }
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
