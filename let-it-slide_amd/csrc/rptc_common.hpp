// Shared host/device helpers of librptc_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/rptc_hip.h"

namespace rptc {

constexpr int kWave = 64;              // CDNA4 wavefront
constexpr int kMaxLds = 160 * 1024;    // LDS per workgroup on gfx950

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));

struct DeviceInfo {
    int device = -1;
    int cus = 0;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
};

// Per-device state, created on first use with that device current.  Returns a status.
int device_info(DeviceInfo **out);

// Brackets a launch with the two cached events when ms != nullptr.
struct Timer {
    hipStream_t stream;
    float *ms;
    DeviceInfo *dev;
    int begin(DeviceInfo *d, hipStream_t s, float *out_ms)
    {
        dev = d;
        stream = s;
        ms = out_ms;
        if (!ms) return 0;
        return (int)hipEventRecord(dev->ev_start, stream);
    }
    int end()
    {
        int rc = (int)hipGetLastError();
        if (rc) return rc;
        if (!ms) return 0;
        rc = (int)hipEventRecord(dev->ev_stop, stream);
        if (rc) return rc;
        rc = (int)hipEventSynchronize(dev->ev_stop);
        if (rc) return rc;
        return (int)hipEventElapsedTime(ms, dev->ev_start, dev->ev_stop);
    }
};

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#ifdef __HIPCC__
// ---------------------------------------------------------------- device helpers

__device__ __forceinline__ uint32_t alignbit(uint32_t hi, uint32_t lo, uint32_t shift)
{
    // low 32 bits of ({hi, lo} >> shift), shift in [0, 31]: v_alignbit_b32
    return __builtin_amdgcn_alignbit(hi, lo, shift);
}

// both 16-bit halves of g: h*h + h mod 2^16.  Written as asm because the compiler turns the C
// expression into an add and a multiply.
__device__ __forceinline__ uint32_t pk_hash16(uint32_t g)
{
    uint32_t h;
    asm("v_pk_mad_u16 %0, %1, %1, %1" : "=v"(h) : "v"(g));
    return h;
}

// (a & mask) | c in one op; mask must sit in a scalar register (no literals in VOP3 on gfx9)
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t c)
{
    uint32_t d;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(c));
    return d;
}

// byte permute of {hi, lo}: selector byte i picks the source of result byte i
// (0-3 = bytes of lo, 4-7 = bytes of hi, 0x0C = zero)
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel)
{
    uint32_t d;
    asm("v_perm_b32 %0, %1, %2, %3" : "=v"(d) : "v"(hi), "v"(lo), "s"(sel));
    return d;
}

// 32-bit LDS read at an absolute LDS byte address (no base is added)
__device__ __forceinline__ uint32_t lds_read_abs(uint32_t byte_address)
{
    typedef __attribute__((address_space(3))) const uint32_t lds_u32;
    return *reinterpret_cast<lds_u32 *>(static_cast<uintptr_t>(byte_address));
}

__device__ __forceinline__ float dot2(uint32_t w, uint32_t a, float acc)
{
    // acc + w.lo*a.lo + w.hi*a.hi with the products and the sum in fp32: v_dot2_f32_f16
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, w), __builtin_bit_cast(half2_t, a), acc, false);
}

// Sum over the 64 lanes of a wave with DPP adds only (no LDS traffic); the total ends up in
// lane 63.  Steps: within rows of 16 lanes, then row 0 into 1 and 2 into 3, then rows 0-1 into 2-3.
__device__ __forceinline__ float wave_sum(float v)
{
#define RPTC_DPP_ADD(ctrl, row_mask, bank_mask)                                                      \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(uint32_t, v), \
                                                               ctrl, row_mask, bank_mask, false))
    RPTC_DPP_ADD(0x111, 0xF, 0xF);   // row_shr:1
    RPTC_DPP_ADD(0x112, 0xF, 0xF);   // row_shr:2
    RPTC_DPP_ADD(0x114, 0xF, 0xF);   // row_shr:4
    RPTC_DPP_ADD(0x118, 0xF, 0xF);   // row_shr:8   -> lane 15 of each row holds the row's sum
    RPTC_DPP_ADD(0x142, 0xA, 0xF);   // row_bcast:15 into rows 1 and 3
    RPTC_DPP_ADD(0x143, 0xC, 0xF);   // row_bcast:31 into rows 2 and 3
#undef RPTC_DPP_ADD
    return v;
}

// Sums over lanes 0-31 and over lanes 32-63 (in lanes 31 and 63): wave_sum without its last step.
__device__ __forceinline__ float half_wave_sum(float v)
{
#define RPTC_DPP_ADD(ctrl, row_mask, bank_mask)                                                      \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(uint32_t, v), \
                                                               ctrl, row_mask, bank_mask, false))
    RPTC_DPP_ADD(0x111, 0xF, 0xF);   // row_shr:1
    RPTC_DPP_ADD(0x112, 0xF, 0xF);   // row_shr:2
    RPTC_DPP_ADD(0x114, 0xF, 0xF);   // row_shr:4
    RPTC_DPP_ADD(0x118, 0xF, 0xF);   // row_shr:8
#undef RPTC_DPP_ADD
    // row_bcast:15 into rows 1 and 3 as one instruction (the compiler makes three of it); the nop
    // is the distance a DPP operand needs from the vector op that wrote it
    asm("s_nop 1\n"
        "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf" : "+v"(v));
    return v;
}

// Hand-off of partial results between workgroups (which may run on different XCDs, each with an L2 of its own).
// Between publishing() and published() the producing threads write their results with agent-scope stores (`__hip_atomic_store(..., __ATOMIC_RELAXED,
// __HIP_MEMORY_SCOPE_AGENT)`: global_store ... sc1, written through to the level all XCDs share), then call
// published() and meet at a workgroup barrier; one thread then counts the arrival with arrive().  The workgroup
// that sees the last arrival reads the others' results with agent-scope loads (global_load ... sc1, which do not
// hit in a cache that another XCD's store did not update).
// What makes this enough on gfx942 / gfx950: the vector memory counter of a wave is decremented for a store only
// when the store has been acknowledged at the level its scope bits name, so after `s_waitcnt vmcnt(0)` the wave's
// sc1 stores are visible to every sc1 load of the device; the barrier orders all producing waves of the workgroup
// before the counter update; the counter update and the last arrival's loads are separated by the data dependence
// on the returned count, a barrier and a branch.  A release fence at agent scope in front of the barrier and an
// acquire fence behind the branch say the same in the language's memory model, and are what a first version used:
// the compiler turns them into a write-back and an invalidate of the whole L2 of the XCD (buffer_wbl2 sc1,
// buffer_inv sc1), which nothing here needs (no plain store is part of the hand-off) and which costs 15-25 us per
// launch, measured on the transposed mat-vec (4096 x 4096: 27 us with the fences, 8 us without) and on the batched
// product (batch 16 on 4096 x 11008: 67 us against 15 us).
// The three markers are assembler comments: build.py reads them back from the emitted assembly and fails the build when
// a store between publishing() and published() or a load between merging() and merged() is not an sc1 one, or when
// the wait of published() is not followed by a barrier before the arrival is counted (`handoff_violations`).  Their
// "memory" clobbers keep the compiler from moving a store or load across them.
__device__ __forceinline__ void publishing() { asm volatile("; rptc-handoff: publishing" ::: "memory"); }
__device__ __forceinline__ void published() { asm volatile("; rptc-handoff: published\n\ts_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void merging() { asm volatile("; rptc-handoff: merging" ::: "memory"); }
__device__ __forceinline__ void merged() { asm volatile("; rptc-handoff: merged" ::: "memory"); }
__device__ __forceinline__ uint32_t arrive(uint32_t *counter)
{
    return __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f)
{
    _Float16 h = (_Float16)f;   // v_cvt_f16_f32, round to nearest even
    return __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ float half_bits_to_float(uint16_t b)
{
    return (float)__builtin_bit_cast(_Float16, b);
}

// silu(gate) * up on fp16 values: silu in fp32 through the hardware exp2 and reciprocal, rounded to
// fp16, then an fp16 product.  One definition (no contraction) so that every kernel that computes
// the gate rounds the same way.
__device__ __forceinline__ uint16_t silu_mul_bits(uint16_t gate, uint16_t up)
{
#pragma clang fp contract(off)
    const float g = half_bits_to_float(gate);
    const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896f);
    const _Float16 sg = (_Float16)(g * __builtin_amdgcn_rcpf(1.f + e));
    const _Float16 r = sg * __builtin_bit_cast(_Float16, up);
    return __builtin_bit_cast(uint16_t, r);
}

// The same for a register of two halves: the same operations on each half (so the same roundings), with the
// halves left packed for the conversions' sake and one packed fp16 multiply at the end.
__device__ __forceinline__ uint32_t silu_mul_pair(uint32_t gate, uint32_t up)
{
#pragma clang fp contract(off)
    const half2_t g2 = __builtin_bit_cast(half2_t, gate);
    const float g0 = (float)g2.x, g1 = (float)g2.y;
    const float e0 = __builtin_amdgcn_exp2f(g0 * -1.44269504088896f), e1 = __builtin_amdgcn_exp2f(g1 * -1.44269504088896f);
    half2_t sg;
    sg.x = (_Float16)(g0 * __builtin_amdgcn_rcpf(1.f + e0));
    sg.y = (_Float16)(g1 * __builtin_amdgcn_rcpf(1.f + e1));
    return __builtin_bit_cast(uint32_t, sg * __builtin_bit_cast(half2_t, up));
}

// the same for the eight halves of 16 bytes
__device__ __forceinline__ uint4 silu_mul8(const uint4 gate, const uint4 up)
{
    const uint32_t g[4] = {gate.x, gate.y, gate.z, gate.w}, u[4] = {up.x, up.y, up.z, up.w};
    uint32_t r[4];
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = silu_mul_pair(g[i], u[i]);
    return make_uint4(r[0], r[1], r[2], r[3]);
}
#endif

}  // namespace rptc
