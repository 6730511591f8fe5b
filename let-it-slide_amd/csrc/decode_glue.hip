// The small kernels between the quantized projections of a Llama decoder layer, batch 1, one
// token per call: residual add + RMS norm, rotary embedding + KV-cache write, single-query
// attention over the cache, SiLU gate.  They exist so that a decode step is a handful of launches
// per layer instead of dozens of framework element-wise kernels; none of them is in the reference
// (it generates with transformers on dense weights, quantize_hf.py:229-236).
// fp16 in and out, fp32 arithmetic.  The position is read from device memory so that a captured
// HIP graph can be replayed for successive tokens.
#include "rptc_common.hpp"

namespace rptc {

__device__ __forceinline__ float block_sum(float v, float *scratch)
{
    // scratch: one float per wave; returns the sum over the workgroup to every thread
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    if (lane == 63) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < waves; w++) t += scratch[w];
    __syncthreads();
    return t;
}

__device__ __forceinline__ float block_max(float v, float *scratch)
{
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = scratch[0];
    for (int w = 1; w < waves; w++) t = fmaxf(t, scratch[w]);
    __syncthreads();
    return t;
}

// Rotation of the pair (a, b) by the angle with cosine c and sine s: fp16 products and an fp16
// difference / sum, as the element-wise framework path computes them.  Contraction is off so that
// every kernel that rotates rounds the same way (a fused multiply-add would skip one rounding, and
// which product it skips is the compiler's choice).
__device__ __forceinline__ void rope_pair(float a, float b, float c, float s, uint16_t &ra, uint16_t &rb)
{
#pragma clang fp contract(off)
    const _Float16 ha = (_Float16)a, hb = (_Float16)b, hc = (_Float16)c, hs = (_Float16)s;
    const _Float16 ac = ha * hc, bs = hb * hs, as = ha * hs, bc = hb * hc;
    const _Float16 x = ac - bs, y = as + bc;
    ra = __builtin_bit_cast(uint16_t, x);
    rb = __builtin_bit_cast(uint16_t, y);
}

// x_out = x_in + delta (delta may be null);  h_out = x_out * rsqrt(mean(x_out^2) + eps) * weight
__global__ __launch_bounds__(1024) void add_rmsnorm_kernel(const uint16_t *__restrict__ x_in, const uint16_t *delta,
                                                            const uint16_t *__restrict__ weight, uint16_t *x_out,
                                                            uint16_t *__restrict__ h_out, int d, float eps)
{
    __shared__ float scratch[16];
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        float v = half_bits_to_float(x_in[i]);
        if (delta) v = half_bits_to_float(float_to_half_bits(v + half_bits_to_float(delta[i])));   // the fp16 residual stream
        x_out[i] = float_to_half_bits(v);
        ss += v * v;
    }
    const float inv = rsqrtf(block_sum(ss, scratch) / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = half_bits_to_float(x_out[i]);
        h_out[i] = float_to_half_bits(half_bits_to_float(float_to_half_bits(v * inv)) * half_bits_to_float(weight[i]));
    }
}

// qkv = [q | k | v], each heads*hd.  Rotates the (2i, 2i+1) pairs of q and k by the angle of the
// position, writes q to q_out and k, v into the caches [heads][max_len][hd] at that position.
__global__ __launch_bounds__(256) void rope_cache_kernel(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ cos_t,
                                                         const uint16_t *__restrict__ sin_t, const int64_t *__restrict__ pos_p,
                                                         uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_cache,
                                                         uint16_t *__restrict__ v_cache, int heads, int hd, int max_len)
{
    const int64_t pos64 = *pos_p;
    // a position outside the caches (a graph replayed past max_len) writes nothing
    if (pos64 < 0 || pos64 >= (int64_t)max_len) return;
    const int pos = (int)pos64;
    const int half = hd >> 1, d = heads * hd;
    const int t = blockIdx.x * blockDim.x + threadIdx.x;        // one (head, pair) per thread
    if (t >= heads * half) return;
    const int h = t / half, i = t - h * half;
    const float c = half_bits_to_float(cos_t[pos * half + i]), s = half_bits_to_float(sin_t[pos * half + i]);
    const int e = h * hd + 2 * i;
    const size_t ce = ((size_t)h * max_len + pos) * hd + 2 * i;
    const float qa = half_bits_to_float(qkv[e]), qb = half_bits_to_float(qkv[e + 1]);
    const float ka = half_bits_to_float(qkv[d + e]), kb = half_bits_to_float(qkv[d + e + 1]);
    rope_pair(qa, qb, c, s, q_out[e], q_out[e + 1]);
    rope_pair(ka, kb, c, s, k_cache[ce], k_cache[ce + 1]);
    v_cache[ce] = qkv[2 * d + e];
    v_cache[ce + 1] = qkv[2 * d + e + 1];
}

// Single-query attention: softmax(q . K^T / sqrt(hd)) V over cache positions 0..pos.
// A head's keys are cut into `splits` contiguous pieces, one 256-thread workgroup each, so that a
// decode step with few heads still fills the chip (heads * splits workgroups).  A workgroup
// produces the piece's maximum score m, the sum l of exp(score - m) and the unnormalised
// acc = sum exp(score - m) * V; they go to a static scratch buffer with device-scope stores, and
// the workgroup that arrives last at the head's counter merges the pieces in piece order:
// out = sum_i acc_i * exp(m_i - M) / sum_i l_i * exp(m_i - M).  Every sum has a fixed order.
// hd/8 lanes share a key (16 bytes of it each), add their partial dot products with shuffles, and
// read 16 bytes of the key's value row each (8 output dimensions).  Such a group keeps a running
// softmax over its own keys (maximum, sum of exponentials, unnormalised value sum), the groups of
// a wave are merged with shuffles and the waves through LDS, always in the same order.
// ROPE = true: q is the projection output [q | k | v]; every workgroup rotates its head's q into
// LDS, and the one whose piece holds *pos also rotates k and appends k and v to the caches (as
// rope_cache_kernel does); it uses the new row from LDS.
constexpr int kAttnThreads = 256;

// v + (v of the lane the DPP pattern names): one vector op, no trip through LDS
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(uint32_t, v), CTRL, 0xF, 0xF, true));
}

// Sum over the lanes_per_key (2, 4, 8, 16 or 32) consecutive lanes that share a key, the same value in each of
// them: neighbours, pairs of neighbours, the mirrored half row and the mirrored row (after the first two steps
// the four lanes of a quad hold one value, so a mirror pairs the right quads), all as DPP adds.  (A loop of
// cross-lane shuffles with a run-time distance is a trip through the LDS hardware per step and key.)
__device__ __forceinline__ float group_sum(float v, int lanes_per_key)
{
    v = dpp_add<0xB1>(v);                                   // quad_perm [1, 0, 3, 2]
    if (lanes_per_key > 2) v = dpp_add<0x4E>(v);            // quad_perm [2, 3, 0, 1]
    if (lanes_per_key > 4) v = dpp_add<0x141>(v);           // row_half_mirror
    if (lanes_per_key > 8) v = dpp_add<0x140>(v);           // row_mirror
    if (lanes_per_key > 16) v += __shfl_xor(v, 16, 64);
    return v;
}
constexpr int kAttnMaxParts = 4096;            // heads * splits
constexpr int kAttnMaxHeads = 1024;
constexpr int kAttnPartStride = 256 + 2;       // acc[hd <= 256], m, l

static __device__ __align__(256) float g_attn_part[kAttnMaxParts * kAttnPartStride];
static __device__ __align__(256) uint32_t g_attn_arrived[kAttnMaxHeads];

// (arguments in the order of their first use: the first 14 dwords arrive preloaded in SGPRs)
template <bool ROPE>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(
    const int64_t *__restrict__ pos_p, const uint16_t *__restrict__ q, uint16_t *k_cache, uint16_t *v_cache,
    int heads, int hd, int max_len, int splits, const uint16_t *__restrict__ cos_t,
    const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ out, float *__restrict__ parts,
    uint32_t *__restrict__ arrived)
{
    extern __shared__ float lds_f[];
    float *scratch = lds_f;                      // [16]: the "came last" flag
    float *acc = scratch + 16;                   // the waves' sums [waves][hd], then their m and l: < 2048 floats
    uint16_t *q_rot = reinterpret_cast<uint16_t *>(acc + 2048);   // [3][hd] halves (q, new k, new v), ROPE only
    const int h = blockIdx.x / splits, sp = blockIdx.x - h * splits, tid = threadIdx.x;
    // A position outside the caches (a graph replayed past max_len) would index the tables and the caches out
    // of bounds: every workgroup of the launch leaves at once (the same value for all), `out` keeps what it held.
    const int64_t pos64 = *pos_p;
    if (pos64 < 0 || pos64 >= (int64_t)max_len) return;
    const int len = (int)pos64 + 1;
    // this workgroup's keys: [s_begin, s_end)
    const int chunk = ((len + splits - 1) / splits + 15) & ~15;
    const int s_begin = sp * chunk, s_end = min(len, s_begin + chunk), cnt = max(0, s_end - s_begin);
    uint16_t *kh = k_cache + (size_t)h * max_len * hd, *vh = v_cache + (size_t)h * max_len * hd;
    const float scale = rsqrtf((float)hd);
    const int pos = len - 1;
    const bool owns_pos = ROPE && pos >= s_begin && pos < s_end;     // this piece holds the new row

    // Every load the piece needs is requested before anything is used: up to kKeysInFlight keys and
    // kValuesInFlight values per thread (the cache is far larger than L2: each load is a memory round
    // trip, and the values do not depend on the scores).  Longer pieces take further rounds.
    const int lanes_per_key = hd >> 3;           // 16 bytes = 8 values per lane
    const int sub = tid % lanes_per_key, slot = tid / lanes_per_key, slots = kAttnThreads / lanes_per_key;
    constexpr int kKeysInFlight = 8;
    uint4 kv[kKeysInFlight], vv[kKeysInFlight];
    // Requests without a condition (a slot past the piece repeats the last position of the context: a row
    // that exists, and what it returns is masked out below): requests under a condition cannot be counted,
    // and the rotation of q would then wait for every key and value instead of for its own five loads.
    auto load_keys = [&](int s0) {
#pragma unroll
        for (int u = 0; u < kKeysInFlight; u++) {
            const int row = min(s_begin + s0 + u * slots + slot, len - 1);
            kv[u] = *reinterpret_cast<const uint4 *>(kh + (size_t)row * hd + 8 * sub);
        }
    };
    auto load_values = [&](int s0) {                  // same shape as the keys: 16 bytes of a row per lane
#pragma unroll
        for (int u = 0; u < kKeysInFlight; u++) {
            const int row = min(s_begin + s0 + u * slots + slot, len - 1);
            vv[u] = *reinterpret_cast<const uint4 *>(vh + (size_t)row * hd + 8 * sub);
        }
    };
    uint16_t *k_new = q_rot + hd, *v_new = k_new + hd;            // the new row, ROPE only
    if (ROPE) {
        const int half = hd >> 1, d = heads * hd;
        float qa = 0.f, qb = 0.f, ka = 0.f, kb = 0.f, c = 0.f, sn = 0.f;
        uint16_t va = 0, vb = 0;
        if (tid < half) {
            // (under a condition, and in front of the keys and values: a block the compiler does not move
            // loads out of, so these come back first)
            const int tp = tid, e = h * hd + 2 * tp;
            c = half_bits_to_float(cos_t[pos * half + tp]);
            sn = half_bits_to_float(sin_t[pos * half + tp]);
            qa = half_bits_to_float(q[e]);
            qb = half_bits_to_float(q[e + 1]);
            ka = half_bits_to_float(q[d + e]);
            kb = half_bits_to_float(q[d + e + 1]);
            va = q[2 * d + e];
            vb = q[2 * d + e + 1];
        }
        // those few loads come back first, and the rotation runs while the keys and values are on their way
        load_keys(0);
        load_values(0);
        // both rotations in every thread (so that none of the loads above moves under the condition below)
        uint16_t qra, qrb, kra, krb;
        rope_pair(qa, qb, c, sn, qra, qrb);
        rope_pair(ka, kb, c, sn, kra, krb);
        if (tid < half) {
            q_rot[2 * tid] = qra;
            q_rot[2 * tid + 1] = qrb;
            if (owns_pos) {
                // the row goes to the caches for later tokens; this launch takes it from LDS, because
                // the loads above may have fetched the row before it was written
                k_new[2 * tid] = kra;
                k_new[2 * tid + 1] = krb;
                v_new[2 * tid] = va;
                v_new[2 * tid + 1] = vb;
                uint16_t *kd = kh + (size_t)pos * hd + 2 * tid, *vd = vh + (size_t)pos * hd + 2 * tid;
                kd[0] = kra;
                kd[1] = krb;
                vd[0] = va;
                vd[1] = vb;
            }
        }
        __syncthreads();
    } else {
        load_keys(0);
        load_values(0);
    }

    // The lanes that share a key (a group) keep a running softmax of their own keys: maximum m,
    // sum l of exp(score - m) and the unnormalised value sum a8 (8 output dimensions a lane), so
    // nothing leaves the group before the piece's last key.  Then the groups of a wave are merged
    // with shuffles, the waves through LDS: one barrier for the whole piece.
    float qf[8];
    {
        const uint4 v = ROPE ? *reinterpret_cast<const uint4 *>(q_rot + 8 * sub)
                             : *reinterpret_cast<const uint4 *>(q + h * hd + 8 * sub);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int u = 0; u < 4; u++) {
            qf[2 * u] = half_bits_to_float((uint16_t)(w[u] & 0xFFFFu));
            qf[2 * u + 1] = half_bits_to_float((uint16_t)(w[u] >> 16));
        }
    }
    float m_g = -INFINITY, l_g = 0.f, a8[8];
#pragma unroll
    for (int c = 0; c < 8; c++) a8[c] = 0.f;
    for (int s0 = 0; s0 < cnt; s0 += kKeysInFlight * slots) {
        if (s0 > 0) {
            load_keys(s0);
            load_values(s0);
        }
        float sc[kKeysInFlight];
        float m_new = m_g;
#pragma unroll
        for (int u = 0; u < kKeysInFlight; u++) {
            const int s = s0 + u * slots + slot;
            uint4 kq = kv[u];
            if (owns_pos && s_begin + s == pos) kq = *reinterpret_cast<const uint4 *>(k_new + 8 * sub);
            const uint32_t w[4] = {kq.x, kq.y, kq.z, kq.w};
            float dot = 0.f;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                dot += half_bits_to_float((uint16_t)(w[c] & 0xFFFFu)) * qf[2 * c];
                dot += half_bits_to_float((uint16_t)(w[c] >> 16)) * qf[2 * c + 1];
            }
            dot = group_sum(dot, lanes_per_key);
            sc[u] = s < cnt ? dot * scale : -INFINITY;
            m_new = fmaxf(m_new, sc[u]);
        }
        // a group with no key yet keeps m = -inf: its factors must be 0, not exp(-inf - -inf)
        const float keep = m_g == -INFINITY ? 0.f : __expf(m_g - m_new);
        l_g *= keep;
#pragma unroll
        for (int c = 0; c < 8; c++) a8[c] *= keep;
        m_g = m_new;
#pragma unroll
        for (int u = 0; u < kKeysInFlight; u++) {
            const int s = s0 + u * slots + slot;
            uint4 vq = vv[u];
            if (owns_pos && s_begin + s == pos) vq = *reinterpret_cast<const uint4 *>(v_new + 8 * sub);
            const float p = sc[u] == -INFINITY ? 0.f : __expf(sc[u] - m_g);
            l_g += p;
            // a slot past the piece holds whatever the repeated row held (possibly not a number): cleared,
            // since 0 * NaN is not 0
            const uint32_t live = s < cnt ? 0xFFFFFFFFu : 0u;
            const uint32_t w[4] = {vq.x & live, vq.y & live, vq.z & live, vq.w & live};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                a8[2 * c] += p * half_bits_to_float((uint16_t)(w[c] & 0xFFFFu));
                a8[2 * c + 1] += p * half_bits_to_float((uint16_t)(w[c] >> 16));
            }
        }
    }
    // the groups of a wave (lanes sub, sub + lanes_per_key, ...): butterfly over the lane bits above
    // the group's, in a fixed order
    for (int off = lanes_per_key; off < 64; off <<= 1) {
        const float m_o = __shfl_xor(m_g, off, 64), l_o = __shfl_xor(l_g, off, 64);
        const float m_n = fmaxf(m_g, m_o);
        const float f_s = m_g == -INFINITY ? 0.f : __expf(m_g - m_n), f_o = m_o == -INFINITY ? 0.f : __expf(m_o - m_n);
        l_g = l_g * f_s + l_o * f_o;
#pragma unroll
        for (int c = 0; c < 8; c++) a8[c] = a8[c] * f_s + __shfl_xor(a8[c], off, 64) * f_o;
        m_g = m_n;
    }
    // the waves: [wave][hd] sums, then m and l of each wave behind them
    constexpr int kWaves = kAttnThreads / 64;
    float *w_acc = acc, *w_m = acc + kWaves * 256, *w_l = w_m + kWaves;
    const int wave = tid >> 6, lane = tid & 63;
    if (lane < lanes_per_key) {
#pragma unroll
        for (int c = 0; c < 8; c++) w_acc[wave * hd + 8 * sub + c] = a8[c];
        if (lane == 0) {
            w_m[wave] = m_g;
            w_l[wave] = l_g;
        }
    }
    __syncthreads();
    float mx = w_m[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) mx = fmaxf(mx, w_m[w]);
    float y = 0.f, sum = 0.f;                    // thread i < hd: output dimension i of this piece
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
        const float f = w_m[w] == -INFINITY ? 0.f : __expf(w_m[w] - mx);
        sum += w_l[w] * f;
        if (tid < hd) y += w_acc[w * hd + tid] * f;
    }
    if (splits == 1) {
        if (tid < hd) out[h * hd + tid] = float_to_half_bits(y / sum);
        return;
    }

    // publish the piece, count the arrival, and let the last workgroup of the head merge
    float *mine = parts + (size_t)blockIdx.x * kAttnPartStride;
    publishing();
    if (tid < hd) __hip_atomic_store(&mine[tid], y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) {
        __hip_atomic_store(&mine[256], mx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&mine[257], sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // (the hand-off between workgroups: see published() / arrive() in rptc_common.hpp)
    published();
    __syncthreads();
    uint32_t *flag = reinterpret_cast<uint32_t *>(scratch);
    if (tid == 0) {
        const uint32_t prev = arrive(&arrived[h]);
        const bool last = prev == (uint32_t)(splits - 1);
        if (last) __hip_atomic_store(&arrived[h], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        *flag = last;
    }
    __syncthreads();
    if (!*flag || tid >= hd) return;
    const float *head_parts = parts + (size_t)h * splits * kAttnPartStride;
    constexpr int kMaxSplits = 16;
    float pm[kMaxSplits], pl[kMaxSplits], pa[kMaxSplits];
    merging();
#pragma unroll
    for (int i = 0; i < kMaxSplits; i++) {
        pm[i] = -INFINITY;
        pl[i] = pa[i] = 0.f;
        if (i < splits) {
            const float *pp = head_parts + (size_t)i * kAttnPartStride;
            pm[i] = __hip_atomic_load(&pp[256], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            pl[i] = __hip_atomic_load(&pp[257], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            pa[i] = __hip_atomic_load(&pp[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    merged();
    float M = pm[0];                             // piece 0 is never empty
#pragma unroll
    for (int i = 1; i < kMaxSplits; i++) M = fmaxf(M, pm[i]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxSplits; i++) {
        const float w = __expf(pm[i] - M);       // an empty piece has m = -inf, so w = 0
        num += pa[i] * w;
        den += pl[i] * w;
    }
    out[h * hd + tid] = float_to_half_bits(num / den);
}

// gu = [gate | up], each f:  out = silu(gate) * up
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t *__restrict__ gu, uint16_t *__restrict__ out, int f)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= f) return;
    out[i] = silu_mul_bits(gu[i], gu[f + i]);
}

// Greedy hand-over from one token to the next in one launch: the arg-max of the logits (the first of
// equal maxima, as the framework's argmax), appended to the output list, becomes the next input token,
// whose embedding row is copied to the decoder's input; the position and the output index move on.
// One workgroup: the vocabulary is scanned once, 16 bytes a thread and step.
constexpr int kGreedyThreads = 1024;

__global__ __launch_bounds__(kGreedyThreads) void greedy_next_kernel(
    const uint16_t *__restrict__ logits, int vocab, const uint16_t *__restrict__ embed, int d, int64_t *token,
    int64_t *out_list, int64_t *out_index, int64_t *pos, uint16_t *__restrict__ x)
{
    __shared__ float s_val[kGreedyThreads / 64];
    __shared__ int s_idx[kGreedyThreads / 64];
    __shared__ int s_best;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float best = -INFINITY;
    int best_i = 0x7FFFFFFF;
    auto take = [&](float v, int i) {          // indices rise along a thread's scan: the first maximum stays
        if (v > best) {
            best = v;
            best_i = i;
        }
    };
    // 16 bytes a load, four loads of a thread asked for before the first is looked at
    const int n8 = vocab >> 3;
    const uint4 *l4 = reinterpret_cast<const uint4 *>(logits);
    constexpr int kInFlight = 4;
    for (int c0 = tid; c0 < n8; c0 += kGreedyThreads * kInFlight) {
        uint4 v[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; u++) v[u] = l4[min(c0 + u * kGreedyThreads, n8 - 1)];
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const int c = c0 + u * kGreedyThreads;
            if (c >= n8) break;
            const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                take(half_bits_to_float((uint16_t)(w[k] & 0xFFFFu)), 8 * c + 2 * k);
                take(half_bits_to_float((uint16_t)(w[k] >> 16)), 8 * c + 2 * k + 1);
            }
        }
    }
    for (int i = 8 * n8 + tid; i < vocab; i += kGreedyThreads) take(half_bits_to_float(logits[i]), i);
    // the larger value wins, the smaller index among equal values
    for (int off = 1; off < 64; off <<= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(best_i, off, 64);
        if (ov > best || (ov == best && oi < best_i)) {
            best = ov;
            best_i = oi;
        }
    }
    if (lane == 0) {
        s_val[wave] = best;
        s_idx[wave] = best_i;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kGreedyThreads / 64; w++)
            if (s_val[w] > best || (s_val[w] == best && s_idx[w] < best_i)) {
                best = s_val[w];
                best_i = s_idx[w];
            }
        if (best_i >= vocab) best_i = 0;       // no logit compared greater than -inf (all not-a-numbers)
        s_best = best_i;
        *token = best_i;
        out_list[*out_index] = best_i;
        *out_index += 1;
        *pos += 1;
    }
    __syncthreads();
    const uint16_t *row = embed + (size_t)s_best * d;
    if ((d & 7) == 0) {                        // rows are 16-byte aligned when the table is
        const uint4 *r4 = reinterpret_cast<const uint4 *>(row);
        uint4 *x4 = reinterpret_cast<uint4 *>(x);
        for (int i = tid; i < (d >> 3); i += kGreedyThreads) x4[i] = r4[i];
    } else {
        for (int i = tid; i < d; i += kGreedyThreads) x[i] = row[i];
    }
}

}  // namespace rptc

using namespace rptc;

extern "C" int rptc_greedy_next(const uint16_t *logits, int64_t vocab, const uint16_t *embed, int64_t d, int64_t *token,
                                int64_t *out_list, int64_t *out_index, int64_t *pos, uint16_t *x, void *stream)
{
    if (!logits || !embed || !token || !out_list || !out_index || !pos || !x) return RPTC_ENULL;
    if (vocab < 1 || vocab >= ((int64_t)1 << 31) || d < 1 || d > (1 << 20)) return RPTC_ESHAPE;
    if (!aligned16(logits) || !aligned16(embed) || !aligned16(x)) return RPTC_EALIGN;
    hipLaunchKernelGGL(greedy_next_kernel, dim3(1), dim3(kGreedyThreads), 0, static_cast<hipStream_t>(stream), logits,
                       (int)vocab, embed, (int)d, token, out_list, out_index, pos, x);
    return (int)hipGetLastError();
}

extern "C" int rptc_add_rmsnorm(const uint16_t *x_in, const uint16_t *delta, const uint16_t *weight, uint16_t *x_out,
                                uint16_t *h_out, int64_t d, float eps, void *stream)
{
    if (!x_in || !weight || !x_out || !h_out) return RPTC_ENULL;
    if (d < 1 || d > (1 << 20)) return RPTC_ESHAPE;
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream), x_in, delta, weight,
                       x_out, h_out, (int)d, eps);
    return (int)hipGetLastError();
}

extern "C" int rptc_rope_cache(const uint16_t *qkv, const uint16_t *cos_t, const uint16_t *sin_t, const int64_t *pos,
                               uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache, int64_t heads, int64_t hd,
                               int64_t max_len, void *stream)
{
    if (!qkv || !cos_t || !sin_t || !pos || !q_out || !k_cache || !v_cache) return RPTC_ENULL;
    if (heads < 1 || hd < 2 || hd % 2 != 0 || max_len < 1) return RPTC_ESHAPE;
    const int threads = (int)(heads * hd / 2);
    hipLaunchKernelGGL(rope_cache_kernel, dim3((threads + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), qkv,
                       cos_t, sin_t, pos, q_out, k_cache, v_cache, (int)heads, (int)hd, (int)max_len);
    return (int)hipGetLastError();
}

namespace rptc {
struct AttnScratch {
    float *parts;
    uint32_t *arrived;
};
static AttnScratch g_attn[64];   // per device: addresses of the static scratch arrays

int prepare_decode_glue(int device)
{
    // the device addresses of the static scratch arrays (the symbols themselves are not device addresses)
    int rc = (int)hipGetSymbolAddress(reinterpret_cast<void **>(&g_attn[device].parts), HIP_SYMBOL(g_attn_part));
    if (rc) return rc;
    return (int)hipGetSymbolAddress(reinterpret_cast<void **>(&g_attn[device].arrived), HIP_SYMBOL(g_attn_arrived));
}

void attn_counters(int device, uint32_t **counters, int *count)
{
    *counters = g_attn[device].arrived;
    *count = kAttnMaxHeads;
}

template <bool ROPE>
static int launch_attn(const uint16_t *q, const uint16_t *cos_t, const uint16_t *sin_t, const int64_t *pos, uint16_t *k_cache,
                       uint16_t *v_cache, uint16_t *out, int64_t heads, int64_t hd, int64_t max_len, void *stream)
{
    // hd a power of two in [16, 256]: 16 bytes per lane, whole keys per wave, whole groups per workgroup
    if (heads < 1 || hd < 16 || hd > 256 || (hd & (hd - 1)) != 0 || max_len < 1) return RPTC_ESHAPE;
    if (heads > kAttnMaxHeads || max_len > (1 << 20)) return RPTC_ELIMIT;
    DeviceInfo *dev;
    int rc = device_info(&dev);
    if (rc) return rc;
    // pieces per head: enough workgroups for every CU, at most 16, none shorter than 16 keys of max_len
    int splits = (int)(dev->cus / heads);
    if (splits > 16) splits = 16;
    if (splits > max_len / 16) splits = (int)(max_len / 16);
    if (splits < 1) splits = 1;
    if (heads * splits > kAttnMaxParts) splits = (int)(kAttnMaxParts / heads);
    const size_t lds = (size_t)(16 + 2048) * 4 + (size_t)hd * 6;
    const AttnScratch &sc = g_attn[dev->device];
    hipLaunchKernelGGL(attn_decode_kernel<ROPE>, dim3((unsigned)(heads * splits)), dim3(kAttnThreads), lds,
                       static_cast<hipStream_t>(stream), pos, q, k_cache, v_cache, (int)heads, (int)hd, (int)max_len, splits,
                       cos_t, sin_t, out, sc.parts, sc.arrived);
    return (int)hipGetLastError();
}
}  // namespace rptc

extern "C" int rptc_attn_decode(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, const int64_t *pos,
                                uint16_t *out, int64_t heads, int64_t hd, int64_t max_len, void *stream)
{
    if (!q || !k_cache || !v_cache || !pos || !out) return RPTC_ENULL;
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache)) return RPTC_EALIGN;
    return launch_attn<false>(q, nullptr, nullptr, pos, const_cast<uint16_t *>(k_cache), const_cast<uint16_t *>(v_cache), out,
                              heads, hd, max_len, stream);
}

extern "C" int rptc_rope_attn_decode(const uint16_t *qkv, const uint16_t *cos_t, const uint16_t *sin_t, const int64_t *pos,
                                     uint16_t *k_cache, uint16_t *v_cache, uint16_t *out, int64_t heads, int64_t hd,
                                     int64_t max_len, void *stream)
{
    if (!qkv || !cos_t || !sin_t || !pos || !k_cache || !v_cache || !out) return RPTC_ENULL;
    if (!aligned16(qkv) || !aligned16(k_cache) || !aligned16(v_cache)) return RPTC_EALIGN;
    return launch_attn<true>(qkv, cos_t, sin_t, pos, k_cache, v_cache, out, heads, hd, max_len, stream);
}

extern "C" int rptc_silu_mul(const uint16_t *gate_up, uint16_t *out, int64_t f, void *stream)
{
    if (!gate_up || !out) return RPTC_ENULL;
    if (f < 1 || f > (1 << 24)) return RPTC_ESHAPE;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((f + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       gate_up, out, (int)f);
    return (int)hipGetLastError();
}
