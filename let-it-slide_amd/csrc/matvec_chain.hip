// A chain of fused decode + mat-vecs (the op of matvec.hip: rptc_kernels/csrc/rptc_kernels/inference.cu:189-277)
// in ONE launch: layer k of the chain is out_k = W_k x_k on its own stream, activations and output.  Host side:
// the plan and the launch; the kernels are the loop forms of the per-launch kernel in matvec.hip.
//
// Why: a mat-vec of a few megabytes lasts a few microseconds, and a launch per layer spends about half of that on
// things that are not the layer: the dispatch of the grid, the table build and staging in front of the first decode,
// and a tail in which most waves have run out of work.  In a chain the grid is launched once and stays (one 16-wave
// workgroup per CU), the LDS table is built once, and everything a layer reads is requested a layer ahead.
//
// The one-launch form holds layers that do not depend on each other.  A chain in which a layer reads or overwrites
// what another layer writes is refused at plan time (RPTC_EDEPEND): a grid-wide hand-over between dependent layers
// inside one launch costs four dependent trips to memory (rows out and acknowledged, arrival counted, counter
// polled, activations in), which measured slower than the launch boundary it replaces, so such layers are the
// caller's to run as separate launches on one stream.
#include <string.h>

#include <vector>

#include "matvec_loop.hpp"
#include "rptc_common.hpp"

namespace rptc {

constexpr uint64_t kChainMagic = 0x5250544343484E33ull;           // "RPTCCHN3"

struct ChainPlanHost {            // what rptc_chain_t holds (see the header): written by rptc_chain_plan
    uint64_t magic;
    void *device_desc;
    int32_t count, grid, lds_bytes, xslot_words, part_floats, max_items;
    int32_t steady;               // every layer has one shape, and it fits the kernel of matvec_steady.hip: its geometry follows
    int32_t m, n, rows_per_block, rw_tail, items_tail;
    uint32_t full_magic;
    int32_t device;
};
static_assert(sizeof(ChainPlanHost) <= sizeof(rptc_chain_t), "the public struct holds the plan");

static bool overlaps(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes)
{
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + (uintptr_t)b_bytes && b0 < a0 + (uintptr_t)a_bytes;
}

// pointers, shapes, alignment; the descriptor area is one 64-byte descriptor per layer
static int chain_check(const rptc_chain_layer *layers, int64_t count, int64_t *total_bytes)
{
    if (!layers) return RPTC_ENULL;
    if (count < 1 || count > 65535) return RPTC_ESHAPE;
    for (int64_t k = 0; k < count; k++) {
        const rptc_chain_layer &u = layers[k];
        if (!u.compressed || !u.x || !u.out) return RPTC_ENULL;
        if (u.m < 1 || u.n < 64 || u.n % 64 != 0) return RPTC_ESHAPE;
        if (u.m >= (1 << 24) || u.m * u.n >= ((int64_t)1 << 34)) return RPTC_ELIMIT;     // stream < 4 GiB: 32-bit offsets
        if (!aligned16(u.compressed) || !aligned16(u.x)) return RPTC_EALIGN;
    }
    *total_bytes = (count * (int64_t)sizeof(LoopLayer) + 255) & ~(int64_t)255;
    return 0;
}

}  // namespace rptc

using namespace rptc;

extern "C" int64_t rptc_chain_desc_bytes(const rptc_chain_layer *layers, int64_t count)
{
    int64_t total = 0;
    const int rc = chain_check(layers, count, &total);
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
    int64_t total_bytes = 0;
    if ((rc = chain_check(layers, count, &total_bytes))) return rc;
    if (device_desc_bytes < total_bytes) return RPTC_ELIMIT;
    // Nothing orders a layer's reads behind another layer's writes, and the kernel asks for a layer's stream and
    // activations a layer ahead: no output may overlap anything another layer (or the layer itself) reads or writes.
    for (int64_t k = 0; k < count; k++) {
        const rptc_chain_layer &a = layers[k];
        const int64_t out_bytes = 2 * a.m;
        for (int64_t j = 0; j < count; j++) {
            const rptc_chain_layer &b = layers[j];
            if (overlaps(a.out, out_bytes, b.x, 2 * b.n) || overlaps(a.out, out_bytes, b.compressed, b.m * b.n / 4) ||
                (j != k && overlaps(a.out, out_bytes, b.out, 2 * b.m)))
                return RPTC_EDEPEND;
        }
    }
    std::vector<LoopLayer> image((size_t)total_bytes / sizeof(LoopLayer));
    int xslot_words = 0, part_floats = 0, lds_bytes = 0, max_items = 0, uniform = 0;
    if ((rc = matvec_loop_plan(layers, count, dev->cus, image.data(), &xslot_words, &part_floats, &lds_bytes, &max_items, &uniform)))
        return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((rc = (int)hipMemcpyAsync(device_desc, image.data(), (size_t)total_bytes, hipMemcpyHostToDevice, s))) return rc;
    if ((rc = (int)hipStreamSynchronize(s))) return rc;
    ChainPlanHost p;
    memset(&p, 0, sizeof(p));
    p.magic = kChainMagic;
    p.device_desc = device_desc;
    p.count = (int)count;
    p.grid = dev->cus;
    p.lds_bytes = lds_bytes;
    p.xslot_words = xslot_words;
    p.part_floats = part_floats;
    p.max_items = max_items;
    p.steady = uniform && matvec_steady_fits(image[0]) ? 1 : 0;
    p.m = image[0].m, p.n = image[0].n, p.rows_per_block = image[0].rows_per_block;
    p.rw_tail = image[0].rw_tail, p.items_tail = image[0].items_tail, p.full_magic = image[0].full_magic;
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
    auto a_layers = reinterpret_cast<const LoopLayer *>(p.device_desc);
    auto a_cb = reinterpret_cast<const uint32_t *>(codebook);
    if (p.steady) {
        LoopLayer shape{};
        shape.m = p.m, shape.n = p.n, shape.rows_per_block = p.rows_per_block;
        shape.rw_tail = p.rw_tail, shape.items_tail = p.items_tail, shape.full_magic = p.full_magic;
        rc = matvec_steady_launch(a_layers, shape, a_cb, p.count, p.max_items, p.grid, S, carry_mode, s);
    } else {
        rc = matvec_loop_launch(a_layers, a_cb, p.count, p.xslot_words, p.part_floats, p.lds_bytes, p.max_items, p.grid, S, carry_mode, s);
    }
    if (rc) return rc;
    return t.end();
}
