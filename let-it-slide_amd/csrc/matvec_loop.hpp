// A chain of independent mat-vecs in one launch of the per-launch kernel's body (matvec.hip): what the chain's host
// code (matvec_chain.hip) needs to plan and launch it.
#pragma once
#include "rptc_common.hpp"

namespace rptc {

struct LoopLayer {               // one layer as the kernel reads it (through the scalar cache): 64 bytes
    const uint32_t *comp;        // [T][m][32] uint4, then the ragged slab [m][Lt]
    const uint4 *x;              // fp16 [n]
    uint16_t *out;               // fp16 [m]
    int32_t m, n, rows_per_block, rw_tail, items_tail;
    uint32_t full_magic;         // floor(2^32 / items_full) + 1 (0 for items_full = 1)
    int32_t same_shape_as_previous;   // m and n equal those of the layer in front: its geometry can be taken over
    int32_t pad[3];
};
static_assert(sizeof(LoopLayer) == 64, "a descriptor is one 64-byte line");

// Fills `out[count]` for a device of `cus` compute units.  Returns 0 when the kernel can run the chain (every layer's
// activations fit a thread's two registers, a wave has at most four stream elements of a layer, two activation images and
// two sets of partial sums fit in LDS beside the table), RPTC_ELIMIT when it cannot; the caller has checked pointers,
// shapes and that no layer depends on another.  max_items: 3 or 4, the kernel variant that holds a wave's elements;
// uniform: 1 when every layer has the shape of the first.
int matvec_loop_plan(const rptc_chain_layer *layers, int64_t count, int cus, LoopLayer *out, int *xslot_words,
                     int *part_floats, int *lds_bytes, int *max_items, int *uniform);
// One launch over `count` layers whose descriptors are in device memory; returns hipGetLastError()'s value.
int matvec_loop_launch(const LoopLayer *device_layers, const uint32_t *codebook, int count, int xslot_words,
                       int part_floats, int lds_bytes, int max_items, int grid, int S, int carry_mode, hipStream_t stream);

// The same chain when every layer has the shape of `shape` and that shape fits the fixed LDS layout of the kernel of
// matvec_steady.hip (`matvec_steady_fits`): the loop over layers as one hand-written block.
bool matvec_steady_fits(const LoopLayer &shape);
int matvec_steady_launch(const LoopLayer *device_layers, const LoopLayer &shape, const uint32_t *codebook, int count, int max_items,
                         int grid, int S, int carry_mode, hipStream_t stream);

// One layer per launch with the chain kernel's hand-written body (matvec_steady.hip): whether a layer of width n whose
// workgroups own rows_per_block rows fits its fixed LDS layout and its four elements a wave, and the launch (the
// arguments of the per-launch kernel).  prologue: 0 none; 1 x is [gate | up] and the activations are silu(gate) * up;
// 2 the activations are the RMS norm of x + delta (delta may be null) times norm_w, and x + delta goes to x_out.
bool matvec_one_fits(int n, int rows_per_block, int items_tail);
int matvec_one_launch(const uint32_t *comp, const uint32_t *codebook, const uint4 *x, uint16_t *out, int m, int n,
                      int rows_per_block, int rw_tail, int items_tail, uint32_t full_magic, int grid, int S, int carry_mode,
                      int prologue, const uint4 *delta, const uint4 *norm_w, uint4 *x_out, float eps, hipStream_t stream);

}  // namespace rptc
