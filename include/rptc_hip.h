/*
 * rptc_hip.h -- C ABI of librptc_hip.so: gfx950 (MI355X) kernels for the trellis-coded
 * linear layer's inference path.
 *
 * Every entry point takes plain device pointers and sizes, launches on the HIP stream the
 * caller passes (NULL = the legacy default stream), allocates no device memory, keeps no
 * reference to the caller's buffers and returns a status instead of exiting:
 *     0   success
 *   < 0   an RPTC_E* argument error (nothing was launched)
 *   > 0   a hipError_t reported by the runtime
 * rptc_status_string() turns either into text.  When `ms` is not NULL the call brackets its
 * kernels with two events on `stream`, waits for the second and stores the elapsed
 * milliseconds (the reference ops return this figure: wrapper.cpp:4-56); when it is NULL the
 * call is asynchronous.
 *
 * fp16 values travel as uint16_t bit patterns.  `carry_mode` selects how a decoder treats the
 * places where the reference CUDA source departs from one unbroken shift register per row
 * (rptc.py:74-85): RPTC_AS_WRITTEN reproduces the CUDA arithmetic, RPTC_CONTINUOUS the
 * unbroken register.
 *
 * Reference paths below are relative to rptc_kernels/csrc/rptc_kernels/ in the reference tree.
 */
#ifndef RPTC_HIP_H
#define RPTC_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RPTC_AS_WRITTEN 0
#define RPTC_CONTINUOUS 1

#define RPTC_OK 0
#define RPTC_ENULL (-1)      /* a required pointer is NULL */
#define RPTC_ESHAPE (-2)     /* a size breaks the op's shape rule */
#define RPTC_EALIGN (-3)     /* a pointer is not 16-byte aligned */
#define RPTC_EMODE (-4)      /* carry_mode is not one of the two modes */
#define RPTC_ELIMIT (-5)     /* a size exceeds what the kernel's LDS staging can hold */
#define RPTC_EDEVICE (-6)    /* the current device is not gfx950 */
#define RPTC_EALIAS (-7)     /* an output buffer aliases an input the op still reads */
#define RPTC_EDEPEND (-8)    /* a layer of a chain reads or overwrites what a layer of the chain writes */

/* Library version, major*10000 + minor*100 + patch. */
int rptc_version(void);

/* Text for a status returned by any entry point (static storage, never NULL). */
const char *rptc_status_string(int status);

/*
 * Optional.  Prepares the calling thread's current device (queries its properties, creates the
 * two timing events, raises the kernels' dynamic-LDS limits) so that the first op call does not
 * pay for it.  Every op does the same lazily.  Returns RPTC_EDEVICE on anything but gfx950.
 */
int rptc_init(void);

/*
 * The ops that split one output over several workgroups (rptc_decompress_matmul*, rptc_decompress_matvec_t_*
 * on short matrices, rptc_attn_decode / rptc_rope_attn_decode) count arrivals in counters that live in static
 * device memory and return to zero at the end of every launch.  A launch that never finished (a fault in another
 * kernel, a reset) can leave one non-zero, and later launches would then merge too early.  This call counts the
 * counters of the current device that are not zero into *nonzero and, with reset != 0, clears them.  It waits for
 * `stream` (host-synchronous; not for use inside a stream capture) and must not overlap with the ops above.
 * No counterpart in the reference.
 */
int rptc_scratch_check(int reset, int *nonzero, void *stream);

/*
 * Decode only.  Replaces `float decompress(Tensor& compressed, Tensor& codebook, Tensor& out)`
 * (inference.cu:99-160, kernel inference.cu:42-96; bound at wrapper.cpp:60).
 *   compressed  int32 [m][words_per_row], words_per_row % 128 == 0 (inference.cu:106)
 *   codebook    fp16 [65536]                                      (inference.cu:116)
 *   out         fp16 [m][16 * words_per_row], overwritten         (inference.cu:120-123)
 */
int rptc_decompress(const int32_t *compressed, const uint16_t *codebook, uint16_t *out,
                    int64_t m, int64_t words_per_row, int carry_mode, void *stream, float *ms);

/*
 * Fused decode + mat-vec on the [slab][row][lane] stream with the hashed pair codebook.
 * Replace `float decompress_matvec_{L}_{S}_1(Tensor& compressed, Tensor& codebook, Tensor& x,
 * Tensor& out)` (inference.cu:280-380, kernel inference.cu:189-277; bound at
 * wrapper.cpp:61-64).  L names the variant only: the reference kernel never reads it, every
 * variant slides a 16-bit window.
 *   compressed  int32, m*n/16 words: [n/2048][m][32][4]; when n % 2048 != 0 one more slab
 *               [m][(n % 2048)/64][4] follows (an extension of this library; the reference
 *               requires n % 2048 == 0, inference.cu:295-300)
 *   codebook    fp16 [2^(S+1)]: 2^S pairs                         (inference.cu:303-305)
 *   x           fp16 [n], n % 64 == 0
 *   out         fp16 [m], overwritten.  The reference needs m % 32 == 0 (inference.cu:320);
 *               any m >= 1 is accepted here.
 * Products are accumulated in fp32 and rounded once (the reference accumulates in fp16).
 */
int rptc_decompress_matvec_16_6_1(const int32_t *compressed, const uint16_t *codebook,
                                  const uint16_t *x, uint16_t *out, int64_t m, int64_t n,
                                  int carry_mode, void *stream, float *ms);
int rptc_decompress_matvec_20_6_1(const int32_t *compressed, const uint16_t *codebook,
                                  const uint16_t *x, uint16_t *out, int64_t m, int64_t n,
                                  int carry_mode, void *stream, float *ms);
int rptc_decompress_matvec_16_8_1(const int32_t *compressed, const uint16_t *codebook,
                                  const uint16_t *x, uint16_t *out, int64_t m, int64_t n,
                                  int carry_mode, void *stream, float *ms);
int rptc_decompress_matvec_20_8_1(const int32_t *compressed, const uint16_t *codebook,
                                  const uint16_t *x, uint16_t *out, int64_t m, int64_t n,
                                  int carry_mode, void *stream, float *ms);

/*
 * A chain of the mat-vecs above in ONE launch: layer k computes out_k = W_k x_k for its own stream, activations
 * and output (the arithmetic of rptc_decompress_matvec_16_{S}_1, one codebook and one carry mode for the whole
 * chain; 2 bits per weight; n <= 16384, at most four stream elements of a layer per wave: m * n up to
 * 2^26 on 256 compute units).  No counterpart in the reference, whose ops are one launch per layer
 * (inference.cu:318-342).  The grid stays resident: the codebook table is built once and everything a layer reads
 * is requested while the layer in front is decoded.  Each out_k is the same as a separate launch would give, up to
 * the order of the fp32 sums of a row (fixed, so the bits repeat from run to run).
 * The layers must not depend on each other: nothing orders a layer's reads behind another layer's writes.  A chain
 * in which an `out` overlaps any layer's `x` or `compressed` (its own included) or another layer's `out` is refused
 * with RPTC_EDEPEND; run such layers as separate calls on one stream, whose launch boundaries order them (a
 * hand-over between dependent layers inside one launch measured slower than a launch boundary).  The codebook must
 * not overlap any `out` either (not checked: it is passed at launch time).
 *
 *   rptc_chain_desc_bytes(...)     device bytes the caller provides for the chain's descriptors
 *                                  (< 0: a status; at most 65535 layers, each stream below 4 GiB)
 *   rptc_chain_plan(...)           checks the layers, writes the descriptors into device_desc (256-byte aligned
 *                                  device memory; copied on `stream`, which is waited for: a set-up call, not
 *                                  for stream capture) and fills *plan (host memory, opaque).  RPTC_ELIMIT: a
 *                                  layer does not fit the one-launch form; RPTC_EDEPEND: see above.  The plan and
 *                                  the descriptors stay valid until the caller frees device_desc; pointers and
 *                                  sizes of the layers are fixed in them, the contents of the buffers are not.
 *   rptc_decompress_matvec_chain   one launch on `stream` (asynchronous unless ms != NULL)
 */
typedef struct rptc_chain_layer {
    const int32_t *compressed;     /* the stream of rptc_decompress_matvec_16_{S}_1 for m x n */
    const uint16_t *x;             /* fp16 [n] */
    uint16_t *out;                 /* fp16 [m], overwritten */
    int64_t m, n;
} rptc_chain_layer;
typedef struct rptc_chain_t {
    uint64_t opaque[10];
} rptc_chain_t;
int64_t rptc_chain_desc_bytes(const rptc_chain_layer *layers, int64_t count);
int rptc_chain_plan(const rptc_chain_layer *layers, int64_t count, void *device_desc, int64_t device_desc_bytes,
                    rptc_chain_t *plan, void *stream);
int rptc_decompress_matvec_chain(const rptc_chain_t *plan, const uint16_t *codebook, int S, int carry_mode,
                                 void *stream, float *ms);

/*
 * Fused decode + mat-vec on the column-interleaved stream with a scalar 2^L codebook.
 * Replace `float decompress_matvec_t_{16,14}(Tensor& compressed, Tensor& codebook, Tensor& x,
 * Tensor& out)` (inference_t.cu:178-268, kernel inference_t.cu:68-175; bound at
 * wrapper.cpp:65-66).
 *   compressed  int32, at least m*n/16 words, read as uint4 [n/64][m]   (inference_t.cu:116)
 *   codebook    fp16 [2^L]                                              (inference_t.cu:206)
 *   x           fp16 [n], n % 64 == 0, n <= 32768 (the reference's constant-memory bound,
 *               inference_t.cu:49,216)
 *   out         fp16 [m]; the product is ADDED to it                    (inference_t.cu:170-171)
 */
int rptc_decompress_matvec_t_16(const int32_t *compressed, const uint16_t *codebook,
                                const uint16_t *x, uint16_t *out, int64_t m, int64_t n,
                                int carry_mode, void *stream, float *ms);
int rptc_decompress_matvec_t_14(const int32_t *compressed, const uint16_t *codebook,
                                const uint16_t *x, uint16_t *out, int64_t m, int64_t n,
                                int carry_mode, void *stream, float *ms);

/*
 * The dense fp16 matrix a stream stands for, W [m][n] row-major, so that decoded weights can be
 * compared bit for bit.  No counterpart in the reference (its fused kernels never materialise
 * W); the column each decoded pair lands in is fixed by the activation pairing of
 * inference.cu:215-221,249 and inference_t.cu:141-146.
 *   S in {6, 8};  L in {14, 16}.
 */
int rptc_matvec_dense(const int32_t *compressed, const uint16_t *codebook, uint16_t *W,
                      int64_t m, int64_t n, int S, int carry_mode, void *stream, float *ms);
int rptc_matvec_t_dense(const int32_t *compressed, const uint16_t *codebook, uint16_t *W,
                        int64_t m, int64_t n, int L, int carry_mode, void *stream, float *ms);

/*
 * Fused decode + small-batch mat-mat on the hashed pair stream (the stream, codebook and dense
 * matrix W of rptc_decompress_matvec_*; S in {6, 8}):  out[b][r] = sum_c W[r][c] * x[b][c].
 * No counterpart in the reference, which only has the batch-1 kernels (inference.cu:189-277).
 *   x    fp16 [batch][n], batch in [1, 32], n % 64 == 0, n <= 32768
 *   out  fp16 [batch][m], overwritten
 * fp16 products accumulated in fp32 on the matrix cores, rounded once.
 * This is the entry point that allocates nothing: it has no counterpart in the reference and is for callers
 * that cannot allocate device memory or bring a workspace (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  Its scratch - packed activations (2 MiB), partial tiles (32 MiB), arrival
 * counters (128 KiB) - sits in static device arrays that each GPU the library runs on holds until the process
 * ends; a matrix whose partial tiles exceed the 32 MiB is done in several launches, n > 32768 or batch > 32 is
 * refused with RPTC_ELIMIT.  Every call on a device shares those arrays (the counters are cleared at the start
 * of each call): calls that overlap on one device race, whatever their streams.  rptc_decompress_matmul_ws
 * below is the same product with the scratch in a buffer of the caller, for calls that must overlap.
 */
int rptc_decompress_matmul(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                           uint16_t *out, int64_t m, int64_t n, int64_t batch, int S, int carry_mode,
                           void *stream, float *ms);
/* The same at `bits` (2, 3, 4) bits per weight: the stream of rptc_decompress_matvec_bits. */
int rptc_decompress_matmul_bits(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                uint16_t *out, int64_t m, int64_t n, int64_t batch, int S, int bits,
                                int carry_mode, void *stream, float *ms);
/*
 * The same with the scratch memory (packed activations, partial tiles, arrival counters) in a buffer the caller
 * brings: `workspace` is device memory, 256-byte aligned, of at least
 * rptc_decompress_matmul_workspace_bytes(m, n, batch, bits) bytes (< 0: an RPTC_E* status for those sizes); its
 * contents need no initialisation and mean nothing afterwards.  Calls with different workspaces may overlap on
 * different streams of one device; the output is bit-identical to rptc_decompress_matmul_bits.
 */
int64_t rptc_decompress_matmul_workspace_bytes(int64_t m, int64_t n, int64_t batch, int bits);
int rptc_decompress_matmul_ws(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                              uint16_t *out, int64_t m, int64_t n, int64_t batch, int S, int bits,
                              int carry_mode, void *workspace, int64_t workspace_bytes, void *stream, float *ms);

/*
 * The hashed pair stream at `bits` = 2, 3 or 4 bits per weight, S in {6, 8}.  No counterpart in
 * the reference for 3 and 4 (all its kernels are 2 bits/weight); bits == 2 is exactly
 * rptc_decompress_matvec_16_{S}_1.  A step still emits two weights through the same hash of a
 * 16-bit window but consumes 2*bits stream bits; an element still holds 32 steps, so it is
 * 2*bits words long and the stream is int32 [n/2048][m][32][2*bits] (+ ragged slab
 * [m][(n % 2048)/64][2*bits]), m*n*bits/32 words.  x, out, accumulation as for the mat-vec.
 * rptc_matvec_bits_dense writes the dense fp16 matrix W [m][n] such a stream stands for.
 */
int rptc_decompress_matvec_bits(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                uint16_t *out, int64_t m, int64_t n, int S, int bits, int carry_mode,
                                void *stream, float *ms);
int rptc_matvec_bits_dense(const int32_t *compressed, const uint16_t *codebook, uint16_t *W, int64_t m,
                           int64_t n, int S, int bits, int carry_mode, void *stream, float *ms);

/*
 * Random-sign Hadamard (incoherence) transform on activations, fp16 in and out, fp32 inside.
 * No counterpart in the reference (quantize_hf.py:77-117 conditions weights by a scale-and-bias
 * factorisation instead).  Each row of x [batch][n] is cut into blocks of `block` elements
 * (a power of two dividing n, at most 32768; 0 = the largest such power of two) and each block
 * is mapped by
 *     inverse == 0:  y = H (signs .* x) / sqrt(block)
 *     inverse != 0:  y = signs .* (H x) / sqrt(block)
 * with H the Sylvester Hadamard matrix in natural order and signs fp16 [n] of +-1; the two
 * directions undo each other.  out may alias x.
 */
int rptc_sign_hadamard(const uint16_t *x, const uint16_t *signs, uint16_t *out, int64_t batch,
                       int64_t n, int64_t block, int inverse, void *stream, float *ms);

/*
 * The small kernels between the quantized projections of a Llama decoder layer, batch 1, one token
 * per call (no counterpart in the reference, which generates with transformers on dense weights,
 * quantize_hf.py:229-236).  fp16 in and out, fp32 arithmetic, asynchronous on `stream`; `pos` is a
 * device pointer to the token's position so that a captured HIP graph can be replayed.  A position outside
 * [0, max_len) makes rptc_rope_cache, rptc_attn_decode and rptc_rope_attn_decode write nothing (no cache row,
 * no output) instead of indexing the tables and caches out of bounds.
 *   rptc_add_rmsnorm  x_out = x_in + delta (delta may be NULL); h_out = rmsnorm(x_out) * weight; all [d]
 *   rptc_rope_cache   qkv = [q|k|v], each heads*hd: rotate the (2i, 2i+1) pairs of q and k by
 *                     cos/sin [max_len][hd/2] at *pos, write q_out and k, v into caches [heads][max_len][hd]
 *   rptc_attn_decode  out[h] = softmax(q[h] . K[h]^T / sqrt(hd)) V[h] over cache positions 0..*pos
 *   rptc_silu_mul     gate_up = [gate|up], each f: out = silu(gate) * up
 *   rptc_rope_attn_decode  rptc_rope_cache followed by rptc_attn_decode in one launch (q stays on chip)
 *   rptc_greedy_next  greedy hand-over to the next token: *token = argmax(logits[0..vocab)) (first of equal
 *                     maxima), out_list[*out_index] = *token, x[0..d) = embed[*token][0..d), then
 *                     *out_index += 1 and *pos += 1; all pointers are device memory (the caller makes
 *                     out_list long enough), so a captured graph needs nothing from the host per token
 */
int rptc_add_rmsnorm(const uint16_t *x_in, const uint16_t *delta, const uint16_t *weight, uint16_t *x_out,
                     uint16_t *h_out, int64_t d, float eps, void *stream);
int rptc_rope_cache(const uint16_t *qkv, const uint16_t *cos_t, const uint16_t *sin_t, const int64_t *pos,
                    uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache, int64_t heads, int64_t hd,
                    int64_t max_len, void *stream);
int rptc_attn_decode(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, const int64_t *pos,
                     uint16_t *out, int64_t heads, int64_t hd, int64_t max_len, void *stream);
int rptc_silu_mul(const uint16_t *gate_up, uint16_t *out, int64_t f, void *stream);
int rptc_greedy_next(const uint16_t *logits, int64_t vocab, const uint16_t *embed, int64_t d, int64_t *token,
                     int64_t *out_list, int64_t *out_index, int64_t *pos, uint16_t *x, void *stream);
int rptc_rope_attn_decode(const uint16_t *qkv, const uint16_t *cos_t, const uint16_t *sin_t, const int64_t *pos,
                          uint16_t *k_cache, uint16_t *v_cache, uint16_t *out, int64_t heads, int64_t hd,
                          int64_t max_len, void *stream);

/*
 * The mat-vec of rptc_decompress_matvec_16_{S}_1 with the element-wise step that precedes it in a
 * decoder layer done inside the kernel, while the stream is on its way from memory (no counterpart
 * in the reference).  Same stream, codebook, shape rules, carry modes and fp16 roundings as the
 * separate calls.
 *   rptc_decompress_matvec_silu     activations = silu(gate) * up, gate_up = [gate | up], each n
 *   rptc_decompress_matvec_rmsnorm  r = x_in + delta (delta may be NULL); x_out = r;
 *                                   activations = r * rsqrt(mean(r^2) + eps) * weight; n <= 16384;
 *                                   x_out must not be x_in or delta (RPTC_EALIAS)
 *   rptc_decompress_matvec_hadamard activations = H_P (signs .* x) / sqrt(P) per block of P elements: the
 *                                   forward transform of rptc_sign_hadamard (block = 0: the largest power
 *                                   of two dividing n); n <= 15360
 */
int rptc_decompress_matvec_silu(const int32_t *compressed, const uint16_t *codebook, const uint16_t *gate_up,
                                uint16_t *out, int64_t m, int64_t n, int S, int carry_mode, void *stream,
                                float *ms);
int rptc_decompress_matvec_hadamard(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                    const uint16_t *signs, uint16_t *out, int64_t m, int64_t n, int64_t block,
                                    int S, int carry_mode, void *stream, float *ms);
int rptc_decompress_matvec_rmsnorm(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x_in,
                                   const uint16_t *delta, const uint16_t *weight, uint16_t *x_out, uint16_t *out,
                                   int64_t m, int64_t n, float eps, int S, int carry_mode, void *stream,
                                   float *ms);

/*
 * The same mat-vecs with the row/column factorisation the reference's quantizer puts around a
 * quantized matrix, W = b_out + b_in + s_out * s_in * W_hat (quantize_hf.py:77-117 finds the four
 * vectors, quantize_hf.py:167 is this formula; the reference applies it to a dense copy of W_hat):
 *     out[r] = s_out[r] * (W_hat (s_in .* a))[r] + b_out[r] * sum(a) + (b_in . a)
 * with a the activations (x; silu(gate) * up; the normed residual), s_in .* a rounded to fp16 and
 * everything behind it in fp32 with one rounding at the end.  scales_in, biases_in: fp16 [n];
 * scales_out, biases_out: fp16 [m]; each may be NULL (scale 1, bias 0).  n <= 16384 and at most 1024 rows
 * per compute unit (RPTC_ELIMIT above: apply the vectors around the plain call instead).
 */
int rptc_decompress_matvec_affine(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x,
                                  const uint16_t *scales_in, const uint16_t *biases_in,
                                  const uint16_t *scales_out, const uint16_t *biases_out, uint16_t *out,
                                  int64_t m, int64_t n, int S, int carry_mode, void *stream, float *ms);
int rptc_decompress_matvec_silu_affine(const int32_t *compressed, const uint16_t *codebook, const uint16_t *gate_up,
                                       const uint16_t *scales_in, const uint16_t *biases_in,
                                       const uint16_t *scales_out, const uint16_t *biases_out, uint16_t *out,
                                       int64_t m, int64_t n, int S, int carry_mode, void *stream, float *ms);
int rptc_decompress_matvec_rmsnorm_affine(const int32_t *compressed, const uint16_t *codebook, const uint16_t *x_in,
                                          const uint16_t *delta, const uint16_t *weight, uint16_t *x_out,
                                          const uint16_t *scales_in, const uint16_t *biases_in,
                                          const uint16_t *scales_out, const uint16_t *biases_out, uint16_t *out,
                                          int64_t m, int64_t n, float eps, int S, int carry_mode, void *stream,
                                          float *ms);

/*
 * The general (L, S, R, V) trellis of the reference's rptc_lite.py: replaces rptc_lite.dequantize
 * (rptc_lite.py:63-73) with its index_fn (rptc_lite.py:12-16).  Per sequence: an int32 register, 0 at the start,
 * register = (register << R) | symbol at every step (never masked, as there), and the step's V outputs are
 * alphabet[index_fn(register)], index_fn(x) = x * (2x + 1) with int32 wraparound, x ^= x >> (L - S) with the
 * arithmetic shift of a signed value, the low S bits.
 *   alphabet  float [2^S][V];  symbols  int32 [rows][length], used with all their 32 bits as the reference uses
 *   them;  out  float [rows][length][V], overwritten
 *   1 <= R <= 16, 1 <= S <= 16, S <= L <= 31, 1 <= V <= 8; alphabet and out 8-byte aligned when V == 2
 */
int rptc_lite_dequantize(const float *alphabet, int L, int S, int R, int V, const int32_t *symbols, int64_t rows,
                         int64_t length, float *out, void *stream, float *ms);

/*
 * Viterbi search for the hashed pair stream: the symbols whose decode by rptc_decompress_matvec_16_{S}_1
 * (carry mode continuous) is closest to the targets.  Replaces the search of the reference's quantizer
 * (rptc.py:13-71, diag_only path: rho[0] = 0 at the start, first index on ties, best end state traced
 * back), on the trellis its inference kernels decode (inference.cu:250-262): 65536 states, 4 stream bits
 * and two weights per step.
 *   targets   float [rows][steps][2], the weight pairs in stream order
 *   weights   NULL, or float per-weight importance [.][steps][2]: row r reads weights + r * weights_row_stride
 *             (0 = one set for all rows); a step costs c0*(x0-w0)^2 + c1*(x1-w1)^2, all sums in fp32
 *   scratch   rptc_viterbi_scratch_bytes(rows, steps) bytes of device memory (the back pointers)
 *   symbols   uint8 [rows][steps], values 0..15;  end_state int32 [rows];  cost float [rows]
 */
int64_t rptc_viterbi_scratch_bytes(int64_t rows, int64_t steps);
int64_t rptc_viterbi_scalar_scratch_bytes(int64_t rows, int64_t steps);
int rptc_viterbi_pairs(const float *targets, const float *weights, int64_t weights_row_stride,
                       const uint16_t *codebook, void *scratch, uint8_t *symbols, int32_t *end_state, float *cost,
                       int64_t rows, int64_t steps, int S, void *stream, float *ms);
/* the same for the streams of rptc_decompress_matvec_bits: bits = 2, 3, 4 per weight, i.e. 4, 6, 8 stream
 * bits per step and symbols 0..15, 0..63, 0..255 */
int rptc_viterbi_pairs_bits(const float *targets, const float *weights, int64_t weights_row_stride,
                            const uint16_t *codebook, void *scratch, uint8_t *symbols, int32_t *end_state, float *cost,
                            int64_t rows, int64_t steps, int S, int bits, void *stream, float *ms);

/*
 * The same search on the reference's own trellis (rptc.py:13-71 as it stands): 2^L states (L = 16 or 14),
 * 2 stream bits and one value per step, the value of state s being alphabet[s]: the stream that
 * rptc_decompress (L = 16) and rptc_decompress_matvec_t_{16,14} decode in carry mode continuous.
 *   targets   float [rows][steps];  weights NULL or float [.][steps] (the reference's
 *             sum(corrections[index]**2), rptc.py:32): a step costs c * (x - alphabet[s])^2 in fp32
 *   alphabet  fp16 [2^L];  scratch rptc_viterbi_scalar_scratch_bytes(rows, steps) bytes
 *   symbols   uint8 [rows][steps], values 0..3;  end_state int32 [rows];  cost float [rows]
 */
int rptc_viterbi_scalar(const float *targets, const float *weights, int64_t weights_row_stride,
                        const uint16_t *alphabet, int L, void *scratch, uint8_t *symbols, int32_t *end_state,
                        float *cost, int64_t rows, int64_t steps, void *stream, float *ms);

/*
 * The search of the reference's rptc_lite.py (quantize, rptc_lite.py:19-60) for the trellis that
 * rptc_lite_dequantize decodes: rho[0] = 0 at the start, per step the cheapest of the 2^R predecessors of every
 * state (first index on ties, as argmin picks), plus sum_v importance[t][v] * (samples[t][v] - alphabet[index_fn(
 * state)][v])^2 in fp32; the cheapest end state is traced back.  symbols[t] is the reference's `quantized[t]`,
 * cost its `expected_loss`.  Any 1 <= S <= L <= 20, R <= min(L, 8), V <= 4 (RPTC_ELIMIT beyond); the parameters the
 * reference's own driver uses (rptc_lite.py:134-139: L = 16, R = 4, V = 2, S <= 9) have a kernel of their own that
 * keeps the path costs in registers, the others a plain one that keeps them in the scratch.
 *   samples     float [rows][steps][V]
 *   importance  NULL (all ones), or float [.][steps][V]: row r reads importance + r * importance_row_stride
 *               (0 = one set for all rows)
 *   alphabet    float [2^S][V];  scratch rptc_lite_viterbi_scratch_bytes(L, R, rows, steps) bytes of device memory
 *   symbols     uint8 [rows][steps], values below 2^R;  end_state int32 [rows];  cost float [rows]
 */
int rptc_lite_viterbi(const float *samples, const float *importance, int64_t importance_row_stride,
                      const float *alphabet, int L, int S, int R, int V, void *scratch, uint8_t *symbols,
                      int32_t *end_state, float *cost, int64_t rows, int64_t steps, void *stream, float *ms);

/* Bytes of scratch rptc_lite_viterbi needs (back pointers of every step, and the path costs where they are not held
 * in registers); 0 for parameters it does not take.  No counterpart in the reference, which lets jax allocate. */
int64_t rptc_lite_viterbi_scratch_bytes(int L, int R, int64_t rows, int64_t steps);

#ifdef __cplusplus
}
#endif

#endif /* RPTC_HIP_H */
