/*
 * frink_hip.h -- C ABI of the MI355X (gfx950) quantized-matmul backend for Frink.
 *
 * What a `frink-hip` backend crate binds: plain pointers and sizes, an int
 * status, a thread-local error string.  No function here panics, aborts or
 * throws across the boundary; shapes are validated before any kernel is
 * launched (the reference's seam contract: a failed launch is an error value
 * the caller logs before falling back, crates/frink-core/src/weight_matrix/
 * gpu_backend.rs:185-194, 676-703).
 *
 * Layouts are the reference's: quantized weights are verbatim GGUF block
 * bytes, row-major, one row = cols/block_elems consecutive blocks, no padding
 * (crates/frink-core/src/weight_matrix.rs:978-1052); activations are
 * [batch][cols] f32; outputs are [batch][rows] f32 (weight_matrix.rs:2310-2316,
 * crates/frink-cuda/src/mul_mm_launch.rs:34-35).
 *
 * Two families of entry points:
 *   frk_hip_launch_*   host buffers in, host buffers out: the drop-in for the
 *                      reference's per-backend launch functions.  Weights are
 *                      kept resident on the device between calls.
 *   frk_hip_*_dev      operands already in HBM, asynchronous on a caller's
 *                      stream: what a resident decode/prefill stack and the
 *                      benchmark use.
 */
#ifndef FRINK_HIP_H
#define FRINK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  0 is success; negative values are errors and
 * frk_hip_last_error() holds the message. */
enum {
    FRK_OK = 0,
    FRK_ERR_NO_DEVICE = -1,   /* no usable gfx950 device, or the backend is switched off */
    FRK_ERR_UNSUPPORTED = -2, /* no kernel for this quant kind: the reference's `None` */
    FRK_ERR_SHAPE = -3,       /* shape/length violation caught before launch */
    FRK_ERR_ARG = -4,         /* null pointer or otherwise unusable argument */
    FRK_ERR_HIP = -5,         /* a HIP runtime call failed: the reference's `Some(Err)` */
    FRK_ERR_OOM = -6
};

/* Quant kinds, numbered by ggml type id (crates/frink-gguf/src/lib.rs:236-242).
 * Names are QuantKind::name() (crates/frink-core/src/weight_matrix.rs:264-290). */
enum { FRK_KIND_Q4_0 = 2, FRK_KIND_Q5_0 = 6, FRK_KIND_Q8_0 = 8, FRK_KIND_Q4_K = 12, FRK_KIND_Q5_K = 13, FRK_KIND_Q6_K = 14,
       FRK_KIND_IQ4_XS = 23, FRK_KIND_MXFP4 = 39 };
/* Q5_0, IQ4_XS and MXFP4 (the 17-byte GGUF block form) have the dequantizer / row gather and the
 * decode GEMV on the f32 activation (dot_q5_0_f32, dot_iq4_xs_f32, dot_mxfp4_gguf_f32,
 * crates/frink-quant/src/lib.rs:4380-4418, 4894-4934, 5506); a batch is one such GEMV per row, the
 * reference's own path below its GEMM threshold (crates/frink-core/src/weight_matrix.rs:2636-2652). */

/* Q8_0 GEMV arithmetic.  F32 multiplies dequantized weights by the f32
 * activation (dot_q8_0_f32, crates/frink-quant/src/lib.rs:663-686); INT8
 * quantizes the activation to Q8_0 blocks first (dot_q8_0_q8, lib.rs:711-733,
 * activation form Avx of crates/frink-quant/src/act_quant.rs:157-189).  The
 * K-quants always take the integer path against Q8_K activations
 * (dot_q4_k_q8 lib.rs:822-869, dot_q6_k_q8 lib.rs:1069-1110). */
enum { FRK_ACT_F32 = 0, FRK_ACT_INT8 = 1, FRK_ACT_F32_DOT = 2 };
/* FRK_ACT_F32_DOT (frk_hip_gemv_dev only): the K-quants multiply their dequantized weights by the f32
 * activation, the numerics of the reference's default x86 decode path (WeightMatrix::dot,
 * crates/frink-core/src/weight_matrix.rs:2044-2048; dot_q4_k_f32, dot_q5_k_f32, dot_q6_k_f32,
 * crates/frink-quant/src/lib.rs:370-415, 461-515, 558-605), within float summation order; rows of at
 * most 16384 columns.  For Q8_0 and Q4_0 it is FRK_ACT_F32. */

typedef struct frk_weights frk_weights; /* opaque: one weight matrix resident in HBM */

/* replaces frink_cuda::gpu::probe / CudaInfo (crates/frink-cuda/src/gpu.rs:79-145) */
typedef struct {
    int32_t device_count;
    int32_t compute_units;
    char name[128];      /* first device's marketing name */
    char gcn_arch[64];   /* e.g. "gfx950:sramecc+:xnack-" */
    uint64_t total_vram_bytes;
    uint64_t free_vram_bytes;
} frk_device_info;

/* Never aborts on a GPU-less host: returns FRK_ERR_NO_DEVICE there. */
int frk_hip_probe(frk_device_info *out);

/* BackendDispatch::dense_enabled (gpu_backend.rs:153-195): env FRINK_HIP with the
 * reference's grammar (0|false|off|cpu = off without opening a device,
 * 1|true|on|hip|rocm = on, anything else = probe; gpu_backend.rs:545-552).
 * Decided once per process. */
int frk_hip_dense_enabled(void);

/* Message of the last error on the calling thread ("" if none). */
const char *frk_hip_last_error(void);

/* BackendCaps::matvec_kernel / gemm_supported / BackendDispatch::has_launch
 * (gpu_backend.rs:110-150, 153-195).  matvec_kernel returns the kind's name
 * ("Q8_0", "Q4_K", "Q6_K") or NULL when there is no decode kernel. */
const char *frk_hip_matvec_kernel(int kind);
int frk_hip_gemm_supported(int kind);
int frk_hip_has_launch(int kind);
/* block geometry (crates/frink-gguf/src/lib.rs:308-314); 0 for an unknown kind */
int frk_hip_block_bytes(int kind);
int frk_hip_block_elems(int kind);
/* worth_a_gemm (crates/frink-cuda/src/mul_mm.rs:634-638): batch sizes the GEMM entry
 * point should take rather than `batch` matvecs.  Here every batch >= 2 qualifies. */
int frk_hip_worth_a_gemm(size_t batch);

/* ---- resident weights (crates/frink-cuda/src/resident.rs:1-120) ----
 * register: uploads `len` bytes of GGUF blocks (borrowed for the duration of the
 * call) and returns a handle.  A later register of the same (pointer, len) whose
 * 192 sampled bytes (first, middle, last 64) still match returns the cached
 * handle; a mismatch re-uploads.  Q6_K and Q8_0 are byte-permuted once into
 * 16-byte-aligned planes on the device; dequantization is bit-identical. */
int frk_hip_weights_register(int kind, const void *host_bytes, size_t len, size_t rows,
                             size_t cols, frk_weights **out);
/* Same, from `len` bytes of GGUF blocks already in device memory (copied/permuted
 * into the library's own allocation; the source may be freed afterwards). */
int frk_hip_weights_from_device(int kind, const void *dev_bytes, size_t len, size_t rows,
                                size_t cols, void *stream, frk_weights **out);
int frk_hip_weights_release(frk_weights *w);
/* Q5_0 / IQ4_XS / MXFP4 (scale bytes within 104..143) reach the matrix cores decoded to signed bytes; a batched call
 * (frk_hip_gemm_dev from four rows on, frk_hip_gemm_grouped_dev, frk_hip_moe_ffn_dev from 32 tokens on) decodes
 * into its scratch memory each time.  This keeps the decoded rows beside the resident ones until the handle is
 * released -- twice the bytes of a Q8_0 matrix of that shape, for a part with HBM to spare -- and those calls skip
 * the decoding (same results, bit for bit).  Decodes on `stream` and synchronizes it.  The reference has no
 * counterpart: its GPU GEMM dequantizes inside the kernel (crates/frink-cuda/src/mul_mm.rs:146-205).  Other kinds:
 * FRK_ERR_UNSUPPORTED. */
int frk_hip_weights_keep_decoded(frk_weights *w, void *stream);
size_t frk_hip_weights_rows(const frk_weights *w);
size_t frk_hip_weights_cols(const frk_weights *w);
int frk_hip_weights_kind(const frk_weights *w);

/* ---- host-buffer entry points: the reference's launch functions ---- */

/* BackendDispatch::launch_matvec (gpu_backend.rs:188-194) /
 * frink_cuda::gpu::launch_q4_k_matvec and siblings (crates/frink-cuda/src/gpu.rs:319-446):
 * out[rows] = W x.  Checks weights_len == rows*row_bytes, row_bytes a whole number of
 * blocks, x_len == blocks*block_elems, rows > 0. */
int frk_hip_launch_matvec(int kind, const uint8_t *weights, size_t weights_len, const float *x,
                          size_t x_len, size_t rows, size_t row_bytes, float *out);

/* frink_cuda::mul_mm_launch::launch_mul_mm (crates/frink-cuda/src/mul_mm_launch.rs:40-68) with
 * validate_shape's checks (crates/frink-cuda/src/mul_mm.rs:581-625):
 * out[token*n_rows + row] = sum_k W[row][k] * x_batch[token*n_cols + k]. */
int frk_hip_launch_mul_mm(int kind, const uint8_t *weights, size_t weights_len,
                          const float *x_batch, size_t x_len, size_t n_rows, size_t n_cols,
                          size_t batch, size_t row_bytes, float *out);

/* One matvec of a group that shares an activation:
 * frink_cuda::matvec_launch::MatvecLaunch (crates/frink-cuda/src/matvec_launch.rs:485-493). */
typedef struct {
    int kind;
    const uint8_t *weights;
    size_t weights_len;
    size_t rows;
    size_t row_bytes;
} frk_matvec_launch;

/* frink_cuda::matvec_launch::launch_matvec_multi (matvec_launch.rs:500-534): uploads x once, runs
 * the n matvecs (q/k/v, or gate and up) on resident weights -- the K-quant matrices share ONE Q8_K
 * quantization of x -- and downloads outs[i][launches[i].rows]. */
int frk_hip_launch_matvec_multi(const float *x, size_t x_len, const frk_matvec_launch *launches,
                                size_t n, float *const *outs);

/* frink_cuda::matvec_launch::launch_dense_ffn_swiglu (matvec_launch.rs:551-570):
 * out = down(silu(gate x) * up x) with one upload of x and one download of out.  gate and up have
 * the same rows and columns; down's columns equal their rows. */
int frk_hip_launch_dense_ffn_swiglu(const frk_matvec_launch *gate, const frk_matvec_launch *up,
                                    const frk_matvec_launch *down, const float *x, size_t x_len,
                                    float *out);

/* ---- device-pointer entry points (asynchronous on `stream`, a hipStream_t or NULL) ----
 * Scratch memory (quantized activations, intermediates) is one library-owned buffer PER STREAM, held by
 * the calling thread while it enqueues a call's launches: calls on different streams never share
 * scratch, calls on one stream from several threads go out one after the other (as the reference's
 * rayon workers call the seam, gpu_backend.rs:722-725).  A buffer that is too small is replaced by a
 * larger one (a hipMalloc on the first call of a larger shape; the old one is retired behind an event
 * and reused, never given back to the driver by a call: nothing in these calls waits for the device).
 * HIP graphs: while a stream is being captured its buffer cannot grow -- run each shape once before
 * capturing it (a call that would need to grow returns FRK_ERR_HIP and launches nothing) -- and a
 * buffer that was current during a capture belongs to that graph from then on: a later, larger call
 * on the stream gets a new buffer and the old one stays allocated and untouched until the process
 * ends, so replays of the graph stay valid (at the price of that memory).  Callers that capture
 * without a warm call, or cannot have the library allocate at all, use frk_hip_gemm_noalloc_dev. */

/* y[rows] = W x for one activation vector in HBM.  K-quants: x is quantized to Q8_K
 * on the device first (bit-exact with quantize_activations_q8_k,
 * crates/frink-quant/src/act_quant.rs:69-104). */
int frk_hip_gemv_dev(const frk_weights *w, const float *x_dev, float *y_dev, int act_mode,
                     void *stream);

/* The same from activations the caller has already quantized to Q8_K (q[cols] i8, d[cols/256] f32,
 * bsums[cols/16] i16 in HBM), so projections that read one activation -- q/k/v, gate/up -- quantize
 * it once: the reference's shared MatvecInput (crates/frink-cuda/src/matvec_launch.rs:500-534) and
 * BatchActs::Q8K (crates/frink-core/src/weight_matrix.rs:757-768).  K-quants only. */
int frk_hip_gemv_q8k_dev(const frk_weights *w, const int8_t *q_dev, const float *d_dev,
                         const int16_t *bsums_dev, float *y_dev, void *stream);

/* The device forms of the two calls above: ys[i][ws[i]->rows] = ws[i] x for matrices of equal
 * column count (WeightMatrix::apply_gpu_multi, crates/frink-core/src/weight_matrix.rs:3504-3667), and
 * y[down->rows] = down(silu(gate x) * up x) (WeightMatrix::apply_gpu_dense_ffn_swiglu,
 * weight_matrix.rs:3676-3787; silu as crates/frink-core/src/matmul.rs:634-650). */
int frk_hip_gemv_multi_dev(const frk_weights *const *ws, size_t n, const float *x_dev,
                           float *const *ys_dev, void *stream);
int frk_hip_ffn_swiglu_dev(const frk_weights *gate, const frk_weights *up, const frk_weights *down,
                           const float *x_dev, float *y_dev, void *stream);

/* y[batch][rows] = x[batch][cols] W^T (WeightMatrix::apply_batch_with_acts,
 * crates/frink-core/src/weight_matrix.rs:2481).  Any batch >= 1.  Q4_K and Q6_K multiply Q8_K
 * activations at every batch size, and so does Q5_K (16 rows per launch of its batched kernel).  Q8_0 follows the reference's host: one row is the f32 dot of its
 * decode path (FRK_ACT_F32), two or more rows are quantized to Q8_0 activation blocks and multiplied
 * as integers (weight_matrix.rs:2701-2829, the arithmetic of FRK_ACT_Q8); Q4_0 does the same. */
int frk_hip_gemm_dev(const frk_weights *w, const float *x_dev, size_t batch, float *y_dev,
                     void *stream);

/* frk_hip_gemm_dev for a thin batch whose activations the caller (the kernel that produced them, or an earlier
 * call over the same batch) has already quantized to Q8_K: q [batch][cols] i8, d [batch][cols/256] f32,
 * bsums [batch][cols/16] i16, the layout frk_hip_quantize_q8_k_dev writes (BatchActs::Q8K,
 * crates/frink-core/src/weight_matrix.rs:757-768, handed to apply_batch_with_acts, :2481-2487).  Bit for bit
 * frk_hip_gemm_dev's result (one row: frk_hip_gemv_q8k_dev).  K-quants; the batches that frk_hip_gemm_dev multiplies on its thin kernels (up to 16
 * or 32 rows for Q4_K and up to 24 or 40 for Q6_K by the matrix's size, 32 for Q5_K): FRK_ERR_UNSUPPORTED beyond, where the
 * matrix-core GEMM quantizes into a tiled form of its own. */
int frk_hip_gemm_q8k_dev(const frk_weights *w, const int8_t *q_dev, const float *d_dev, const int16_t *bsums_dev,
                         size_t batch, float *y_dev, void *stream);

/* WeightMatrix::apply_batch_pair_with_acts (crates/frink-core/src/weight_matrix.rs:2447-2479) with
 * BatchActs::Q8K (:757-768): two matrices of one column count over ONE quantization of the batch -- gate
 * and up of a prefill FFN.  y0 and y1 are bit for bit what two frk_hip_gemm_dev calls give. */
int frk_hip_gemm_pair_dev(const frk_weights *w0, const frk_weights *w1, const float *x_dev, size_t batch,
                          float *y0_dev, float *y1_dev, void *stream);

/* A batch's activations quantized ONCE and multiplied by any number of matrices at ANY batch size:
 * WeightMatrix::quantize_batch_acts -> BatchActs::Q8K -> apply_batch_with_acts / apply_batch_pair_with_acts
 * (crates/frink-core/src/weight_matrix.rs:2348-2426, 757-768, 2481-2487, 2447-2479): the q/k/v triple or
 * gate and up of a prefill, or activations a caller keeps.  The object owns its device memory
 * (frk_hip_batch_acts_create allocates for up to max_batch rows of cols columns, _release frees; neither
 * belongs in a hot loop) and holds the batch in whichever form the kernels of that batch size read: plain
 * Q8_K rows (the decode and thin kernels), the tiled form of the matrix-core GEMMs, or both.
 * frk_hip_quantize_batch_acts_dev and frk_hip_gemm_acts_dev allocate nothing themselves (a GEMM whose
 * blocks are split between workgroups takes room for the parts from the stream's scratch buffer, like
 * frk_hip_gemm_dev); y is bit for bit frk_hip_gemm_dev's for two rows and more, and frk_hip_gemv_q8k_dev's for
 * one (which is frk_hip_gemv_dev's wherever both forms of the decode step are one kernel, and the same integers
 * added in another order for rows of more than 20 blocks).  K-quant matrices (Q4_K, Q5_K, Q6_K) of `cols`
 * columns; other kinds return FRK_ERR_UNSUPPORTED.  A quantization and the GEMMs that read it are ordered
 * by the stream they are enqueued on; the object is not to be re-quantized while a GEMM that reads it is
 * still in flight on another stream. */
typedef struct frk_batch_acts frk_batch_acts;
int frk_hip_batch_acts_create(size_t max_batch, size_t cols, frk_batch_acts **out);
int frk_hip_batch_acts_release(frk_batch_acts *acts);
int frk_hip_quantize_batch_acts_dev(frk_batch_acts *acts, const float *x_dev, size_t batch, void *stream);
int frk_hip_gemm_acts_dev(const frk_weights *w, const frk_batch_acts *acts, float *y_dev, void *stream);

/* frk_hip_gemm_dev for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, same
 * kernels and bit for bit the same y, but the scratch memory (quantized activations, the parts of a
 * split GEMM) is a fixed array of FRK_NOALLOC_SCRATCH_MIB MiB inside the library's device image, looked
 * up on the first call on a device; the call never allocates or frees.  A shape whose scratch does not
 * fit returns FRK_ERR_SHAPE and launches nothing (it fits every batch of up to 64 rows of matrices up to
 * 16384 columns, and prefill batches of 512 rows of 4096 columns that need no split).  Every call on a
 * GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race -- enqueue
 * them on one stream. */
#define FRK_NOALLOC_SCRATCH_MIB 16
int frk_hip_gemm_noalloc_dev(const frk_weights *w, const float *x_dev, size_t batch, float *y_dev,
                             void *stream);

/* frink_moe::route_top_k_softmax (crates/frink-moe/src/lib.rs:567-589) for a batch of tokens:
 * logits[batch][n_experts] -> ids[batch][k] (probability descending), weights[batch][k]
 * (probs[ids], divided by their sum when norm != 0).  Equal probabilities, which the reference's
 * unstable sort leaves undefined, resolve to the lower expert id. */
int frk_hip_route_top_k_softmax_dev(const float *logits_dev, size_t batch, size_t n_experts, size_t k,
                                    int norm, int32_t *ids_dev, float *weights_dev, void *stream);

/* Decoder::moe_ffn_batch (crates/frink-models/src/decoder/ffn_batch.rs:343-434) with SwiGLU experts
 * (frink_moe::run_expert, crates/frink-moe/src/lib.rs:1068-1165): out[batch][hidden] =
 * sum over each token's k routed experts of weights * down_e(silu(gate_e x) * up_e x), added in the
 * reference's order for a batch of this size: ascending expert id from 32 tokens on (its bucket path,
 * ffn_batch.rs:355), routing order below (the per-position path's combine_expert_outputs,
 * crates/frink-moe/src/lib.rs:1246-1263).  gate/up/down hold the experts stacked row-wise
 * (expert e = rows [e*ffn, (e+1)*ffn) of gate and up, [e*hidden, (e+1)*hidden) of down); gate and up
 * are Q4_K, down is Q4_K or Q6_K; or all three of Q5_0 / IQ4_XS / MXFP4 (gate and up of one kind): below 32 tokens
 * every (token, slot) pair runs on the integer decode kernel of its kind, from 32 on the pairs are bucketed by
 * expert and the experts, decoded to signed bytes in scratch memory, run on the grouped matrix-core kernel (an MXFP4
 * stack with scale bytes outside 104..143 keeps the per-pair jobs).  Other combinations: FRK_ERR_UNSUPPORTED.
 * ids[batch][k] / weights[batch][k] are a RoutingDecision per token (lib.rs:112-115); an id outside
 * [0, n_experts) contributes nothing. */
int frk_hip_moe_ffn_dev(const frk_weights *gate, const frk_weights *up, const frk_weights *down,
                        size_t n_experts, const float *x_dev, size_t batch, const int32_t *ids_dev,
                        const float *weights_dev, size_t k, float *out_dev, void *stream);

/* The grouped (indexed) GEMM on its own, for a caller with its own routing and activation:
 * enqueue_mul_mm_grouped_dev (crates/frink-cuda/src/mul_mm_launch.rs:391-470) and enqueue_mmq_grouped
 * (crates/frink-cuda/src/mmq/mod.rs:144-217).  Group g's matrix is rows [g*R, (g+1)*R) of `stacked` (R = rows /
 * n_groups; the reference's table[g], here one resident stack), Q4_K or Q6_K, or Q5_0 / IQ4_XS / MXFP4 with scale
 * bytes within 104..143 (decoded to signed bytes per call); others: FRK_ERR_UNSUPPORTED;
 * group_off_dev[n_groups + 1] are non-decreasing pair indices from 0 to pairs; pair p of group g reads activation
 * row gather_dev[p] of x_dev[x_rows][cols] (row p when gather_dev is null) and writes y_dev[p][R] -- every pair of
 * every group, no gaps.  Everything is read on the device, so the call can follow the kernel that built the
 * lists without a host round trip; the activation rows are quantized once each, to Q8_K or (Q5_0, MXFP4) to
 * Q8_0 blocks, as the reference's integer tier does.  n_groups <= 1024.  Offsets out of order or gather entries outside x are clamped, not
 * trusted. */
int frk_hip_gemm_grouped_dev(const frk_weights *stacked, size_t n_groups, const int32_t *group_off_dev,
                             const int32_t *gather_dev, const float *x_dev, size_t x_rows, size_t pairs, float *y_dev,
                             void *stream);

/* Test hooks for the bit-exact gates. */
/* What the last frk_hip_moe_ffn_dev call of this shape on this stream left behind in the stream's
 * scratch buffer (valid only if no other call on that stream came between), copied out
 * (null = skip): the gate and up projections [batch*k][ffn], silu(gate)*up quantized to Q8_K
 * (act_q [batch*k][ffn] i8, act_d [batch*k][ffn/256] f32), rows in grouped order, and
 * pos_of[tok*k + slot] = the row of a (token, slot) pair (the reference's bucket order,
 * crates/frink-models/src/decoder/ffn_batch.rs:362-386).  FRK_ERR_UNSUPPORTED for the small batches
 * (at most 16 tokens) that run per (token, slot) pair on the decode kernels: they have no grouped order. */
int frk_hip_moe_intermediates_dev(size_t batch, size_t k, size_t n_experts, size_t hidden, size_t ffn,
                                  float *gate_out_dev, float *up_out_dev, int8_t *act_q_dev,
                                  float *act_d_dev, int32_t *pos_of_dev, void *stream);
/* quantize_activations_q8_k over n = 256*k values: q[n] i8, d[n/256] f32, bsums[n/16] i16 */
int frk_hip_quantize_q8_k_dev(const float *x_dev, size_t n, int8_t *q_dev, float *d_dev,
                              int16_t *bsums_dev, void *stream);
/* quantize_activations_q8 (Avx form) over n = 32*k values: q[n] i8, d[n/32] f32 */
int frk_hip_quantize_q8_0_dev(const float *x_dev, size_t n, int8_t *q_dev, float *d_dev,
                              void *stream);
/* dequant_q8_0 / dequant_q4_k / dequant_q6_k (crates/frink-quant/src/lib.rs:271-286, 334-364,
 * 519-552; dequant_q5_k :424-459, dequant_q4_0 :291-310) from the resident (possibly permuted)
 * copy: out[rows*cols] f32. */
int frk_hip_dequant_dev(const frk_weights *w, float *out_dev, void *stream);
/* The embedding gather (get_rows, crates/frink-cuda/src/get_rows.rs:1-60; WeightMatrix::dequant_row):
 * out[n_ids][cols] f32, row r the dequantized row ids[r] of the table, bit for bit what the
 * dequantizer gives.  The host form checks every id against the table and returns FRK_ERR_SHAPE for
 * one outside it, as the reference validates before a launch; the device form cannot, and reads the
 * nearest row for such an id. */
int frk_hip_get_rows_dev(const frk_weights *w, const int32_t *ids_dev, size_t n_ids, float *out_dev,
                         void *stream);
int frk_hip_get_rows(const frk_weights *w, const int32_t *ids_host, size_t n_ids, float *out_host);

/* Plain device copy of `bytes` (multiple of 16), used to calibrate HBM counters and as the
 * practical bandwidth ceiling a streaming kernel of the same size can reach. */
int frk_hip_copy_dev(const void *src_dev, void *dst_dev, size_t bytes, void *stream);
/* Read-only stream over `bytes` (multiple of 16): every 16-byte word is loaded and nothing is
 * written -- a thread stores into sink_dev (>= 64 KiB) only if its words fold to one particular
 * value, which is there to keep the loads alive. */
int frk_hip_read_dev(const void *src_dev, size_t bytes, void *sink_dev, void *stream);
/* Calibration of the matrix-core kernels' issue budget (no counterpart in the reference; synchronous, allocates,
 * not for a hot loop).  Four launches of a loop of dependent v_mfma_i32_32x32x32_i8 with 0, 4, 8 and 12 independent
 * vector instructions behind each MFMA, two wavefronts per SIMD; per launch four floats: shader cycles per MFMA and
 * SIMD (the launch's duration at the clock measured in it), the shader clock in MHz during the loop (cycle counter
 * against the constant 100 MHz counter), microseconds of the launch, and the share of the launch that the first
 * wavefront's own loop took. */
int frk_hip_issue_probe(float *out16_host);
/* Calibration of the decode kernels' fetch shape (no counterpart in the reference).  Reads the first
 * floor(bytes / span) spans of the buffer and writes nothing: every wavefront owns one contiguous span of span_kb KB
 * (2, 4, 9 or 18) and issues all its 16-byte loads before it waits; waves_per_group 1..16; to_lds 0 = into registers,
 * 1 = copied straight into LDS (global_load_lds); policy = cache bits on the loads (0 none, 1 nt, 2 sc1, 3 sc0 sc1).
 * sink_dev as for frk_hip_read_dev. */
int frk_hip_read_shape_dev(const void *src_dev, size_t bytes, void *sink_dev, int span_kb, int waves_per_group,
                           int to_lds, int policy, void *stream);

#ifdef __cplusplus
}
#endif
#endif
