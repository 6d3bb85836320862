// Shared internals of libfrink_hip: error plumbing, the weights handle, kernel launchers.
#pragma once

#include <atomic>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "../../include/frink_hip.h"

namespace frk {

// ---- errors ----
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

#define FRK_HIP_TRY(expr)                                                                     \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess)                                                                 \
            return frk::set_error(e_ == hipErrorOutOfMemory ? FRK_ERR_OOM : FRK_ERR_HIP,      \
                                  "%s failed: %s", #expr, hipGetErrorString(e_));             \
    } while (0)

// ---- block geometry ----
constexpr int QK_K = 256;
constexpr int Q8_0_BYTES = 34, Q8_0_ELEMS = 32;
constexpr int Q4_0_BYTES = 18;  // 32 weights, like Q8_0
constexpr int Q4_K_BYTES = 144;
constexpr int Q5_K_BYTES = 176;
constexpr int Q6_K_BYTES = 210;
constexpr int Q5_0_BYTES = 22, IQ4_XS_BYTES = 136, MXFP4_BYTES = 17;  // 32, 256 and 32 weights

inline int block_bytes(int kind) {
    return kind == FRK_KIND_Q8_0 ? Q8_0_BYTES : kind == FRK_KIND_Q4_0 ? Q4_0_BYTES : kind == FRK_KIND_Q4_K ? Q4_K_BYTES
         : kind == FRK_KIND_Q5_K ? Q5_K_BYTES : kind == FRK_KIND_Q6_K ? Q6_K_BYTES : kind == FRK_KIND_Q5_0 ? Q5_0_BYTES
         : kind == FRK_KIND_IQ4_XS ? IQ4_XS_BYTES : kind == FRK_KIND_MXFP4 ? MXFP4_BYTES : 0;
}
inline int block_elems(int kind) {
    return (kind == FRK_KIND_Q8_0 || kind == FRK_KIND_Q4_0 || kind == FRK_KIND_Q5_0 || kind == FRK_KIND_MXFP4) ? Q8_0_ELEMS
         : (kind == FRK_KIND_Q4_K || kind == FRK_KIND_Q5_K || kind == FRK_KIND_Q6_K || kind == FRK_KIND_IQ4_XS) ? QK_K : 0;
}

// ---- resident layouts ----
// Q4_K stays verbatim: a 144-byte block is nine 16-byte words (header + 8 words of nibbles)
// and every row starts 16-byte aligned.  So does Q5_K: 176 bytes are eleven words (header, two of
// fifth bits, eight of nibbles).
// Q6_K (210-byte blocks, 2-byte aligned) and Q8_0 (34-byte blocks) are permuted per row into
// planes so every load is a 16-byte word:
//   Q6_K row of nb blocks: ql[nb][128] | qh[nb][64] | sc[nb][16] | d[nb] f16, padded to 16
//   Q8_0 row of nb blocks: qs[nb][32] | d[nb] f16, padded to 16
//   Q4_0 row of nb blocks (18-byte blocks): qs[nb][16] | d[nb] f16, padded to 16
// Same bytes, same count per block; only their order changes.
struct Layout {
    size_t row_stride = 0;  // bytes between resident rows
    size_t off_a = 0;       // Q6_K: qh plane offset in a row; Q8_0, Q4_0: d plane offset
    size_t off_b = 0;       // Q6_K: sc plane offset
    size_t off_c = 0;       // Q6_K: d plane offset
};

inline size_t round_up(size_t v, size_t m) { return (v + m - 1) / m * m; }

inline Layout layout_for(int kind, size_t cols) {
    Layout l;
    size_t nb = cols / (size_t)block_elems(kind);
    if (kind == FRK_KIND_Q4_K) {
        l.row_stride = nb * Q4_K_BYTES;
    } else if (kind == FRK_KIND_Q5_K) {
        l.row_stride = nb * Q5_K_BYTES;
    } else if (kind == FRK_KIND_Q6_K) {
        l.off_a = nb * 128;
        l.off_b = l.off_a + nb * 64;
        l.off_c = l.off_b + nb * 16;
        // rows start on a cache line where that costs under 2 % (the ql and qh planes then do too: a wavefront's
        // share of them is whole lines), else 16-byte aligned
        const size_t raw = l.off_c + nb * 2, lines = round_up(raw, 128);
        l.row_stride = (lines - raw) * 50 < raw ? lines : round_up(raw, 16);
    } else if (kind == FRK_KIND_Q8_0) {
        l.off_a = nb * 32;
        l.row_stride = round_up(l.off_a + nb * 2, 16);
    } else if (kind == FRK_KIND_Q4_0) {
        l.off_a = nb * 16;
        l.row_stride = round_up(l.off_a + nb * 2, 16);
    } else {  // Q5_0, IQ4_XS, MXFP4: the GGUF bytes in place, rows 16-byte aligned
        l.row_stride = round_up(nb * (size_t)block_bytes(kind), 16);
    }
    return l;
}

}  // namespace frk

// The handle behind frk_weights.
struct frk_weights {
    int kind = 0;
    size_t rows = 0, cols = 0;
    size_t src_row_bytes = 0;  // GGUF bytes per row
    frk::Layout layout;
    uint8_t *dev = nullptr;    // resident copy (library-owned)
    size_t dev_bytes = 0;
    int device = 0;
    // residency-cache identity (host pointer, length, sampled bytes)
    const void *host_key = nullptr;
    size_t host_len = 0;
    uint8_t fingerprint[192] = {0};
    int refcount = 1;
    bool cached = false;
    // MXFP4: the range of the E8M0 scale bytes (the batched integer path needs them to be f16 values)
    int e8m0_min = 0, e8m0_max = 255;
    // Q5_0 / IQ4_XS / MXFP4: the rows decoded to signed bytes for the matrix cores, kept beside the resident copy
    // on request (frk_hip_weights_keep_decoded); without it every batched call decodes into its scratch memory
    // (written once, under the registry's lock and behind a stream synchronization; read by calls on any thread)
    std::atomic<uint8_t *> decoded{nullptr};
};

namespace frk {

// ---- scratch the library owns (quantized activations, intermediates) ----
// One buffer per caller stream.  A lease holds the stream's buffer for as long as one entry point is
// enqueueing its launches (a recursive lock: entry points call each other), so calls made on one stream
// from several threads go out whole, one after the other, and stream order keeps their use of the buffer
// apart; calls on different streams have different buffers.  A buffer that is too small is replaced, never
// freed in place: the old one is kept until the outermost lease ends, then retired behind an event on the
// stream and handed out again (to any stream) once that event has passed.  A stream that is being captured
// cannot grow its buffer (the caller runs the shape once before capturing).
struct StreamWorkspace;
class WorkspaceLease {
  public:
    WorkspaceLease() = default;
    ~WorkspaceLease();
    WorkspaceLease(const WorkspaceLease &) = delete;
    WorkspaceLease &operator=(const WorkspaceLease &) = delete;
    void *ptr = nullptr;

  private:
    friend int workspace(size_t, hipStream_t, WorkspaceLease &);
    StreamWorkspace *held_ = nullptr;
    hipStream_t stream_ = nullptr;
};
// Leases at least `bytes` of the stream's buffer (the same start address for nested leases).
int workspace(size_t bytes, hipStream_t stream, WorkspaceLease &lease);
hipStream_t own_stream();  // the stream host-buffer entry points run on

// ---- launchers (each validates nothing: callers have checked shapes) ----
int launch_quantize_q8_k(const float *x, size_t n, int8_t *q, float *d, int16_t *bsums, hipStream_t s);
int launch_swiglu_quantize_q8_k(const float *gate, const float *up, size_t n, int8_t *q, float *d, int16_t *bsums, hipStream_t s);
int launch_swiglu_quantize_q8_0(const float *gate, const float *up, size_t n, int8_t *q, float *d, hipStream_t s);
int launch_quantize_q8_0(const float *x, size_t n, int8_t *q, float *d, hipStream_t s);
int launch_dequant(const frk_weights *w, float *out, hipStream_t s);
int launch_dequant_rows(const frk_weights *w, const int32_t *ids, size_t n_out, float *out, hipStream_t s);
int launch_repack(int kind, const uint8_t *src, uint8_t *dst, size_t rows, size_t cols, const Layout &l,
                  hipStream_t s);
int launch_copy(const void *src, void *dst, size_t bytes, hipStream_t s);
int launch_read(const void *src, size_t bytes, void *sink, hipStream_t s);
// calibration of the matrix-core kernels' issue budget (frk_probe.hip): 16 floats, four per count of vector instructions
int launch_issue_probe(float *out, hipStream_t s);
int launch_read_shape(const void *src, size_t bytes, void *sink, int span_kb, int waves, int to_lds, int policy, hipStream_t s);

struct Q8KActs {  // Q8_K activations in HBM, struct-of-arrays per activation row
    const int8_t *q;      // [batch][cols]
    const float *d;       // [batch][cols/256]
    const int16_t *bsums; // [batch][cols/16]
};
int launch_gemv_q4_k(const frk_weights *w, Q8KActs a, float *y, hipStream_t s);
int launch_gemv_q5_k(const frk_weights *w, Q8KActs a, float *y, hipStream_t s);
// Q5_K rows of 2048 / 4096 / 8192 / 16384 columns stored back to back: the whole-cache-line kernel, with the
// activation's quantization inside the launch or from Q8_K activations (frk_gemv_fused.hip)
bool q5_k_lines_gemv_fits(const frk_weights *w);
// Q4_K / Q5_K rows of any block count up to 64 stored back to back: whole rows to a wavefront
bool rows_gemv_fits(const frk_weights *w);
// which form a decode GEMV of the matrix takes on that kernel: none (the other kernels are ahead), one launch
// with the quantization inside, or a quantization launch and the kernel over Q8_K activations
enum { ROWS_FORM_NONE = 0, ROWS_FORM_ONE_LAUNCH = 1, ROWS_FORM_QUANTIZED = 2, ROWS_FORM_COLUMNS = 3 };
int launch_gemv_q4_k_cols(const frk_weights *w, const float *x, float *y, hipStream_t s);
int rows_gemv_form(const frk_weights *w);
bool rows_gemv_takes_quantized(const frk_weights *w);
int launch_gemv_rows_fused(const frk_weights *w, const float *x, float *y, hipStream_t s);
int launch_gemv_rows_preq(const frk_weights *w, Q8KActs a, float *y, hipStream_t s);
int launch_gemv_q5_k_fused(const frk_weights *w, const float *x, float *y, hipStream_t s);
int launch_gemv_q5_k_preq(const frk_weights *w, Q8KActs a, float *y, hipStream_t s);
int launch_gemv_q6_k(const frk_weights *w, Q8KActs a, float *y, hipStream_t s);
// one-launch kernels (activation quantized inside the GEMV); cols <= 16384
// rows of at most this many columns have a one-launch Q4_K GEMV
constexpr size_t FUSED_GEMV_MAX_COLS = 16384;
bool fused_gemv_fits(const frk_weights *w);
int launch_gemv_q4_k_fused(const frk_weights *w, const float *x, float *y, hipStream_t s);
int launch_gemv_q4_k_preq(const frk_weights *w, Q8KActs a, float *y, hipStream_t s);
// gate and up in one launch: act[r] = silu(gate[r] . x) * (up[r] . x) (both Q4_K, one shape, fused_gemv_fits)
int launch_gemv_q4_k_group(const frk_weights *const *ws, size_t n, const float *x, float *const *ys, hipStream_t s);
int launch_gemv_q4_k_experts(const frk_weights *w, const frk_weights *w2, int n_experts, size_t rows_e, const float *x,
                             size_t x_stride, const int32_t *ids, size_t jobs, size_t per_job, float *y, hipStream_t s);
int launch_gemv_q4_k_glu(const frk_weights *gate, const frk_weights *up, const float *x, float *act, hipStream_t s);
// Q8_K activations in the form the matrix-core GEMMs stream: rows in tiles of 32 and, per
// (tile, 256-wide block kb), one record that is exactly what a workgroup copies into LDS:
//   q  [tile][kb][8 slices of 32 k][2 halves of 16 k][32 rows][16 bytes]
//   bs [tile][kb][2 halves of 8 groups][32 rows][8]     the 16-wide sums as f16 (exact: |sum| <= 2032)
//   d  [tile][kb][32 rows]
// Rows past the last one of a partly used tile hold zeros.
struct Q8KTiled {
    int8_t *q;
    _Float16 *bs;
    float *d;
};
// Q8_K of plain rows, each quantized once: q [row][cols], bs [row][block][16] (the 16-wide sums as f16),
// d [row][block]
struct Q8KRows {
    int8_t *q;
    _Float16 *bs;
    float *d;
};
size_t q8k_tiled_bytes(size_t rows, size_t cols);
Q8KTiled q8k_tiled_carve(void *base, size_t rows, size_t cols);
// out row r = x[r] quantized, r < rows; the rest of the last tile becomes zeros
int launch_quantize_q8_k_tiled(const float *x, size_t rows, size_t cols, Q8KTiled out, hipStream_t s);
// out row r = x[gather[r]] quantized (zeros where gather[r] < 0), for the 32-row records of the first
// max_rows rows whose first entry is not negative
int launch_quantize_q8_k_gather(const float *x, size_t cols, const int *gather, size_t max_rows, Q8KTiled out,
                                hipStream_t s);
// batched GEMM on the int8 matrix cores (Q4_K, and Q5_K with q5 set: its fifth bits are a third plane of
// the same kernel); ws must hold gemm_q4_k_workspace_bytes(M, cols, rows, kind is Q5_K)
size_t gemm_q4_k_workspace_bytes(size_t M, size_t cols, size_t rows, bool q5 = false);
int launch_gemm_q4_k(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s);
// the same over activations already quantized into the tiled form; `partial` holds the parts' sums of a split
int launch_gemm_q4_k_acts(const frk_weights *w, Q8KTiled acts, size_t M, float *y, float *partial, hipStream_t s);
// the same for Q6_K (frk_gemm_q6.hip)
size_t gemm_q6_k_workspace_bytes(size_t M, size_t cols, size_t rows);
int launch_gemm_q6_k(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s);
int launch_gemm_q6_k_acts(const frk_weights *w, Q8KTiled acts, size_t M, float *y, float *partial, hipStream_t s);
// its grouped (per-expert) form: tile t = rows [64*t, 64*t+64) of the activations and of y, tiles[t] =
// {expert, 64*t, rows in use, 0}, tiles past *n_tiles idle; expert e owns rows [e*rows_e, (e+1)*rows_e) of w
int launch_gemm_q6_k_grouped(const frk_weights *w, size_t rows_e, Q8KTiled a, const int4 *tiles, const int *n_tiles,
                             int max_tiles, float *y, hipStream_t s);
// and for Q8_0 (frk_gemm_q8.hip), over activations quantized 32 at a time
size_t gemm_q8_0_workspace_bytes(size_t M, size_t cols, size_t rows);
// y[n] = partial[0][n] + partial[1][n] + ... in that order (the split GEMMs' second step; frk_gemm_q6.hip)
int launch_sum_parts(const float *partial, int parts, size_t n, float *y, hipStream_t s);
int launch_gemm_q8_0(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s);
int launch_gemm_q8_0_planar(const uint8_t *W, size_t row_stride, size_t off_d, size_t rows, size_t cols, bool q4, const float *x,
                            size_t M, float *y, void *ws, hipStream_t s);
// IQ4_XS on the matrix cores: the rows decoded to signed bytes with their block scales (launch_iq4_xs_to_sub_planar,
// rows of layout_for(FRK_KIND_Q8_0, cols)'s stride) against Q8_K activations
int launch_iq4_xs_to_sub_planar(const frk_weights *w, uint8_t *dst, size_t dst_stride, size_t off_d, hipStream_t s);
size_t gemm_sub_partial_bytes(size_t M, size_t cols, size_t rows);
// the grouped form over decoded rows of either form, and the Q8_0 activation blocks it reads
int launch_gemm_planar_grouped(const uint8_t *W, size_t row_stride, size_t off_d, size_t rows_g, size_t cols, bool sub,
                               const int8_t *aq, const void *ad, const int *src_rows, const int4 *tiles, const int *n_tiles,
                               size_t max_tiles, float *y, hipStream_t s);
size_t q8_0_gemm_acts_bytes(size_t rows, size_t cols);
int launch_quantize_q8_0_gemm(const float *x, const float *up, size_t rows, size_t cols, int8_t *q, uint16_t *d, hipStream_t s);
// the grouped GEMM over groups of Q5_0 / IQ4_XS / MXFP4 matrices that have a decoded form for the matrix cores
bool units_have_planar_form(const frk_weights *w);
// that form: rows of layout_for(FRK_KIND_Q8_0, cols) -- signed bytes, then f16 scales per 32 (IQ4_XS: per block of
// 256 the eight integer block scales and the f16 d).  units_decoded: the kept copy, or the rows decoded into `room`.
size_t units_planar_bytes(size_t rows, size_t cols);
int launch_units_decode(const frk_weights *w, uint8_t *dst, hipStream_t s);
int units_decoded(const frk_weights *w, uint8_t *room, hipStream_t s, const uint8_t **out);
size_t grouped_units_workspace_bytes(size_t n_groups, size_t w_rows, size_t x_rows, size_t pairs, size_t cols);
int launch_gemm_grouped_units(const frk_weights *w, size_t n_groups, const int32_t *group_off, const int32_t *gather, const float *x,
                              size_t x_rows, size_t pairs, float *y, void *ws, hipStream_t s);
// MoE layer over Q5_0 / IQ4_XS / MXFP4 experts by bucket, on the matrix cores (32 tokens and more)
bool moe_units_takes_grouped_path(const frk_weights *gate, const frk_weights *up, const frk_weights *down, size_t batch);
size_t moe_units_grouped_workspace_bytes(size_t batch, int k, int n_experts, int hidden, int ffn);
int launch_moe_ffn_units_grouped(const frk_weights *gate, const frk_weights *up, const frk_weights *down, int n_experts,
                                 const float *x, size_t batch, const int32_t *ids, const float *weights, int k, float *out,
                                 void *ws, hipStream_t s);
int launch_gemm_sub_planar(const uint8_t *W, size_t row_stride, size_t off_d, size_t rows, size_t cols, const int8_t *aq,
                           const float *ad, size_t M, float *y, void *partial, hipStream_t s);
// grouped (per-expert) GEMM: tile t = rows [64*t, 64*t+64) of the activations and of y, described by
// tiles[t] = {expert, 64*t, rows in use, 0}; expert e owns rows [e*rows_e, (e+1)*rows_e) of the
// stacked matrices; *n_tiles <= max_tiles.  w1/y1 (nullable) is a second stacked matrix over the
// same activations.  (64 rows: an expert's weights are then fetched and unpacked once for up to 64
// of its rows; the second half of a tile costs nothing when it is not in use.)
constexpr int MOE_TILE = 64;
// Up to this many tokens the MoE layer runs per (token, slot) pair on the decode kernels.  Measured
// on the 128-expert, top-8, 2048/768 layer: 8 tokens 47 us against 94 us on the grouped path, 16
// tokens 79 against 123, 32 tokens 146 against 140.
constexpr size_t MOE_PER_TOKEN_MAX_BATCH = 16;
// From this many tokens on the reference buckets a batch by expert (ffn_batch.rs:355) and a token's experts
// add up in ascending expert id; smaller batches run per position and add up in routing order.
constexpr size_t MOE_BUCKET_ORDER_FROM = 32;
bool moe_takes_per_token_path(size_t batch, size_t hidden, size_t ffn, int down_kind);
// The grouped Q4_K GEMM over the tile list (one matrix, or two that share the activations).  The activations
// are `a`, quantized in the grouped order, or -- with `src` -- the source rows' Q8_K and `gather`, the source
// row of every row of the grouped order (gemm_q4_k_stream_gathers tells whether the kernel can address them).
bool gemm_q4_k_stream_gathers(size_t src_rows, size_t cols);
int launch_gemm_q4_k_stream(const frk_weights *w0, const frk_weights *w1, size_t rows_e, Q8KTiled a,
                            const Q8KRows *src, const int *gather, const int4 *tiles, const int *n_tiles,
                            int max_tiles, float *y0, float *y1, hipStream_t s);
// The grouped GEMM over groups the caller lists (Q4_K or Q6_K weights stacked group by group): y[p] = W[group of
// p] . x[gather ? gather[p] : p]; ws must hold grouped_gemm_workspace_bytes(...)
size_t grouped_gemm_workspace_bytes(size_t n_groups, size_t x_rows, size_t pairs, size_t cols);
int launch_gemm_grouped(const frk_weights *w, size_t n_groups, const int32_t *group_off, const int32_t *gather,
                        const float *x, size_t x_rows, size_t pairs, float *y, void *ws, hipStream_t s);
// MoE expert FFN over stacked Q4_K experts; ws must hold moe_workspace_bytes(...)
size_t moe_workspace_bytes(size_t batch, int k, int n_experts, int hidden, int ffn);
int launch_moe_ffn(const frk_weights *gate, const frk_weights *up, const frk_weights *down, int n_experts,
                   const float *x, size_t batch, const int32_t *ids, const float *weights, int k, float *out,
                   void *ws, hipStream_t s);
int moe_copy_intermediates(void *ws, size_t batch, int k, int n_experts, int hidden, int ffn, float *gate_out,
                           float *up_out, int8_t *act_q, float *act_d, int32_t *pos_of, hipStream_t s);
int launch_swiglu(const float *gate, const float *up, size_t n, float *act, hipStream_t s);
int launch_route_top_k_softmax(const float *logits, int batch, int n_experts, int k, int norm, int32_t *ids,
                               float *weights, hipStream_t s);
// prefetch-all GEMVs (one wavefront per row, no LDS) for rows of 33..256 units
bool direct_gemv_fits(const frk_weights *w);
bool q4_0_cols_form(const frk_weights *w);
int launch_gemv_q4_0_f32_cols(const frk_weights *w, const float *x, float *y, hipStream_t s);
bool q6_k_cols_form(const frk_weights *w);  // the one-launch Q6_K GEMV whose wavefronts split the columns
int launch_gemv_q6_k_direct(const frk_weights *w, Q8KActs a, float *y, hipStream_t s);
int launch_gemv_q6_k_fused(const frk_weights *w, const float *x, float *y, hipStream_t s);
// Q5_0, IQ4_XS, MXFP4: dequantizer / row gather and the f32-dot decode GEMV
bool is_unit_kind(int kind);
// the integer tier of Q5_0 / MXFP4 (Q8_0 activation blocks) and IQ4_XS (Q8_K quants and block scales)
bool gemv_units_int_fits(const frk_weights *w);
int launch_gemv_units_int(const frk_weights *w, const int8_t *aq, const float *ad, float *y, hipStream_t s);
int launch_gemv_units_int_jobs(const frk_weights *w, const frk_weights *w2, size_t rows_e, int n_experts, const int32_t *ids,
                               size_t n_jobs, int act_div, const int8_t *aq, const float *ad, float *y, float *y2, hipStream_t s);
// the routed layer over experts of these kinds: every (token, slot) pair a job of the integer decode kernel
size_t moe_units_workspace_bytes(size_t batch, int k, int hidden, int ffn);
int launch_moe_ffn_units(const frk_weights *gate, const frk_weights *up, const frk_weights *down, int n_experts, const float *x,
                         size_t batch, const int32_t *ids, const float *weights, int k, float *out, void *ws, hipStream_t s);
// Q5_0 / MXFP4 rows decoded into the Q8_0 planar form (signed bytes and f16 scales; `dst` rows dst_stride apart, the
// scales at off_d): what the batched integer path multiplies.  MXFP4 scales must be f16 values (mxfp4_scale_range).
int launch_units_to_q8_0_planar(const frk_weights *w, uint8_t *dst, size_t dst_stride, size_t off_d, hipStream_t s);
// the smallest and largest E8M0 scale byte of an MXFP4 matrix (synchronous; at registration)
int mxfp4_scale_range(const frk_weights *w, int *e_min, int *e_max, hipStream_t s);
int launch_dequant_units(const frk_weights *w, const int32_t *ids, size_t n_out, float *out, hipStream_t s);
int launch_gemv_units_f32(const frk_weights *w, const float *x, float *y, hipStream_t s);
// K-quant GEMV on dequantized weights and the f32 activation (the reference's default x86 decode numerics)
bool kquant_f32_gemv_fits(const frk_weights *w);
int launch_gemv_kquant_f32(const frk_weights *w, const float *x, float *y, hipStream_t s);
// Q6_K experts stacked in w, one job per (token, slot): y[j][rows_e] = expert ids[j] times x + j * x_stride
bool q6_k_experts_gemv_fits(const frk_weights *w);
int launch_gemv_q6_k_experts(const frk_weights *w, int n_experts, size_t rows_e, const float *x, size_t x_stride,
                             const int32_t *ids, size_t jobs, float *y, hipStream_t s);
int launch_gemv_q8_0_f32_direct(const frk_weights *w, const float *x, float *y, hipStream_t s);
// thin batched GEMM of the K-quants: 1 <= batch <= thin_gemm_max_batch(w) rows per launch (0: does not fit)
int thin_gemm_max_batch(const frk_weights *w);
int thin_gemm_wide_rows(const frk_weights *w);
int launch_thin_gemm_wide(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s);
int launch_thin_gemm(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s);
int launch_gemv_q8_0_f32(const frk_weights *w, const float *x, float *y, hipStream_t s);
int launch_gemv_q8_0_q8(const frk_weights *w, const int8_t *q, const float *d, float *y, hipStream_t s);
int launch_gemv_q4_0_f32(const frk_weights *w, const float *x, float *y, hipStream_t s);
int launch_gemv_q4_0_q8(const frk_weights *w, const int8_t *q, const float *d, float *y, hipStream_t s);

}  // namespace frk
