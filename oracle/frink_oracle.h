/*
 * frink_oracle.h -- CPU restatement of Frink's quantized-matmul arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is
 * compared against and the CPU baseline that is timed beside it.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * Every function follows one function of the reference (file:line given in
 * frink_oracle.c), operation for operation: no floating-point contraction
 * (build with -ffp-contract=off), fmaf() exactly where the reference writes
 * mul_add, the same summation order.
 */
#ifndef FRINK_ORACLE_H
#define FRINK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* quant kinds; the numbers are the ggml type ids the reference maps from
 * (crates/frink-gguf/src/lib.rs:236-242). */
enum { FO_KIND_Q4_0 = 2, FO_KIND_Q5_0 = 6, FO_KIND_Q8_0 = 8, FO_KIND_Q4_K = 12, FO_KIND_Q5_K = 13, FO_KIND_Q6_K = 14,
       FO_KIND_IQ4_XS = 23, FO_KIND_MXFP4 = 39 };

/* Q8_0 activation forms (crates/frink-quant/src/act_quant.rs:121-127). */
enum { FO_Q8_0_FORM_NEON = 0, FO_Q8_0_FORM_AVX = 1, FO_Q8_0_FORM_SCALAR = 2 };

/* matvec / GEMM arithmetic tiers */
enum { FO_MODE_F32_DOT = 0, FO_MODE_INT_DOT = 1 };

int fo_block_bytes(int kind);
int fo_block_elems(int kind);

float    fo_f16_to_f32(uint16_t h);
uint16_t fo_f32_to_f16(float f);

/* dequantizers: return 0, or -1 when nbytes is not a whole number of blocks */
int fo_dequant_q8_0(const uint8_t *src, size_t nbytes, float *out);
int fo_dequant_q4_0(const uint8_t *src, size_t nbytes, float *out);
int fo_dequant_q4_k(const uint8_t *src, size_t nbytes, float *out);
int fo_dequant_q5_k(const uint8_t *src, size_t nbytes, float *out);
int fo_dequant_q6_k(const uint8_t *src, size_t nbytes, float *out);
int fo_dequant_q5_0(const uint8_t *src, size_t nbytes, float *out);
int fo_dequant_iq4_xs(const uint8_t *src, size_t nbytes, float *out);
int fo_dequant_mxfp4(const uint8_t *src, size_t nbytes, float *out); /* GGUF block form: [E8M0][16 nibble bytes] */
float fo_e8m0_scale(uint8_t e);
int fo_dequant(int kind, const uint8_t *src, size_t nbytes, float *out);
/* independent per-element decoders (index formula, not a block walk) */
float fo_q4_k_element(const uint8_t *block, int i);
float fo_q5_k_element(const uint8_t *block, int i);
float fo_q6_k_element(const uint8_t *block, int i);
void  fo_q4_k_scale_min(int j, const uint8_t *scales12, uint8_t *sc, uint8_t *m);

/* fused f32 dots (scalar twins) */
float fo_dot_q8_0_f32(const uint8_t *row, size_t row_bytes, const float *x);
float fo_dot_q4_0_f32(const uint8_t *row, size_t row_bytes, const float *x);
float fo_dot_q4_k_f32(const uint8_t *row, size_t row_bytes, const float *x);
float fo_dot_q5_k_f32(const uint8_t *row, size_t row_bytes, const float *x);
float fo_dot_q6_k_f32(const uint8_t *row, size_t row_bytes, const float *x);
float fo_dot_q5_0_f32(const uint8_t *row, size_t row_bytes, const float *x);
float fo_dot_iq4_xs_f32(const uint8_t *row, size_t row_bytes, const float *x);
float fo_dot_mxfp4_f32(const uint8_t *row, size_t row_bytes, const float *x);

/* activation quantizers */
void fo_quantize_q8_k(const float *x, size_t n, int8_t *q, float *d, int16_t *bsums);
void fo_quantize_q8_0(const float *x, size_t n, int form, int8_t *q, float *d);

/* integer dots against quantized activations */
float fo_dot_q8_0_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d);
float fo_dot_q4_0_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d);
/* legacy_q8.rs: Q5_0 and GGUF MXFP4 rows against Q8_0 activation blocks; the decoders and the halved E8M0 scale */
void fo_decode_q5_0_block(const uint8_t *blk, int8_t *w32);
void fo_decode_mxfp4_block(const uint8_t *blk, int8_t *w32);
float fo_e8m0_half_scale(uint8_t e);
float fo_dot_q5_0_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d);
float fo_dot_mxfp4_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d);
/* iq4_xs_q8.rs: IQ4_XS rows against Q8_K activations (q, d per 256; the 16-wide sums are not used) */
float fo_dot_iq4_xs_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *dact);
float fo_dot_q4_k_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d,
                      const int16_t *bsums);
float fo_dot_q5_k_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d,
                      const int16_t *bsums);
float fo_dot_q6_k_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d);

/* weight encoders; n must be a whole number of blocks (else -1) */
int   fo_nearest_int(float f);
float fo_make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *l,
                          float *the_min, uint8_t *laux, float rmin, float rdelta, int nstep,
                          int use_mad);
float fo_make_qx_quants(int n, int nmax, const float *x, int8_t *l, int rmse_type);
int fo_encode_row_q8_0(const float *src, size_t n, uint8_t *out);
int fo_encode_row_q4_k(const float *src, size_t n, uint8_t *out);
int fo_encode_row_q5_k(const float *src, size_t n, uint8_t *out);
int fo_encode_row_q6_k(const float *src, size_t n, uint8_t *out);
/* rows encoded in parallel; same bytes as calling the row encoder per row */
int fo_encode_matrix(int kind, const float *src, size_t rows, size_t cols, uint8_t *out,
                     int threads);

/* dispatch-level restatement: out[batch][rows], in[batch][cols] */
int fo_gemv(int kind, const uint8_t *w, size_t rows, size_t cols, const float *x, float *y,
            int mode, int threads);
int fo_gemm(int kind, const uint8_t *w, size_t rows, size_t cols, const float *x, size_t batch,
            float *y, int mode, int threads);
/* rows [row0, row0+nrows) only; y is [batch][nrows] */
int fo_gemm_rows(int kind, const uint8_t *w, size_t rows, size_t cols, size_t row0, size_t nrows,
                 const float *x, size_t batch, float *y, int mode, int threads);

/* MoE */
float fo_silu(float x);
void  fo_swiglu(const float *gate, const float *up, size_t n, float *out);
void  fo_route_top_k_softmax(const float *logits, int n_experts, int k, int norm_topk_prob,
                             int32_t *ids, float *weights);
void  fo_combine_expert_outputs(const float *const *expert_out, const float *weights, int n,
                                int hidden, float *out);
/* Prefill MoE layer: experts' gate/up are [ffn][hidden], down is [hidden][ffn],
 * each expert's three matrices contiguous at index e in their arrays. */
int fo_moe_ffn_batch(int kind, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                     int n_experts, int hidden, int ffn, const float *x, int batch,
                     const int32_t *ids, const float *weights, int k, float *out, int threads);

/* The same layer the way a batch below 32 tokens runs it: per position, slots in routing order. */
int fo_moe_ffn_per_position(int kind, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                            int n_experts, int hidden, int ffn, const float *x, int batch,
                            const int32_t *ids, const float *weights, int k, float *out, int threads);

/* CPU baseline: AVX2 dot where the host has it; returns 1 if AVX2 was used */
int fo_have_avx2(void);

/* The x86 forms the reference runs, for the timed CPU baseline only (cpu_baseline_avx2.c):
 * AVX2+FMA f32 decode dot and AVX2 integer dot (Q8_K activations, `batch` rows of them, weight row
 * outermost), rows over `threads` OpenMP threads.  -1 on a host without AVX2 and FMA. */
int fo_avx2_gemv_q4_k_f32(const uint8_t *w, size_t rows, size_t cols, const float *x, float *y, int threads);
int fo_avx2_gemm_q4_k_q8k(const uint8_t *w, size_t rows, size_t cols, const float *x, size_t batch, float *y,
                          int threads);

#ifdef __cplusplus
}
#endif
#endif
