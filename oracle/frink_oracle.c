/*
 * frink_oracle.c -- CPU restatement of Frink's quantized-matmul arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path and the timed CPU
 * baseline.  The shipped library never links, loads or calls this file.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp (see Makefile).
 * Rust never contracts a*b+c unless mul_add is written, so contraction must be
 * off here and fmaf() appears exactly where the reference writes mul_add.
 *
 * Reference paths are relative to the reference root, crate frink-quant unless
 * another crate is named.  What pins each function (the reference's own golden
 * vectors, closed forms, brute force) is listed in tests/test_oracle_*.py.
 *
 * Parity pinned by identity/tolerance rather than by a reference-emitted
 * vector ("parity unpinned" as exact f32 bit patterns): fo_dot_*_f32,
 * fo_dot_*_q8*, fo_gemv/fo_gemm, fo_moe_ffn_batch.  Their integer parts are
 * exact and their float order follows the source text; tests pin them to the
 * vector-pinned dequantizers through exact-arithmetic identities.
 */
#include "frink_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define Q8_0_BYTES 34
#define Q4_0_BYTES 18
#define Q8_0_ELEMS 32
#define Q4_K_BYTES 144
#define Q5_K_BYTES 176
#define Q6_K_BYTES 210
#define QK_K 256
#define Q5_0_BYTES 22
#define IQ4_XS_BYTES 136
#define MXFP4_BYTES 17

/* src/lib.rs:74-75, 180-182, 196-197 */
int fo_block_bytes(int kind) {
    switch (kind) {
    case FO_KIND_Q8_0: return Q8_0_BYTES;
    case FO_KIND_Q4_0: return Q4_0_BYTES;
    case FO_KIND_Q4_K: return Q4_K_BYTES;
    case FO_KIND_Q5_K: return Q5_K_BYTES;
    case FO_KIND_Q6_K: return Q6_K_BYTES;
    case FO_KIND_Q5_0: return Q5_0_BYTES;
    case FO_KIND_IQ4_XS: return IQ4_XS_BYTES;
    case FO_KIND_MXFP4: return MXFP4_BYTES;
    }
    return 0;
}
int fo_block_elems(int kind) {
    switch (kind) {
    case FO_KIND_Q8_0: case FO_KIND_Q4_0: case FO_KIND_Q5_0: case FO_KIND_MXFP4: return Q8_0_ELEMS;
    case FO_KIND_Q4_K: case FO_KIND_Q5_K: case FO_KIND_Q6_K: case FO_KIND_IQ4_XS: return QK_K;
    }
    return 0;
}

/* ---- IEEE binary16 <-> binary32 (the `half` crate's semantics: exact widening,
 * round-to-nearest-even narrowing; twins in frink-cuda/src/mul_mm.rs:258-280 and
 * frink-cuda/src/matvec_kinds/dp4a_twin.rs:36-61) ---- */
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float fo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: man * 2^-24, exact in f32 */
        float v = (float)man * 5.9604644775390625e-8f;
        return bits_f32(f32_bits(v) | sign);
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112) << 23) | (man << 13));
}

uint16_t fo_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        if (absx == 0x7f800000u) return sign | 0x7c00u;
        uint16_t m = (uint16_t)((absx >> 13) & 0x3ffu);
        return sign | 0x7c00u | (m ? m : 0x200u) | 0x200u;
    }
    if (absx >= 0x477ff000u) return sign | 0x7c00u; /* rounds to >= 2^16 -> inf */
    if (absx < 0x33000001u) return sign;             /* <= 2^-25 -> +-0 (tie to even) */
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7fffffu) | 0x800000u;
    if (e < -14) { /* subnormal result: value = m * 2^(e-23), target unit 2^-24 */
        int shift = (-14 - e) + 13;
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1))) q++;
        return sign | (uint16_t)q;
    }
    uint32_t q = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3ffu);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1))) q++;
    return sign | (uint16_t)q;
}

static inline float rd_f16(const uint8_t *p) { return fo_f16_to_f32((uint16_t)(p[0] | (p[1] << 8))); }
static inline void wr_f16(uint8_t *p, float f) { uint16_t h = fo_f32_to_f16(f); p[0] = h & 0xff; p[1] = h >> 8; }

/* ---- dequantizers ---- */

/* src/lib.rs:271-286 */
int fo_dequant_q8_0(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % Q8_0_BYTES) return -1;
    size_t nb = nbytes / Q8_0_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * Q8_0_BYTES;
        float scale = rd_f16(blk);
        for (int i = 0; i < 32; i++) out[b * 32 + i] = (float)(int8_t)blk[2 + i] * scale;
    }
    return 0;
}

/* src/lib.rs:321-330 */
void fo_q4_k_scale_min(int j, const uint8_t *s, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = s[j] & 63;
        *m = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4));
        *m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

/* src/lib.rs:291-310: block = [d:f16][16 bytes]; byte i holds element i in its low nibble and
 * element i + 16 in its high nibble; y = (nibble - 8) * d */
int fo_dequant_q4_0(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % Q4_0_BYTES) return -1;
    size_t nb = nbytes / Q4_0_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * Q4_0_BYTES;
        float scale = rd_f16(blk);
        for (int i = 0; i < 16; i++) {
            int lo = (int)(blk[2 + i] & 0x0F) - 8, hi = (int)(blk[2 + i] >> 4) - 8;
            out[b * 32 + i] = (float)lo * scale;
            out[b * 32 + i + 16] = (float)hi * scale;
        }
    }
    return 0;
}

/* src/lib.rs:334-364 */
int fo_dequant_q4_k(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % Q4_K_BYTES) return -1;
    size_t nb = nbytes / Q4_K_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * Q4_K_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        float *y = out + b * QK_K;
        int is = 0, q_off = 0;
        for (int p = 0; p < 4; p++) {
            uint8_t sc1, m1, sc2, m2;
            fo_q4_k_scale_min(is, scales, &sc1, &m1);
            fo_q4_k_scale_min(is + 1, scales, &sc2, &m2);
            float d1 = d * (float)sc1, min1 = dmin * (float)m1;
            float d2 = d * (float)sc2, min2 = dmin * (float)m2;
            for (int l = 0; l < 32; l++) *y++ = d1 * (float)(qs[q_off + l] & 0x0F) - min1;
            for (int l = 0; l < 32; l++) *y++ = d2 * (float)(qs[q_off + l] >> 4) - min2;
            q_off += 32;
            is += 2;
        }
    }
    return 0;
}

/* src/lib.rs:424-459: Q4_K's walk, each code's fifth bit from the qh plane (bytes 16..48), whose
 * byte l serves elements l, l+32, l+64, ... of the block through bits 0, 1, 2, ... */
int fo_dequant_q5_k(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % Q5_K_BYTES) return -1;
    size_t nb = nbytes / Q5_K_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * Q5_K_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
        float *y = out + b * QK_K;
        int is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int oi = 0; oi < 4; oi++) {
            uint8_t sc1, m1, sc2, m2;
            fo_q4_k_scale_min(is, scales, &sc1, &m1);
            fo_q4_k_scale_min(is + 1, scales, &sc2, &m2);
            float d1 = d * (float)sc1, min1 = dmin * (float)m1;
            float d2 = d * (float)sc2, min2 = dmin * (float)m2;
            const uint8_t *ql = qs + oi * 32;
            for (int l = 0; l < 32; l++) {
                uint8_t hi = (qh[l] & u1) ? 16 : 0;
                *y++ = d1 * (float)(uint8_t)((ql[l] & 0x0F) + hi) - min1;
            }
            for (int l = 0; l < 32; l++) {
                uint8_t hi = (qh[l] & u2) ? 16 : 0;
                *y++ = d2 * (float)(uint8_t)((ql[l] >> 4) + hi) - min2;
            }
            is += 2;
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
    return 0;
}

/* src/lib.rs:519-552 */
int fo_dequant_q6_k(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % Q6_K_BYTES) return -1;
    size_t nb = nbytes / Q6_K_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * Q6_K_BYTES;
        float d = rd_f16(blk + 208);
        for (int half = 0; half < 2; half++) {
            const uint8_t *ql = blk + half * 64, *qh = blk + 128 + half * 32;
            const int8_t *sc = (const int8_t *)(blk + 192 + half * 8);
            float *y = out + b * QK_K + half * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int8_t q1 = (int8_t)((ql[l] & 0x0F) | ((qh[l] & 3) << 4)) - 32;
                int8_t q2 = (int8_t)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int8_t q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l] = d * (float)sc[is] * (float)q1;
                y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                y[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
        }
    }
    return 0;
}

/* ---- Q5_0, IQ4_XS, MXFP4 (GGUF block form): dequantizers and f32 dots ---- */

/* src/lib.rs:4346-4350: the fifth bits of elements j and j + 16 of a Q5_0 block, at bit 4 */
static void q5_fifth_bits(uint32_t qh, int j, uint8_t *xh0, uint8_t *xh1) {
    *xh0 = (uint8_t)((qh >> j) << 4) & 0x10;
    *xh1 = (uint8_t)(qh >> (j + 12)) & 0x10;
}
/* src/lib.rs:4356-4376: block = [d:f16][qh:u32][16 bytes]; y = (q - 16) * d */
int fo_dequant_q5_0(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % Q5_0_BYTES) return -1;
    size_t nb = nbytes / Q5_0_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * Q5_0_BYTES;
        float d = rd_f16(blk);
        uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
        const uint8_t *qs = blk + 6;
        for (int j = 0; j < 16; j++) {
            uint8_t xh0, xh1;
            q5_fifth_bits(qh, j, &xh0, &xh1);
            int x0 = (int)((qs[j] & 0x0F) | xh0) - 16, x1 = (int)((qs[j] >> 4) | xh1) - 16;
            out[b * 32 + j] = (float)x0 * d;
            out[b * 32 + j + 16] = (float)x1 * d;
        }
    }
    return 0;
}
/* src/lib.rs:4396-4418 */
float fo_dot_q5_0_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / Q5_0_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q5_0_BYTES;
        float d = rd_f16(blk);
        uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
        const uint8_t *qs = blk + 6;
        for (int j = 0; j < 16; j++) {
            uint8_t xh0, xh1;
            q5_fifth_bits(qh, j, &xh0, &xh1);
            int x0 = (int)((qs[j] & 0x0F) | xh0) - 16, x1 = (int)((qs[j] >> 4) | xh1) - 16;
            acc += ((float)x0 * d) * x[b * 32 + j];
            acc += ((float)x1 * d) * x[b * 32 + j + 16];
        }
    }
    return acc;
}

/* src/lib.rs:4801-4803 (ggml's kvalues_iq4nl) */
static const int8_t KVALUES_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
/* src/lib.rs:4860-4890: block = [d:f16][scales_h:u16][scales_l:4][qs:128]; eight sub-blocks of 32, each with a
 * 6-bit scale ls: y = d * (ls - 32) * kvalues[nibble], low nibbles first then high */
int fo_dequant_iq4_xs(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % IQ4_XS_BYTES) return -1;
    size_t nb = nbytes / IQ4_XS_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * IQ4_XS_BYTES;
        float d = rd_f16(blk);
        unsigned scales_h = (unsigned)blk[2] | ((unsigned)blk[3] << 8);
        const uint8_t *scales_l = blk + 4, *qs = blk + 8;
        for (int ib = 0; ib < 8; ib++) {
            uint8_t ls = (uint8_t)(((scales_l[ib / 2] >> (4 * (ib % 2))) & 0xf) | (uint8_t)(((scales_h >> (2 * ib)) & 3) << 4));
            float dl = d * ((float)ls - 32.0f);
            for (int j = 0; j < 16; j++) {
                uint8_t byte = qs[ib * 16 + j];
                out[b * QK_K + ib * 32 + j] = dl * (float)KVALUES_IQ4NL[byte & 0xf];
                out[b * QK_K + ib * 32 + 16 + j] = dl * (float)KVALUES_IQ4NL[byte >> 4];
            }
        }
    }
    return 0;
}
/* src/lib.rs:4910-4934 */
float fo_dot_iq4_xs_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / IQ4_XS_BYTES;
    float acc = 0.0f;
    size_t x_base = 0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * IQ4_XS_BYTES;
        float d = rd_f16(blk);
        unsigned scales_h = (unsigned)blk[2] | ((unsigned)blk[3] << 8);
        const uint8_t *scales_l = blk + 4, *qs = blk + 8;
        for (int ib = 0; ib < 8; ib++) {
            uint8_t ls = (uint8_t)(((scales_l[ib / 2] >> (4 * (ib % 2))) & 0xf) | (uint8_t)(((scales_h >> (2 * ib)) & 3) << 4));
            float dl = d * ((float)ls - 32.0f);
            for (int j = 0; j < 16; j++) {
                uint8_t byte = qs[ib * 16 + j];
                acc += (dl * (float)KVALUES_IQ4NL[byte & 0xf]) * x[x_base + j];
                acc += (dl * (float)KVALUES_IQ4NL[byte >> 4]) * x[x_base + 16 + j];
            }
            x_base += 32;
        }
    }
    return acc;
}

/* src/lib.rs:4947-4949 (E2M1) and :4960-4966 (E8M0: 2^(e-127), e = 0 the subnormal 2^-127) */
static const float KVALUES_MXFP4[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                        -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
float fo_e8m0_scale(uint8_t e) {
    uint32_t bits = e == 0 ? 0x00400000u : (uint32_t)e << 23;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
/* GGUF block form, src/lib.rs:5560-5570: block = [e:E8M0][16 bytes], low nibble -> element j, high -> j + 16;
 * the arithmetic of dequant_mxfp4_row (:4980-5003) */
int fo_dequant_mxfp4(const uint8_t *src, size_t nbytes, float *out) {
    if (nbytes % MXFP4_BYTES) return -1;
    size_t nb = nbytes / MXFP4_BYTES;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = src + b * MXFP4_BYTES;
        float d = fo_e8m0_scale(blk[0]);
        for (int j = 0; j < 16; j++) {
            out[b * 32 + j] = d * KVALUES_MXFP4[blk[1 + j] & 0xf];
            out[b * 32 + 16 + j] = d * KVALUES_MXFP4[blk[1 + j] >> 4];
        }
    }
    return 0;
}
/* src/lib.rs:5025-5040, over GGUF blocks */
float fo_dot_mxfp4_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / MXFP4_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * MXFP4_BYTES;
        float d = fo_e8m0_scale(blk[0]);
        for (int j = 0; j < 16; j++) {
            acc += (d * KVALUES_MXFP4[blk[1 + j] & 0xf]) * x[b * 32 + j];
            acc += (d * KVALUES_MXFP4[blk[1 + j] >> 4]) * x[b * 32 + 16 + j];
        }
    }
    return acc;
}

int fo_dequant(int kind, const uint8_t *src, size_t nbytes, float *out) {
    switch (kind) {
    case FO_KIND_Q8_0: return fo_dequant_q8_0(src, nbytes, out);
    case FO_KIND_Q4_0: return fo_dequant_q4_0(src, nbytes, out);
    case FO_KIND_Q4_K: return fo_dequant_q4_k(src, nbytes, out);
    case FO_KIND_Q5_K: return fo_dequant_q5_k(src, nbytes, out);
    case FO_KIND_Q6_K: return fo_dequant_q6_k(src, nbytes, out);
    case FO_KIND_Q5_0: return fo_dequant_q5_0(src, nbytes, out);
    case FO_KIND_IQ4_XS: return fo_dequant_iq4_xs(src, nbytes, out);
    case FO_KIND_MXFP4: return fo_dequant_mxfp4(src, nbytes, out);
    }
    return -2;
}

/* Independent decoders: element i of one block from the published layout by
 * index arithmetic, written without reference to the block walks above so a
 * stride or pairing mistake in either shows up as a disagreement. */
float fo_q4_k_element(const uint8_t *blk, int i) {
    int sub = i >> 5;           /* 32-element sub-block */
    int within = i & 31;
    int byte = 16 + (sub >> 1) * 32 + within;
    int nib = (sub & 1) ? (blk[byte] >> 4) : (blk[byte] & 15);
    uint8_t sc, m;
    fo_q4_k_scale_min(sub, blk + 4, &sc, &m);
    float d = rd_f16(blk), dmin = rd_f16(blk + 2);
    return (d * (float)sc) * (float)nib - dmin * (float)m;
}
float fo_q5_k_element(const uint8_t *blk, int i) {
    int sub = i >> 5, within = i & 31;
    int byte = 48 + (sub >> 1) * 32 + within;
    int nib = (sub & 1) ? (blk[byte] >> 4) : (blk[byte] & 15);
    int fifth = (blk[16 + within] >> sub) & 1;  /* bit `sub` of qh[within] */
    uint8_t sc, m;
    fo_q4_k_scale_min(sub, blk + 4, &sc, &m);
    float d = rd_f16(blk), dmin = rd_f16(blk + 2);
    return (d * (float)sc) * (float)(nib + 16 * fifth) - dmin * (float)m;
}
float fo_q6_k_element(const uint8_t *blk, int i) {
    int half = i >> 7, r = i & 127, quarter = r >> 5, l = r & 31;
    int qlb = blk[half * 64 + (quarter & 1) * 32 + l];
    int lo = (quarter & 2) ? (qlb >> 4) : (qlb & 15);
    int hi = (blk[128 + half * 32 + l] >> (2 * quarter)) & 3;
    int q = (lo | (hi << 4)) - 32;
    int8_t sc = (int8_t)blk[192 + (i >> 4)];
    return rd_f16(blk + 208) * (float)sc * (float)q;
}

/* ---- fused f32 dots ---- */

/* src/lib.rs:663-686 */
float fo_dot_q8_0_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / Q8_0_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q8_0_BYTES;
        float scale = rd_f16(blk);
        float block_acc = 0.0f;
        for (int i = 0; i < 32; i++) block_acc += (float)(int8_t)blk[2 + i] * x[b * 32 + i];
        acc += block_acc * scale;
    }
    return acc;
}

/* src/lib.rs:4253-4276 */
float fo_dot_q4_0_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / Q4_0_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q4_0_BYTES;
        float scale = rd_f16(blk);
        float block_acc = 0.0f;
        for (int i = 0; i < 16; i++) {
            int lo = (int)(blk[2 + i] & 0x0F) - 8, hi = (int)(blk[2 + i] >> 4) - 8;
            block_acc += (float)lo * x[b * 32 + i];
            block_acc += (float)hi * x[b * 32 + i + 16];
        }
        acc += block_acc * scale;
    }
    return acc;
}

/* src/lib.rs:386-415 */
float fo_dot_q4_k_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / Q4_K_BYTES;
    float acc = 0.0f;
    size_t base = 0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q4_K_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        int is = 0, q_off = 0;
        for (int p = 0; p < 4; p++) {
            uint8_t sc1, m1, sc2, m2;
            fo_q4_k_scale_min(is, scales, &sc1, &m1);
            fo_q4_k_scale_min(is + 1, scales, &sc2, &m2);
            float d1 = d * (float)sc1, min1 = dmin * (float)m1;
            float d2 = d * (float)sc2, min2 = dmin * (float)m2;
            for (int l = 0; l < 32; l++)
                acc += (d1 * (float)(qs[q_off + l] & 0x0F) - min1) * x[base + l];
            for (int l = 0; l < 32; l++)
                acc += (d2 * (float)(qs[q_off + l] >> 4) - min2) * x[base + 32 + l];
            q_off += 32;
            base += 64;
            is += 2;
        }
    }
    return acc;
}

/* src/lib.rs:481-515 */
float fo_dot_q5_k_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / Q5_K_BYTES;
    float acc = 0.0f;
    size_t base = 0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q5_K_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
        int is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int oi = 0; oi < 4; oi++) {
            uint8_t sc1, m1, sc2, m2;
            fo_q4_k_scale_min(is, scales, &sc1, &m1);
            fo_q4_k_scale_min(is + 1, scales, &sc2, &m2);
            float d1 = d * (float)sc1, min1 = dmin * (float)m1;
            float d2 = d * (float)sc2, min2 = dmin * (float)m2;
            const uint8_t *ql = qs + oi * 32;
            for (int l = 0; l < 32; l++) {
                uint8_t hi = (qh[l] & u1) ? 16 : 0;
                acc += (d1 * (float)(uint8_t)((ql[l] & 0x0F) + hi) - min1) * x[base + l];
            }
            for (int l = 0; l < 32; l++) {
                uint8_t hi = (qh[l] & u2) ? 16 : 0;
                acc += (d2 * (float)(uint8_t)((ql[l] >> 4) + hi) - min2) * x[base + 32 + l];
            }
            base += 64;
            is += 2;
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
    return acc;
}

/* src/lib.rs:574-605 */
float fo_dot_q6_k_f32(const uint8_t *row, size_t row_bytes, const float *x) {
    size_t nb = row_bytes / Q6_K_BYTES;
    float acc = 0.0f;
    size_t x_base = 0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q6_K_BYTES;
        float d = rd_f16(blk + 208);
        for (int half = 0; half < 2; half++) {
            const uint8_t *ql = blk + half * 64, *qh = blk + 128 + half * 32;
            const int8_t *sc = (const int8_t *)(blk + 192 + half * 8);
            const float *xh = x + x_base;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int8_t q1 = (int8_t)((ql[l] & 0x0F) | ((qh[l] & 3) << 4)) - 32;
                int8_t q2 = (int8_t)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int8_t q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                acc += d * (float)sc[is] * (float)q1 * xh[l];
                acc += d * (float)sc[is + 2] * (float)q2 * xh[l + 32];
                acc += d * (float)sc[is + 4] * (float)q3 * xh[l + 64];
                acc += d * (float)sc[is + 6] * (float)q4 * xh[l + 96];
            }
            x_base += 128;
        }
    }
    return acc;
}

/* ---- activation quantizers ---- */

static inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* src/act_quant.rs:69-104.  f32::max ignores a NaN operand, as fmaxf does;
 * round_ties_even is rintf under the default rounding mode. */
void fo_quantize_q8_k(const float *x, size_t n, int8_t *q, float *d, int16_t *bsums) {
    size_t nb = n / QK_K;
    memset(q, 0, nb * QK_K);
    memset(d, 0, nb * sizeof(float));
    memset(bsums, 0, nb * 16 * sizeof(int16_t));
    for (size_t b = 0; b < nb; b++) {
        const float *chunk = x + b * QK_K;
        float amax = 0.0f;
        for (int i = 0; i < QK_K; i++) amax = fmaxf(amax, fabsf(chunk[i]));
        if (amax == 0.0f) continue;
        float iscale = 127.0f / amax;
        int8_t *qs = q + b * QK_K;
        for (int i = 0; i < QK_K; i++) {
            float r = clampf(rintf(iscale * chunk[i]), -127.0f, 127.0f);
            qs[i] = (r != r) ? 0 : (int8_t)r; /* Rust `as i8`: NaN -> 0 */
        }
        d[b] = 1.0f / iscale;
        for (int g = 0; g < 16; g++) {
            int32_t s = 0;
            for (int i = 0; i < 16; i++) s += qs[g * 16 + i];
            bsums[b * 16 + g] = (int16_t)s;
        }
    }
}

/* src/act_quant.rs:157-189 */
void fo_quantize_q8_0(const float *x, size_t n, int form, int8_t *q, float *d) {
    size_t nb = n / Q8_0_ELEMS;
    for (size_t b = 0; b < nb; b++) {
        const float *chunk = x + b * Q8_0_ELEMS;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(chunk[i]));
        float scale = amax / 127.0f;
        float inv = 0.0f;
        if (form == FO_Q8_0_FORM_AVX) {
            if (amax != 0.0f) inv = 127.0f / amax;
        } else {
            if (scale != 0.0f) inv = 1.0f / scale;
        }
        d[b] = fo_f16_to_f32(fo_f32_to_f16(scale));
        for (int i = 0; i < 32; i++) {
            float scaled = chunk[i] * inv;
            float r = (form == FO_Q8_0_FORM_SCALAR) ? roundf(scaled) : rintf(scaled);
            r = clampf(r, -127.0f, 127.0f);
            q[b * 32 + i] = (r != r) ? 0 : (int8_t)r;
        }
    }
}

/* ---- integer dots ---- */

/* src/lib.rs:711-733 */
float fo_dot_q8_0_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d) {
    size_t nb = row_bytes / Q8_0_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q8_0_BYTES;
        float dw = rd_f16(blk);
        int32_t isum = 0;
        for (int i = 0; i < 32; i++) isum += (int32_t)(int8_t)blk[2 + i] * (int32_t)q[b * 32 + i];
        acc += dw * d[b] * (float)isum;
    }
    return acc;
}

/* src/lib.rs:772-796: against Q8_0 activation blocks */
float fo_dot_q4_0_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d) {
    size_t nb = row_bytes / Q4_0_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q4_0_BYTES;
        float dw = rd_f16(blk);
        int32_t isum = 0;
        for (int i = 0; i < 16; i++) {
            int32_t q0 = (int32_t)(blk[2 + i] & 0x0F) - 8, q1 = (int32_t)(blk[2 + i] >> 4) - 8;
            isum += q0 * (int32_t)q[b * 32 + i];
            isum += q1 * (int32_t)q[b * 32 + 16 + i];
        }
        acc += dw * d[b] * (float)isum;
    }
    return acc;
}

/* ---- the 32-element block kinds against Q8_0 activation blocks (crates/frink-quant/src/legacy_q8.rs) ----
 * One body (dot_scalar<B>, :169-184) over a per-kind decoder (Block::decode, :63-86) and scale (Block::scale,
 * :58-60): a block contributes act.d[b] * (scale * isum as f32).
 * parity unpinned: the reference holds no numeric vector for these dots; the tests pin them through the
 * dequantizers (decoded integer x scale == the dequantized value, bit for bit, for every code and every
 * E8M0 scale byte) and through exact integer arithmetic on random blocks. */
/* legacy_q8.rs:108-116 with q5_fifth_bits (src/lib.rs:4346-4350): w = (nibble | fifth << 4) - 16 */
void fo_decode_q5_0_block(const uint8_t *blk, int8_t *w) {
    uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
    const uint8_t *qs = blk + 6;
    for (int j = 0; j < 16; j++) {
        uint8_t xh0, xh1;
        q5_fifth_bits(qh, j, &xh0, &xh1);
        w[j] = (int8_t)((int)((qs[j] & 0x0F) | xh0) - 16);
        w[j + 16] = (int8_t)((int)((qs[j] >> 4) | xh1) - 16);
    }
}
/* legacy_q8.rs:150 (ggml's kvalues_mxfp4: E2M1 times two) */
static const int8_t KVALUES_MXFP4_X2[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
/* legacy_q8.rs:154-161 (ggml_e8m0_to_fp32_half): 2^(e - 128), the two subnormal patterns for e < 2 */
float fo_e8m0_half_scale(uint8_t e) {
    uint32_t bits = e < 2 ? (0x00200000u << e) : ((uint32_t)(e - 1) << 23);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
/* legacy_q8.rs:133-147: codes through the doubled E2M1 table, low nibble -> element j, high -> j + 16 */
void fo_decode_mxfp4_block(const uint8_t *blk, int8_t *w) {
    for (int j = 0; j < 16; j++) {
        w[j] = KVALUES_MXFP4_X2[blk[1 + j] & 0xf];
        w[j + 16] = KVALUES_MXFP4_X2[blk[1 + j] >> 4];
    }
}
static float dot_legacy_q8(int kind, const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d) {
    size_t bb = kind == FO_KIND_Q5_0 ? Q5_0_BYTES : MXFP4_BYTES, nb = row_bytes / bb;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * bb;
        int8_t w[32];
        float scale;
        if (kind == FO_KIND_Q5_0) {
            fo_decode_q5_0_block(blk, w);
            scale = rd_f16(blk);
        } else {
            fo_decode_mxfp4_block(blk, w);
            scale = fo_e8m0_half_scale(blk[0]);
        }
        int32_t isum = 0;
        for (int i = 0; i < 32; i++) isum += (int32_t)w[i] * (int32_t)q[b * 32 + i];
        float block_acc = scale * (float)isum;
        acc += d[b] * block_acc;
    }
    return acc;
}
/* legacy_q8.rs:210 (dot_q5_0_q8_scalar) */
float fo_dot_q5_0_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d) {
    return dot_legacy_q8(FO_KIND_Q5_0, row, row_bytes, q, d);
}
/* legacy_q8.rs:213 (dot_mxfp4_q8_scalar) */
float fo_dot_mxfp4_q8(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *d) {
    return dot_legacy_q8(FO_KIND_MXFP4, row, row_bytes, q, d);
}
/* crates/frink-quant/src/iq4_xs_q8.rs:40-45 (sub_scale) and :67-98 (dot_iq4_xs_q8_k_scalar): per block the
 * integer sum of (ls - 32) * (codebook . q8) over the eight sub-blocks, then d * act.d[b] * sumi.
 * parity unpinned, as above: pinned through the dequantizer and exact integers. */
float fo_dot_iq4_xs_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *dact) {
    size_t nb = row_bytes / IQ4_XS_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * IQ4_XS_BYTES;
        float d = rd_f16(blk);
        unsigned scales_h = (unsigned)blk[2] | ((unsigned)blk[3] << 8);
        const uint8_t *scales_l = blk + 4, *qs = blk + 8;
        const int8_t *q8 = q + b * QK_K;
        int32_t sumi = 0;
        for (int ib = 0; ib < 8; ib++) {
            int32_t lo = (scales_l[ib / 2] >> (4 * (ib % 2))) & 0xf, hi = (scales_h >> (2 * ib)) & 3;
            int32_t ls = (lo | (hi << 4)) - 32;
            int32_t s = 0;
            for (int j = 0; j < 16; j++) {
                uint8_t byte = qs[ib * 16 + j];
                s += (int32_t)KVALUES_IQ4NL[byte & 0xf] * (int32_t)q8[ib * 32 + j];
                s += (int32_t)KVALUES_IQ4NL[byte >> 4] * (int32_t)q8[ib * 32 + 16 + j];
            }
            sumi += ls * s;
        }
        acc += d * dact[b] * (float)sumi;
    }
    return acc;
}

/* src/lib.rs:822-869 */
float fo_dot_q4_k_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *dact,
                      const int16_t *bsums_all) {
    size_t nb = row_bytes / Q4_K_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q4_K_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        float da = dact[b];
        const int8_t *q8 = q + b * QK_K;
        const int16_t *bsums = bsums_all + b * 16;

        int32_t sum_min = 0;
        for (int i = 0; i < 8; i++) {
            uint8_t sc, m;
            fo_q4_k_scale_min(i, scales, &sc, &m);
            sum_min += (int32_t)m * ((int32_t)bsums[2 * i] + (int32_t)bsums[2 * i + 1]);
        }
        acc -= dmin * da * (float)sum_min;

        int q_off = 0, base = 0, is = 0;
        for (int p = 0; p < 4; p++) {
            uint8_t sc1, sc2, m_;
            fo_q4_k_scale_min(is, scales, &sc1, &m_);
            fo_q4_k_scale_min(is + 1, scales, &sc2, &m_);
            int32_t isum1 = 0, isum2 = 0;
            for (int l = 0; l < 32; l++) isum1 += (int32_t)(qs[q_off + l] & 0x0F) * (int32_t)q8[base + l];
            for (int l = 0; l < 32; l++) isum2 += (int32_t)(qs[q_off + l] >> 4) * (int32_t)q8[base + 32 + l];
            acc += d * da * ((float)sc1 * (float)isum1 + (float)sc2 * (float)isum2);
            q_off += 32;
            base += 64;
            is += 2;
        }
    }
    return acc;
}

/* src/lib.rs:886-938 */
float fo_dot_q5_k_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *dact,
                      const int16_t *bsums_all) {
    size_t nb = row_bytes / Q5_K_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q5_K_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
        float da = dact[b];
        const int8_t *q8 = q + b * QK_K;
        const int16_t *bsums = bsums_all + b * 16;

        int32_t sum_min = 0;
        for (int i = 0; i < 8; i++) {
            uint8_t sc, m;
            fo_q4_k_scale_min(i, scales, &sc, &m);
            sum_min += (int32_t)m * ((int32_t)bsums[2 * i] + (int32_t)bsums[2 * i + 1]);
        }
        acc -= dmin * da * (float)sum_min;

        int q_off = 0, base = 0, is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int p = 0; p < 4; p++) {
            uint8_t sc1, sc2, m_;
            fo_q4_k_scale_min(is, scales, &sc1, &m_);
            fo_q4_k_scale_min(is + 1, scales, &sc2, &m_);
            int32_t isum1 = 0, isum2 = 0;
            for (int l = 0; l < 32; l++) {
                int32_t hi = (qh[l] & u1) ? 16 : 0;
                isum1 += ((int32_t)(qs[q_off + l] & 0x0F) + hi) * (int32_t)q8[base + l];
            }
            for (int l = 0; l < 32; l++) {
                int32_t hi = (qh[l] & u2) ? 16 : 0;
                isum2 += ((int32_t)(qs[q_off + l] >> 4) + hi) * (int32_t)q8[base + 32 + l];
            }
            acc += d * da * ((float)sc1 * (float)isum1 + (float)sc2 * (float)isum2);
            q_off += 32;
            base += 64;
            is += 2;
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
    return acc;
}

/* src/lib.rs:1069-1110 */
float fo_dot_q6_k_q8k(const uint8_t *row, size_t row_bytes, const int8_t *q, const float *dact) {
    size_t nb = row_bytes / Q6_K_BYTES;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q6_K_BYTES;
        float d = rd_f16(blk + 208);
        float da = dact[b];
        const int8_t *q8 = q + b * QK_K;
        int32_t isum = 0;
        for (int half = 0; half < 2; half++) {
            const uint8_t *ql = blk + half * 64, *qh = blk + 128 + half * 32;
            const int8_t *sc = (const int8_t *)(blk + 192 + half * 8);
            const int8_t *q8h = q8 + half * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int32_t q1 = (int32_t)(int8_t)((ql[l] & 0x0F) | ((qh[l] & 3) << 4)) - 32;
                int32_t q2 = (int32_t)(int8_t)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int32_t q3 = (int32_t)(int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int32_t q4 = (int32_t)(int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                isum += (int32_t)sc[is] * q1 * (int32_t)q8h[l];
                isum += (int32_t)sc[is + 2] * q2 * (int32_t)q8h[l + 32];
                isum += (int32_t)sc[is + 4] * q3 * (int32_t)q8h[l + 64];
                isum += (int32_t)sc[is + 6] * q4 * (int32_t)q8h[l + 96];
            }
        }
        acc += d * da * (float)isum;
    }
    return acc;
}

/* ---- encoders ---- */

/* src/encode/fit.rs:92-96 */
int fo_nearest_int(float fval) {
    float val = fval + 12582912.0f;
    int32_t i = (int32_t)f32_bits(val);
    return (i & 0x007fffff) - 0x00400000;
}

static inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* src/encode.rs:91-108 */
static void encode_block_q8_0(const float *block, uint8_t *out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) {
        float av = fabsf(block[i]);
        amax = amax > av ? amax : av;
    }
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    wr_f16(out, d);
    for (int i = 0; i < 32; i++) {
        float r = roundf(block[i] * id);
        int8_t v = (r != r) ? 0 : (r > 127.0f ? 127 : (r < -128.0f ? -128 : (int8_t)r));
        out[2 + i] = (uint8_t)v;
    }
}

/* src/encode.rs:118-128 */
int fo_encode_row_q8_0(const float *src, size_t n, uint8_t *out) {
    if (n % Q8_0_ELEMS) return -1;
    for (size_t b = 0; b < n / Q8_0_ELEMS; b++) encode_block_q8_0(src + b * 32, out + b * Q8_0_BYTES);
    return 0;
}

/* src/encode/fit.rs:111-206.  Returns scale, *the_min = -min. */
float fo_make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *l,
                          float *the_min, uint8_t *laux, float rmin, float rdelta, int nstep,
                          int use_mad) {
    float min = x[0], max = x[0];
    float sum_w = weights[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        float w = weights[i];
        sum_w += w;
        sum_x = fmaf(w, x[i], sum_x);
    }
    if (min > 0.0f) min = 0.0f;
    if (max == min) {
        for (int i = 0; i < n; i++) l[i] = 0;
        *the_min = -min;
        return 0.0f;
    }
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    float best_error = 0.0f;
    for (int i = 0; i < n; i++) {
        int li = clampi(fo_nearest_int(iscale * (x[i] - min)), 0, nmax);
        l[i] = (uint8_t)li;
        float diff = fmaf(scale, (float)l[i], min) - x[i];
        diff = use_mad ? fabsf(diff) : diff * diff;
        best_error = fmaf(weights[i], diff, best_error);
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (max - min);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        for (int i = 0; i < n; i++) {
            int li = clampi(fo_nearest_int(iscale * (x[i] - min)), 0, nmax);
            laux[i] = (uint8_t)li;
            float w = weights[i];
            sum_l = fmaf(w, (float)li, sum_l);
            sum_l2 = fmaf(w * (float)li, (float)li, sum_l2);
            sum_xl = fmaf(w * (float)li, x[i], sum_xl);
        }
        float det = fmaf(sum_w, sum_l2, -(sum_l * sum_l));
        if (det > 0.0f) {
            float this_scale = fmaf(sum_w, sum_xl, -(sum_x * sum_l)) / det;
            float this_min = fmaf(sum_l2, sum_x, -(sum_l * sum_xl)) / det;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.0f;
            for (int i = 0; i < n; i++) {
                float diff = fmaf(this_scale, (float)laux[i], this_min) - x[i];
                diff = use_mad ? fabsf(diff) : diff * diff;
                cur_error = fmaf(weights[i], diff, cur_error);
            }
            if (cur_error < best_error) {
                memcpy(l, laux, (size_t)n);
                best_error = cur_error;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

/* src/encode/fit.rs:216-226 with qw = None */
static inline float qx_weight(const float *x, int rmse_type, int i) {
    switch (rmse_type) {
    case 1: return x[i] * x[i];
    case 2: return 1.0f;
    case 3: return fabsf(x[i]);
    default: return sqrtf(fabsf(x[i]));
    }
}

/* src/encode/fit.rs:243-323 (no importance matrix) */
float fo_make_qx_quants(int n, int nmax, const float *x, int8_t *l, int rmse_type) {
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax < 1e-15f) {
        for (int i = 0; i < n; i++) l[i] = 0;
        return 0.0f;
    }
    float iscale = -(float)nmax / max;
    if (rmse_type == 0) {
        for (int i = 0; i < n; i++) {
            int li = fo_nearest_int(iscale * x[i]);
            l[i] = (int8_t)(nmax + clampi(li, -nmax, nmax - 1));
        }
        return 1.0f / iscale;
    }
    int return_early = 0;
    if (rmse_type < 0) {
        rmse_type = -rmse_type;
        return_early = 1;
    }
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int li = clampi(fo_nearest_int(iscale * x[i]), -nmax, nmax - 1);
        l[i] = (int8_t)(li + nmax);
        float w = qx_weight(x, rmse_type, i);
        sumlx = fmaf(w * x[i], (float)li, sumlx);
        suml2 = fmaf(w * (float)li, (float)li, suml2);
    }
    float scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
    if (return_early) return suml2 > 0.0f ? 0.5f * (scale + 1.0f / iscale) : 1.0f / iscale;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)is) / max;
        sumlx = 0.0f;
        suml2 = 0.0f;
        for (int i = 0; i < n; i++) {
            int li = clampi(fo_nearest_int(iscale * x[i]), -nmax, nmax - 1);
            float w = qx_weight(x, rmse_type, i);
            sumlx = fmaf(w * x[i], (float)li, sumlx);
            suml2 = fmaf(w * (float)li, (float)li, suml2);
        }
        if (suml2 > 0.0f && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; i++) {
                int li = fo_nearest_int(iscale * x[i]);
                l[i] = (int8_t)(nmax + clampi(li, -nmax, nmax - 1));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

/* src/encode/fit.rs:583-592 */
static void pack_scale_min(uint8_t *packed, int j, uint8_t ls, uint8_t lm) {
    if (j < 4) {
        packed[j] = ls;
        packed[j + 4] = lm;
    } else {
        packed[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
        packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
        packed[j] |= (uint8_t)((lm >> 4) << 6);
    }
}

/* fit_qk_super_block, src/encode/fit.rs:416-571 (plain path): the fit Q4_K and Q5_K share, with
 * QkFit's numbers as arguments -- Q4_K_FIT = {15, -1.0, 0.1, 20} (src/encode/q4_k.rs:42-48),
 * Q5_K_FIT = {31, -0.5, 0.1, 15} (src/encode/q5_k.rs:38-44).  Leaves the codes in l, the packed
 * 6-bit scales and mins, and the two f16 fields. */
static void fit_qk_super_block(const float *block, int nmax, float rmin, float rdelta, int nstep, uint8_t *l,
                               uint8_t *packed, uint16_t *dh_out, uint16_t *dminh_out) {
    uint8_t laux[32];
    float weights[32], mins[8], scales[8];
    memset(l, 0, QK_K);
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; j++) {
        const float *xs = block + 32 * j;
        /* qk_sub_block_weights, src/encode/fit.rs:327-336 */
        float sum_x2 = 0.0f;
        for (int i = 0; i < 32; i++) sum_x2 += xs[i] * xs[i];
        float av_x = sqrtf(sum_x2 / 32.0f);
        for (int i = 0; i < 32; i++) weights[i] = av_x + fabsf(xs[i]);
        float mn;
        float sc = fo_make_qkx2_quants(32, nmax, xs, weights, l + 32 * j, &mn, laux, rmin, rdelta, nstep, 0);
        scales[j] = sc;
        mins[j] = mn;
        if (sc > max_scale) max_scale = sc;
        if (mn > max_min) max_min = mn;
    }
    memset(packed, 0, 12);
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    for (int j = 0; j < 8; j++) {
        /* the narrowing to u8 comes BEFORE the clamp to 63 */
        uint8_t ls = (uint8_t)fo_nearest_int(inv_scale * scales[j]);
        uint8_t lm = (uint8_t)fo_nearest_int(inv_min * mins[j]);
        if (ls > 63) ls = 63;
        if (lm > 63) lm = 63;
        pack_scale_min(packed, j, ls, lm);
    }
    uint16_t dh = fo_f32_to_f16(max_scale / 63.0f), dminh = fo_f32_to_f16(max_min / 63.0f);
    float d = fo_f16_to_f32(dh), dmin = fo_f16_to_f32(dminh);
    for (int j = 0; j < 8; j++) {
        uint8_t sc, m;
        fo_q4_k_scale_min(j, packed, &sc, &m);
        float dj = d * (float)sc;
        if (dj == 0.0f) continue;
        float dm = dmin * (float)m;
        for (int ii = 0; ii < 32; ii++) {
            int idx = 32 * j + ii;
            l[idx] = (uint8_t)clampi(fo_nearest_int((block[idx] + dm) / dj), 0, nmax);
        }
    }
    *dh_out = dh;
    *dminh_out = dminh;
}

/* the nibble packing of src/encode/q4_k.rs:83-102 */
static void encode_block_q4_k(const float *block, uint8_t *out) {
    uint8_t l[QK_K], packed[12];
    uint16_t dh, dminh;
    fit_qk_super_block(block, 15, -1.0f, 0.1f, 20, l, packed, &dh, &dminh);
    out[0] = dh & 0xff; out[1] = dh >> 8;
    out[2] = dminh & 0xff; out[3] = dminh >> 8;
    memcpy(out + 4, packed, 12);
    uint8_t *qs = out + 16;
    for (int j = 0; j < QK_K; j += 64)
        for (int i = 0; i < 32; i++) *qs++ = (uint8_t)(l[j + i] | (l[j + i + 32] << 4));
}

/* src/encode/q5_k.rs:55-100: the fifth bit of a code goes to the qh plane, bit 2g of qh[j] for
 * element 64g + j and bit 2g + 1 for element 64g + 32 + j */
static void encode_block_q5_k(const float *block, uint8_t *out) {
    uint8_t l[QK_K], packed[12];
    uint16_t dh, dminh;
    fit_qk_super_block(block, 31, -0.5f, 0.1f, 15, l, packed, &dh, &dminh);
    out[0] = dh & 0xff; out[1] = dh >> 8;
    out[2] = dminh & 0xff; out[3] = dminh >> 8;
    memcpy(out + 4, packed, 12);
    uint8_t *qh = out + 16, *ql = out + 48;
    memset(qh, 0, 32);
    uint8_t m1 = 1, m2 = 2;
    for (int g = 0; g < 4; g++) {
        for (int j = 0; j < 32; j++) {
            uint8_t l1 = l[64 * g + j], l2 = l[64 * g + j + 32];
            if (l1 > 15) { l1 -= 16; qh[j] |= m1; }
            if (l2 > 15) { l2 -= 16; qh[j] |= m2; }
            ql[32 * g + j] = (uint8_t)(l1 | (l2 << 4));
        }
        m1 = (uint8_t)(m1 << 2);
        m2 = (uint8_t)(m2 << 2);
    }
}

/* src/encode/q4_k.rs:120-131 */
int fo_encode_row_q4_k(const float *src, size_t n, uint8_t *out) {
    if (n % QK_K) return -1;
    for (size_t b = 0; b < n / QK_K; b++) encode_block_q4_k(src + b * QK_K, out + b * Q4_K_BYTES);
    return 0;
}

/* src/encode/q5_k.rs:118-130 */
int fo_encode_row_q5_k(const float *src, size_t n, uint8_t *out) {
    if (n % QK_K) return -1;
    for (size_t b = 0; b < n / QK_K; b++) encode_block_q5_k(src + b * QK_K, out + b * Q5_K_BYTES);
    return 0;
}

/* src/encode/q6_k.rs:72-164 */
static void encode_block_q6_k(const float *block, uint8_t *out) {
    int8_t l[QK_K];
    float scales[16];
    memset(l, 0, sizeof l);
    float max_scale = 0.0f, max_abs_scale = 0.0f;
    for (int ib = 0; ib < 16; ib++) {
        float scale = fo_make_qx_quants(16, 32, block + 16 * ib, l + 16 * ib, 1);
        scales[ib] = scale;
        float abs_scale = fabsf(scale);
        if (abs_scale > max_abs_scale) {
            max_abs_scale = abs_scale;
            max_scale = scale;
        }
    }
    if (max_abs_scale < 1e-15f) {
        memset(out, 0, Q6_K_BYTES);
        return;
    }
    float iscale = -128.0f / max_scale;
    uint16_t dh = fo_f32_to_f16(1.0f / iscale);
    float d = fo_f16_to_f32(dh);
    int8_t qscales[16];
    for (int ib = 0; ib < 16; ib++) {
        int v = fo_nearest_int(iscale * scales[ib]);
        if (v > 127) v = 127;     /* clamp BEFORE narrowing */
        qscales[ib] = (int8_t)v; /* wraps like C's int8_t store */
    }
    for (int j = 0; j < 16; j++) {
        float dj = d * (float)qscales[j];
        if (dj == 0.0f) continue;
        for (int ii = 0; ii < 16; ii++) {
            int idx = 16 * j + ii;
            l[idx] = (int8_t)(clampi(fo_nearest_int(block[idx] / dj), -32, 31) + 32);
        }
    }
    uint8_t *ql = out, *qh = out + 128;
    for (int half = 0; half < 2; half++) {
        int j = half * 128, qlo = half * 64, qho = half * 32;
        for (int i = 0; i < 32; i++) {
            uint8_t q1 = (uint8_t)(l[j + i] & 0xF), q2 = (uint8_t)(l[j + i + 32] & 0xF);
            uint8_t q3 = (uint8_t)(l[j + i + 64] & 0xF), q4 = (uint8_t)(l[j + i + 96] & 0xF);
            ql[qlo + i] = (uint8_t)(q1 | (q3 << 4));
            ql[qlo + i + 32] = (uint8_t)(q2 | (q4 << 4));
            qh[qho + i] = (uint8_t)((uint8_t)(l[j + i] >> 4) | ((uint8_t)(l[j + i + 32] >> 4) << 2) |
                                    ((uint8_t)(l[j + i + 64] >> 4) << 4) |
                                    ((uint8_t)(l[j + i + 96] >> 4) << 6));
        }
    }
    memcpy(out + 192, qscales, 16);
    out[208] = dh & 0xff;
    out[209] = dh >> 8;
}

/* src/encode/q6_k.rs:179-190 */
int fo_encode_row_q6_k(const float *src, size_t n, uint8_t *out) {
    if (n % QK_K) return -1;
    for (size_t b = 0; b < n / QK_K; b++) encode_block_q6_k(src + b * QK_K, out + b * Q6_K_BYTES);
    return 0;
}

static int pick_threads(int threads) {
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#else
    threads = 1;
#endif
    return threads < 1 ? 1 : threads;
}

/* Row-major matrix, one row = cols/block_elems consecutive blocks, no padding
 * (frink-core/src/weight_matrix.rs:978-1052). */
int fo_encode_matrix(int kind, const float *src, size_t rows, size_t cols, uint8_t *out, int threads) {
    int be = fo_block_elems(kind), bb = fo_block_bytes(kind);
    if (!be || cols % (size_t)be) return -1;
    /* (only these four have an encoder: any other kind would be written with another kind's block size) */
    if (kind != FO_KIND_Q8_0 && kind != FO_KIND_Q4_K && kind != FO_KIND_Q5_K && kind != FO_KIND_Q6_K) return -2;
    size_t row_bytes = cols / (size_t)be * (size_t)bb;
    threads = pick_threads(threads);
    int rc = 0;
#pragma omp parallel for schedule(static) num_threads(threads)
    for (long r = 0; r < (long)rows; r++) {
        const float *s = src + (size_t)r * cols;
        uint8_t *o = out + (size_t)r * row_bytes;
        int e = kind == FO_KIND_Q8_0 ? fo_encode_row_q8_0(s, cols, o)
              : kind == FO_KIND_Q4_K ? fo_encode_row_q4_k(s, cols, o)
              : kind == FO_KIND_Q5_K ? fo_encode_row_q5_k(s, cols, o)
                                     : fo_encode_row_q6_k(s, cols, o);
        if (e) rc = e;
    }
    return rc;
}

/* ---- dispatch-level restatement ----
 * WeightMatrix::apply_cpu / apply_batch_with_acts (frink-core/src/weight_matrix.rs:1716-2073,
 * 2481-3365): out[b*rows + r] = dot(row r, activation b); int-dot tier quantizes each
 * activation row once (Q8_K for the K-quants and IQ4_XS, Q8_0 host form for Q8_0, Q4_0, Q5_0 and MXFP4 --
 * q8k_row_dot / q8_row_dot, weight_matrix.rs:392-420; an x86 host with AVX takes the Avx form,
 * src/act_quant.rs:129-148). */
typedef struct {
    int8_t *q;
    float *d;
    int16_t *bsums;
} acts_t;

static int acts_alloc(acts_t *a, int kind, size_t cols, size_t batch) {
    size_t be = (size_t)fo_block_elems(kind);
    a->q = (int8_t *)malloc(batch * cols);
    a->d = (float *)malloc(batch * (cols / be) * sizeof(float));
    int q8_0_acts = kind == FO_KIND_Q8_0 || kind == FO_KIND_Q4_0 || kind == FO_KIND_Q5_0 || kind == FO_KIND_MXFP4;
    a->bsums = q8_0_acts ? NULL : (int16_t *)malloc(batch * (cols / 16) * sizeof(int16_t));
    return a->q && a->d && (q8_0_acts || a->bsums) ? 0 : -1;
}
static void acts_free(acts_t *a) { free(a->q); free(a->d); free(a->bsums); }

static void acts_quantize(acts_t *a, int kind, const float *x, size_t cols, size_t batch) {
    size_t be = (size_t)fo_block_elems(kind);
    for (size_t b = 0; b < batch; b++) {
        if (kind == FO_KIND_Q8_0 || kind == FO_KIND_Q4_0 || kind == FO_KIND_Q5_0 || kind == FO_KIND_MXFP4)
            fo_quantize_q8_0(x + b * cols, cols, FO_Q8_0_FORM_AVX, a->q + b * cols, a->d + b * (cols / be));
        else
            fo_quantize_q8_k(x + b * cols, cols, a->q + b * cols, a->d + b * (cols / be),
                             a->bsums + b * (cols / 16));
    }
}

static inline float row_dot_int(int kind, const uint8_t *row, size_t row_bytes, const acts_t *a,
                                size_t b, size_t cols) {
    size_t be = (size_t)fo_block_elems(kind);
    const int8_t *q = a->q + b * cols;
    const float *d = a->d + b * (cols / be);
    switch (kind) {
    case FO_KIND_Q8_0: return fo_dot_q8_0_q8(row, row_bytes, q, d);
    case FO_KIND_Q4_0: return fo_dot_q4_0_q8(row, row_bytes, q, d);
    case FO_KIND_Q5_0: return fo_dot_q5_0_q8(row, row_bytes, q, d);
    case FO_KIND_MXFP4: return fo_dot_mxfp4_q8(row, row_bytes, q, d);
    case FO_KIND_IQ4_XS: return fo_dot_iq4_xs_q8k(row, row_bytes, q, d);
    case FO_KIND_Q4_K: return fo_dot_q4_k_q8k(row, row_bytes, q, d, a->bsums + b * (cols / 16));
    case FO_KIND_Q5_K: return fo_dot_q5_k_q8k(row, row_bytes, q, d, a->bsums + b * (cols / 16));
    default: return fo_dot_q6_k_q8k(row, row_bytes, q, d);
    }
}
static inline float row_dot_f32(int kind, const uint8_t *row, size_t row_bytes, const float *x) {
    switch (kind) {
    case FO_KIND_Q8_0: return fo_dot_q8_0_f32(row, row_bytes, x);
    case FO_KIND_Q4_0: return fo_dot_q4_0_f32(row, row_bytes, x);
    case FO_KIND_Q5_0: return fo_dot_q5_0_f32(row, row_bytes, x);
    case FO_KIND_IQ4_XS: return fo_dot_iq4_xs_f32(row, row_bytes, x);
    case FO_KIND_MXFP4: return fo_dot_mxfp4_f32(row, row_bytes, x);
    case FO_KIND_Q4_K: return fo_dot_q4_k_f32(row, row_bytes, x);
    case FO_KIND_Q5_K: return fo_dot_q5_k_f32(row, row_bytes, x);
    default: return fo_dot_q6_k_f32(row, row_bytes, x);
    }
}

int fo_gemm_rows(int kind, const uint8_t *w, size_t rows, size_t cols, size_t row0, size_t nrows,
                 const float *x, size_t batch, float *y, int mode, int threads) {
    int be = fo_block_elems(kind), bb = fo_block_bytes(kind);
    if (!be || cols == 0 || cols % (size_t)be || row0 + nrows > rows) return -1;
    size_t row_bytes = cols / (size_t)be * (size_t)bb;
    threads = pick_threads(threads);
    acts_t a = {0, 0, 0};
    if (mode == FO_MODE_INT_DOT) {
        if (acts_alloc(&a, kind, cols, batch)) { acts_free(&a); return -3; }
        acts_quantize(&a, kind, x, cols, batch);
    }
#pragma omp parallel for schedule(static) num_threads(threads)
    for (long r = 0; r < (long)nrows; r++) {
        const uint8_t *row = w + (row0 + (size_t)r) * row_bytes;
        for (size_t b = 0; b < batch; b++) {
            y[b * nrows + (size_t)r] = mode == FO_MODE_INT_DOT
                                           ? row_dot_int(kind, row, row_bytes, &a, b, cols)
                                           : row_dot_f32(kind, row, row_bytes, x + b * cols);
        }
    }
    if (mode == FO_MODE_INT_DOT) acts_free(&a);
    return 0;
}

int fo_gemm(int kind, const uint8_t *w, size_t rows, size_t cols, const float *x, size_t batch,
            float *y, int mode, int threads) {
    return fo_gemm_rows(kind, w, rows, cols, 0, rows, x, batch, y, mode, threads);
}

int fo_gemv(int kind, const uint8_t *w, size_t rows, size_t cols, const float *x, float *y,
            int mode, int threads) {
    return fo_gemm_rows(kind, w, rows, cols, 0, rows, x, 1, y, mode, threads);
}

/* ---- MoE ---- */

/* frink-core/src/matmul.rs:634-650.  (The reference's SIMD build evaluates exp with a
 * polynomial a few ulp from libm; this is the scalar definition.) */
float fo_silu(float x) { return x / (1.0f + expf(-x)); }
void fo_swiglu(const float *gate, const float *up, size_t n, float *out) {
    for (size_t i = 0; i < n; i++) out[i] = fo_silu(gate[i]) * up[i];
}

/* frink-moe/src/lib.rs:567-589.  The reference sorts by probability with an unstable sort and
 * no tie-break; equal probabilities have no defined order there.  This picks the lowest index
 * among equals. */
void fo_route_top_k_softmax(const float *logits, int n, int k, int norm, int32_t *ids, float *weights) {
    float max = -INFINITY;
    for (int i = 0; i < n; i++) max = fmaxf(max, logits[i]);
    float *probs = (float *)malloc((size_t)n * sizeof(float));
    char *taken = (char *)calloc((size_t)n, 1);
    float sum = 0.0f;
    for (int i = 0; i < n; i++) {
        probs[i] = expf(logits[i] - max);
        sum += probs[i];
    }
    for (int i = 0; i < n; i++) probs[i] = probs[i] / sum;
    if (k > n) k = n;
    for (int s = 0; s < k; s++) {
        int best = -1;
        for (int i = 0; i < n; i++)
            if (!taken[i] && (best < 0 || probs[i] > probs[best])) best = i;
        taken[best] = 1;
        ids[s] = best;
        weights[s] = probs[best];
    }
    if (norm) {
        float top_sum = 0.0f;
        for (int s = 0; s < k; s++) top_sum += weights[s];
        for (int s = 0; s < k; s++) weights[s] /= top_sum;
    }
    free(probs);
    free(taken);
}

/* frink-moe/src/lib.rs:1246-1263 (routed part): the slots of one token in the order given */
void fo_combine_expert_outputs(const float *const *expert_out, const float *weights, int n,
                               int hidden, float *out) {
    for (int i = 0; i < hidden; i++) out[i] = 0.0f;
    for (int e = 0; e < n; e++)
        for (int i = 0; i < hidden; i++) out[i] += expert_out[e][i] * weights[e];
}

/* The path of a batch below 32 tokens (ffn_batch.rs:355 returns None, the caller then runs every
 * position alone): per token, run_expert (frink-moe/src/lib.rs:1068-1165: gate and up over one
 * quantization of the token, SwiGLU, down over a quantization of its own) for each routed slot,
 * then combine_expert_outputs over the slots in routing order.  A slot whose id is outside
 * [0, n_experts) is left out. */
int fo_moe_ffn_per_position(int kind, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                            int n_experts, int hidden, int ffn, const float *x, int batch,
                            const int32_t *ids, const float *weights, int k, float *out, int threads) {
    int be = fo_block_elems(kind), bb = fo_block_bytes(kind);
    if (!be || hidden % be || ffn % be) return -1;
    size_t gu_bytes = (size_t)ffn * ((size_t)hidden / (size_t)be) * (size_t)bb;
    size_t dn_bytes = (size_t)hidden * ((size_t)ffn / (size_t)be) * (size_t)bb;
    float *g = (float *)malloc((size_t)ffn * sizeof(float));
    float *u = (float *)malloc((size_t)ffn * sizeof(float));
    float *outs = (float *)malloc((size_t)k * (size_t)hidden * sizeof(float));
    const float **ptrs = (const float **)malloc((size_t)k * sizeof(float *));
    float *w = (float *)malloc((size_t)k * sizeof(float));
    for (int b = 0; b < batch; b++) {
        const float *xb = x + (size_t)b * hidden;
        int n = 0;
        for (int s = 0; s < k; s++) {
            int e = ids[b * k + s];
            if (e < 0 || e >= n_experts) continue;
            fo_gemv(kind, gate + (size_t)e * gu_bytes, (size_t)ffn, (size_t)hidden, xb, g, FO_MODE_INT_DOT, threads);
            fo_gemv(kind, up + (size_t)e * gu_bytes, (size_t)ffn, (size_t)hidden, xb, u, FO_MODE_INT_DOT, threads);
            fo_swiglu(g, u, (size_t)ffn, g);
            fo_gemv(kind, down + (size_t)e * dn_bytes, (size_t)hidden, (size_t)ffn, g, outs + (size_t)n * hidden,
                    FO_MODE_INT_DOT, threads);
            ptrs[n] = outs + (size_t)n * hidden;
            w[n] = weights[b * k + s];
            n++;
        }
        fo_combine_expert_outputs(ptrs, w, n, hidden, out + (size_t)b * hidden);
    }
    free(g); free(u); free(outs); free((void *)ptrs); free(w);
    return 0;
}

/* frink-models/src/decoder/ffn_batch.rs:343-434: bucket tokens by expert (token-major fill),
 * for each expert in ascending id: gather rows, quantize once for gate and up, gate/up GEMMs,
 * SwiGLU, down GEMM (which quantizes its own input), acc[tok] += w * down. */
int fo_moe_ffn_batch(int kind, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                     int n_experts, int hidden, int ffn, const float *x, int batch,
                     const int32_t *ids, const float *weights, int k, float *out, int threads) {
    int be = fo_block_elems(kind), bb = fo_block_bytes(kind);
    if (!be || hidden % be || ffn % be) return -1;
    size_t gu_bytes = (size_t)ffn * ((size_t)hidden / (size_t)be) * (size_t)bb;
    size_t dn_bytes = (size_t)hidden * ((size_t)ffn / (size_t)be) * (size_t)bb;
    size_t pairs = (size_t)batch * (size_t)k;
    int *tok = (int *)malloc(pairs * sizeof(int));
    float *w = (float *)malloc(pairs * sizeof(float));
    float *gathered = (float *)malloc((size_t)batch * (size_t)hidden * sizeof(float));
    float *g = (float *)malloc((size_t)batch * (size_t)ffn * sizeof(float));
    float *u = (float *)malloc((size_t)batch * (size_t)ffn * sizeof(float));
    float *dn = (float *)malloc((size_t)batch * (size_t)hidden * sizeof(float));
    memset(out, 0, (size_t)batch * (size_t)hidden * sizeof(float));
    for (int e = 0; e < n_experts; e++) {
        int n = 0;
        for (int b = 0; b < batch; b++)
            for (int s = 0; s < k; s++)
                if (ids[b * k + s] == e) {
                    tok[n] = b;
                    w[n] = weights[b * k + s];
                    n++;
                }
        if (n == 0) continue;
        for (int i = 0; i < n; i++)
            memcpy(gathered + (size_t)i * hidden, x + (size_t)tok[i] * hidden, (size_t)hidden * sizeof(float));
        fo_gemm(kind, gate + (size_t)e * gu_bytes, (size_t)ffn, (size_t)hidden, gathered, (size_t)n, g,
                FO_MODE_INT_DOT, threads);
        fo_gemm(kind, up + (size_t)e * gu_bytes, (size_t)ffn, (size_t)hidden, gathered, (size_t)n, u,
                FO_MODE_INT_DOT, threads);
        fo_swiglu(g, u, (size_t)n * (size_t)ffn, g);
        fo_gemm(kind, down + (size_t)e * dn_bytes, (size_t)hidden, (size_t)ffn, g, (size_t)n, dn,
                FO_MODE_INT_DOT, threads);
        for (int i = 0; i < n; i++) {
            float *row = out + (size_t)tok[i] * hidden;
            const float *o = dn + (size_t)i * hidden;
            for (int j = 0; j < hidden; j++) row[j] += w[i] * o[j];
        }
    }
    free(tok); free(w); free(gathered); free(g); free(u); free(dn);
    return 0;
}

int fo_have_avx2(void) {
#if defined(__x86_64__)
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
#else
    return 0;
#endif
}
