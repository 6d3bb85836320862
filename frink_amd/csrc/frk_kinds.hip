// Q5_0, IQ4_XS and MXFP4 (GGUF block form): dequantizer / row gather and the decode GEMV on the f32
// activation -- the kinds behind the reference's per-kind seam that the Q4_K_M model family does not use
// (crates/frink-cuda/src/mul_mm.rs:146-205; CPU forms dequant_q5_0 / dot_q5_0_f32,
// crates/frink-quant/src/lib.rs:4356-4418, dequant_iq4_xs / dot_iq4_xs_f32 :4860-4934, the E8M0 x E2M1
// arithmetic of dequant_mxfp4_row / dot_mxfp4_row_f32 :4947-5040 over 17-byte GGUF blocks :5560-5570).
// The resident copy keeps the GGUF bytes of a row in place (rows start 16-byte aligned); a weight is the
// dequantizer's value bit for bit.  The GEMV is the f32 dot of the reference's decode path: a wavefront
// per row, a lane per unit of 32 weights, the activation staged in LDS; the integer tier of these kinds
// (Q8_0 / Q8_K activations, crates/frink-quant/src/legacy_q8.rs, iq4_xs_q8.rs) is the second half of this file.
#include "frk_device.hpp"

namespace frk {

__device__ __forceinline__ float e8m0_scale(uint32_t e) { return __uint_as_float(e == 0 ? 0x00400000u : e << 23); }

// Four table look-ups at once, the tables in registers: v_perm_b32 picks each byte of its result out of eight
// bytes (S1 = entries 0..3, S0 = entries 4..7) by a selector byte.  (A table in constant memory is a load per
// weight: the IQ4_XS decode GEMV took 35 us at 14336x4096, the MXFP4 one 47.)
__device__ __forceinline__ uint32_t perm8(uint32_t hi4, uint32_t lo4, uint32_t sel) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_perm(hi4, lo4, sel);
#else
    return 0;
#endif
}
// kvalues_iq4nl of four 4-bit codes (one a byte of n): four signed bytes
__device__ __forceinline__ uint32_t iq4nl_lookup4(uint32_t n) {
    const uint32_t sel = n & 0x07070707u;
    const uint32_t lo = perm8(0xF6EADDCFu, 0xBFAD9881u, sel);  // -127 -104 -83 -65 | -49 -35 -22 -10
    const uint32_t hi = perm8(0x71594535u, 0x26190D01u, sel);  //    1   13  25  38 |  53  69  89 113
    const uint32_t m = ((n >> 3) & 0x01010101u) * 0xffu;       // 0xff in the bytes whose code is 8 or more
    return (hi & m) | (lo & ~m);
}
__device__ __forceinline__ float signed_byte(uint32_t v, int k) { return (float)(int)(int8_t)((v >> (8 * k)) & 0xff); }
// the E2M1 values of four 4-bit codes as the two upper bytes of their f32 patterns (the lower two are zero):
// 0 .5 1 1.5 2 3 4 6 = 0000 3F00 3F80 3FC0 4000 4040 4080 40C0, the code's bit 3 the sign
struct E2M1x4 {
    uint32_t top, second;
};
__device__ __forceinline__ E2M1x4 e2m1_lookup4(uint32_t n) {
    const uint32_t c = n & 0x07070707u;
    E2M1x4 r;
    r.top = perm8(0x40404040u, 0x3F3F3F00u, c) | ((n & 0x08080808u) << 4);
    r.second = perm8(0xC0804000u, 0xC0800000u, c);
    return r;
}
__device__ __forceinline__ float e2m1_value(const E2M1x4 &v, int k) {
    // byte 3 = top.byte[k] (entries 4..7 of the pair), byte 2 = second.byte[k], bytes 1 and 0 = 0x00 (selector 0x0c)
    return __uint_as_float(perm8(v.top, v.second, ((uint32_t)(4 + k) << 24) | ((uint32_t)k << 16) | 0x0c0cu));
}
__device__ __forceinline__ uint32_t load_u16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }

// the 32 weights of unit u of a row (a block of Q5_0 / MXFP4, a sub-block of IQ4_XS), in element order
template <int KIND>
__device__ __forceinline__ void unit_weights(const uint8_t *__restrict__ row, int u, float (&w)[32]) {
    if (KIND == FRK_KIND_Q5_0) {
        const uint8_t *blk = row + (size_t)u * Q5_0_BYTES;  // 2-byte aligned
        const float d = h2f(load_u16(blk));
        const uint32_t qh = load_u16(blk + 2) | (load_u16(blk + 4) << 16);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t two = load_u16(blk + 6 + 2 * i);
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int j = 2 * i + k;
                const uint32_t byte = (two >> (8 * k)) & 0xff;
                const int x0 = (int)((byte & 0x0f) | (((qh >> j) << 4) & 0x10)) - 16;
                const int x1 = (int)((byte >> 4) | ((qh >> (j + 12)) & 0x10)) - 16;
                w[j] = __fmul_rn((float)x0, d);
                w[j + 16] = __fmul_rn((float)x1, d);
            }
        }
    } else if (KIND == FRK_KIND_IQ4_XS) {
        const int b = u >> 3, ib = u & 7;
        const uint8_t *blk = row + (size_t)b * IQ4_XS_BYTES;  // 8-byte aligned
        const uint32_t head = *reinterpret_cast<const uint32_t *>(blk), sl = *reinterpret_cast<const uint32_t *>(blk + 4);
        const float d = h2f(head & 0xffffu);
        const uint32_t scales_h = head >> 16;
        const uint32_t ls = ((sl >> (8 * (ib >> 1) + 4 * (ib & 1))) & 0xf) | (((scales_h >> (2 * ib)) & 3) << 4);
        const float dl = __fmul_rn(d, (float)ls - 32.0f);
        const uint2 qa = *reinterpret_cast<const uint2 *>(blk + 8 + ib * 16), qb = *reinterpret_cast<const uint2 *>(blk + 16 + ib * 16);
        const uint32_t q[4] = {qa.x, qa.y, qb.x, qb.y};
#pragma unroll
        for (int i = 0; i < 4; i++) {  // four bytes of codes: elements 4i .. 4i+3 in the low nibbles, 16 more on in the high
            const uint32_t lo = iq4nl_lookup4(q[i] & 0x0f0f0f0fu), hi = iq4nl_lookup4((q[i] >> 4) & 0x0f0f0f0fu);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                w[4 * i + k] = __fmul_rn(dl, signed_byte(lo, k));
                w[4 * i + k + 16] = __fmul_rn(dl, signed_byte(hi, k));
            }
        }
    } else {  // MXFP4: 17-byte blocks, no alignment
        const uint8_t *blk = row + (size_t)u * MXFP4_BYTES;
        const float d = e8m0_scale(blk[0]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q = (uint32_t)blk[1 + 4 * i] | ((uint32_t)blk[2 + 4 * i] << 8) | ((uint32_t)blk[3 + 4 * i] << 16) |
                               ((uint32_t)blk[4 + 4 * i] << 24);
            const E2M1x4 lo = e2m1_lookup4(q & 0x0f0f0f0fu), hi = e2m1_lookup4((q >> 4) & 0x0f0f0f0fu);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                w[4 * i + k] = __fmul_rn(d, e2m1_value(lo, k));
                w[4 * i + k + 16] = __fmul_rn(d, e2m1_value(hi, k));
            }
        }
    }
}

// one thread per unit of 32 output values; with a list of row numbers, the embedding gather
template <int KIND>
__global__ __launch_bounds__(256) void dequant_units_kernel(const uint8_t *__restrict__ W, size_t n_out, size_t cols, size_t row_stride,
                                                           const int32_t *__restrict__ ids, size_t table_rows,
                                                           float *__restrict__ out) {
    const size_t units = cols / 32;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n_out * units) return;
    const size_t r_out = i / units, u = i % units;
    size_t r = r_out;
    if (ids) {
        const int32_t id = ids[r_out];
        r = id < 0 ? 0 : (size_t)id >= table_rows ? table_rows - 1 : (size_t)id;
    }
    float w[32];
    unit_weights<KIND>(W + r * row_stride, (int)u, w);
    float4 *dst = reinterpret_cast<float4 *>(out + r_out * cols + u * 32);
#pragma unroll
    for (int k = 0; k < 8; k++) dst[k] = make_float4(w[4 * k], w[4 * k + 1], w[4 * k + 2], w[4 * k + 3]);
}

template <int KIND>
__global__ __launch_bounds__(512) void gemv_units_f32_kernel(const uint8_t *__restrict__ W, size_t row_stride, int rows, int cols,
                                                            const float *__restrict__ x, float *__restrict__ y) {
    extern __shared__ uint4 smem_kinds[];
    float *xs = reinterpret_cast<float *>(smem_kinds);
    for (int i = threadIdx.x; i < cols / 4; i += 512) reinterpret_cast<float4 *>(xs)[i] = reinterpret_cast<const float4 *>(x)[i];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int units = cols / 32;
    for (int r = (int)blockIdx.x * 8 + wave; r < rows; r += (int)gridDim.x * 8) {
        const uint8_t *row = W + (size_t)r * row_stride;
        float acc = 0.0f;
        for (int u = lane; u < units; u += 64) {
            float w[32];
            unit_weights<KIND>(row, u, w);
            const float4 *x4 = reinterpret_cast<const float4 *>(xs + (size_t)u * 32);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float4 xv = x4[k];
                acc = fmaf(w[4 * k], xv.x, acc);
                acc = fmaf(w[4 * k + 1], xv.y, acc);
                acc = fmaf(w[4 * k + 2], xv.z, acc);
                acc = fmaf(w[4 * k + 3], xv.w, acc);
            }
        }
        acc = part_sum<64>(acc);
        if (lane == 0) y[r] = acc;
    }
}

// ---- the integer tier: Q5_0 and MXFP4 rows against Q8_0 activation blocks (dot_q5_0_q8 / dot_mxfp4_q8,
// crates/frink-quant/src/legacy_q8.rs:169-213), IQ4_XS rows against Q8_K activations (dot_iq4_xs_q8_k,
// crates/frink-quant/src/iq4_xs_q8.rs:67-98).  A unit decodes to 32 signed bytes (Q5_0: nibble | fifth bit << 4,
// minus 16; MXFP4: the doubled E2M1 table, with the halved E8M0 scale; IQ4_XS: kvalues_iq4nl), four to a register,
// and meets the activation's bytes in v_dot4: the integers are the reference's, the float step per block its
// expression -- act.d[b] * (scale * isum) for the 32-element kinds, d * act.d[b] * sum(ls * s) per 256 for IQ4_XS.

// bit k of the low four bits of b to bit 8k (k = 0..3): the four shifted copies do not overlap, so no carry
__device__ __forceinline__ uint32_t spread4(uint32_t b) { return ((b & 0xfu) * 0x00204081u) & 0x01010101u; }
// four 5-bit codes (one a byte) minus 16, as signed bytes: with 128 added first no byte borrows
__device__ __forceinline__ uint32_t minus16_bytes(uint32_t c) { return ((c | 0x80808080u) - 0x10101010u) ^ 0x80808080u; }
// kvalues_mxfp4 (E2M1 times two) of four 4-bit codes: 0 1 2 3 4 6 8 12, the code's bit 3 the sign
__device__ __forceinline__ uint32_t mxfp4_x2_lookup4(uint32_t n) {
    const uint32_t sel = n & 0x07070707u;
    const uint32_t pos = perm8(0x0C080604u, 0x03020100u, sel);
    const uint32_t neg = perm8(0xF4F8FAFCu, 0xFDFEFF00u, sel);
    const uint32_t m = ((n >> 3) & 0x01010101u) * 0xffu;
    return (neg & m) | (pos & ~m);
}
// ggml_e8m0_to_fp32_half (legacy_q8.rs:154-161): 2^(e - 128), the two subnormal patterns for e < 2
__device__ __forceinline__ float e8m0_half_scale(uint32_t e) { return __uint_as_float(e < 2 ? 0x00200000u << e : (e - 1) << 23); }

// The 32 codes of unit u of a row held in LDS, as eight registers of four signed bytes: c[0..3] = elements 0..15,
// c[4..7] = elements 16..31; `scale` = the unit's multiplier (Q5_0: d; MXFP4: the halved E8M0 scale; IQ4_XS: ls - 32
// as an integer in scale_i, the block's d in scale).
template <int KIND>
__device__ __forceinline__ void unit_codes(const uint8_t *row, int u, uint32_t (&c)[8], float &scale, int &scale_i) {
    scale_i = 1;
    if (KIND == FRK_KIND_Q5_0) {
        const uint8_t *blk = row + u * Q5_0_BYTES;  // 2-byte aligned
        scale = h2f(load_u16(blk));
        const uint32_t qh = load_u16(blk + 2) | (load_u16(blk + 4) << 16);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q = load_u16(blk + 6 + 4 * i) | (load_u16(blk + 8 + 4 * i) << 16);
            c[i] = minus16_bytes((q & 0x0f0f0f0fu) | (spread4(qh >> (4 * i)) << 4));
            c[4 + i] = minus16_bytes(((q >> 4) & 0x0f0f0f0fu) | (spread4(qh >> (16 + 4 * i)) << 4));
        }
    } else if (KIND == FRK_KIND_IQ4_XS) {
        const int b = u >> 3, ib = u & 7;
        const uint8_t *blk = row + b * IQ4_XS_BYTES;  // 8-byte aligned
        const uint32_t head = *reinterpret_cast<const uint32_t *>(blk), sl = *reinterpret_cast<const uint32_t *>(blk + 4);
        scale = h2f(head & 0xffffu);
        const uint32_t scales_h = head >> 16;
        scale_i = (int)(((sl >> (8 * (ib >> 1) + 4 * (ib & 1))) & 0xf) | (((scales_h >> (2 * ib)) & 3) << 4)) - 32;
        const uint2 qa = *reinterpret_cast<const uint2 *>(blk + 8 + ib * 16), qb = *reinterpret_cast<const uint2 *>(blk + 16 + ib * 16);
        const uint32_t q[4] = {qa.x, qa.y, qb.x, qb.y};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            c[i] = iq4nl_lookup4(q[i] & 0x0f0f0f0fu);
            c[4 + i] = iq4nl_lookup4((q[i] >> 4) & 0x0f0f0f0fu);
        }
    } else {  // MXFP4: 17-byte blocks, no alignment -- the sixteen code bytes out of five aligned words
        const uint32_t at = (uint32_t)u * MXFP4_BYTES;
        scale = e8m0_half_scale(row[at]);
        const uint32_t *words = reinterpret_cast<const uint32_t *>(row) + ((at + 1) >> 2);
        const uint32_t shift = (at + 1) & 3;  // (0: the fifth word is read and not used; the slot ends in slack for it)
        const uint32_t g0 = words[0], g1 = words[1], g2 = words[2], g3 = words[3], g4 = words[4];
        const uint32_t q[4] = {__builtin_amdgcn_alignbyte(g1, g0, shift), __builtin_amdgcn_alignbyte(g2, g1, shift),
                               __builtin_amdgcn_alignbyte(g3, g2, shift), __builtin_amdgcn_alignbyte(g4, g3, shift)};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            c[i] = mxfp4_x2_lookup4(q[i] & 0x0f0f0f0fu);
            c[4 + i] = mxfp4_x2_lookup4((q[i] >> 4) & 0x0f0f0f0fu);
        }
    }
}

// A wavefront per row, a lane per unit.  The quantized activation sits in LDS for the whole launch; a row's bytes go
// global -> registers (whole 16-byte pieces, the next row's while this one is multiplied) -> the wavefront's own
// LDS slot, from where the lanes pick their blocks apart (22- and 17-byte blocks have no alignment to load by).
// JOBS: a grid of expert-indexed jobs (run_expert's projections, crates/frink-moe/src/lib.rs:1068-1165): job
// blockIdx.y multiplies the rows of expert ids[job] (a slice of `rows` rows of the stacked matrix) with activation
// row job / act_div and writes output row job; a job whose id is outside the experts does nothing.
struct UnitsJobs {
    const int32_t *ids;
    int n_experts, job0, act_div;
    // a second stack of the same shape over the same jobs and activations (gate and up in one launch): grid rows
    // n_jobs .. 2 * n_jobs - 1 multiply W2 and write y2
    const uint8_t *W2;
    float *y2;
    int n_jobs;
};
template <int KIND, int MAXP, bool JOBS = false>
__global__ __launch_bounds__(512) void gemv_units_int_kernel(const uint8_t *__restrict__ W, size_t row_stride, int rows, int cols,
                                                            const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                                            float *__restrict__ y, UnitsJobs jobs) {
    extern __shared__ uint4 smem_kinds[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem_kinds);
    const int units = cols / 32, nd = KIND == FRK_KIND_IQ4_XS ? cols / QK_K : units;
    if (JOBS) {
        int job = jobs.job0 + (int)blockIdx.y;
        if (jobs.W2 && job >= jobs.n_jobs) {  // (uniform per workgroup)
            job -= jobs.n_jobs;
            W = jobs.W2;
            y = jobs.y2;
        }
        const int e = jobs.ids[job];
        if (e < 0 || e >= jobs.n_experts) return;  // (uniform per workgroup)
        W += (size_t)e * rows * row_stride;
        aq += (size_t)(job / jobs.act_div) * cols;
        ad += (size_t)(job / jobs.act_div) * nd;
        y += (size_t)job * rows;
    }
    int8_t *sq = reinterpret_cast<int8_t *>(lds);
    float *sd = reinterpret_cast<float *>(lds + cols);
    const int pieces = (int)(row_stride / 16);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    typedef uint32_t piece_t __attribute__((ext_vector_type(4)));
    piece_t *mine = reinterpret_cast<piece_t *>(lds + ((cols + nd * 4 + 15) & ~15)) + (size_t)wave * pieces;
    for (int i = threadIdx.x; i < cols / 16; i += 512) reinterpret_cast<uint4 *>(sq)[i] = reinterpret_cast<const uint4 *>(aq)[i];
    for (int i = threadIdx.x; i < nd; i += 512) sd[i] = ad[i];
    // (a piece past the row's end: the row's last piece again, stored to the same place by the lanes that hold it;
    // the array is only ever indexed by unrolled constants, and no lambda takes it: it stays in registers)
    piece_t pre[MAXP];
    const int step = (int)gridDim.x * 8;
    int r = (int)blockIdx.x * 8 + wave;
    {
        const piece_t *src = reinterpret_cast<const piece_t *>(W + (size_t)min(r, rows - 1) * row_stride);
#pragma unroll
        for (int p = 0; p < MAXP; p++) pre[p] = src[min(lane + 64 * p, pieces - 1)];
    }
    __syncthreads();
    for (; r < rows; r += step) {
#pragma unroll
        for (int p = 0; p < MAXP; p++) mine[min(lane + 64 * p, pieces - 1)] = pre[p];
        {
            const piece_t *src = reinterpret_cast<const piece_t *>(W + (size_t)min(r + step, rows - 1) * row_stride);
#pragma unroll
            for (int p = 0; p < MAXP; p++) pre[p] = src[min(lane + 64 * p, pieces - 1)];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint8_t *row = reinterpret_cast<const uint8_t *>(mine);
        float acc = 0.0f;
        for (int u0 = 0; u0 < units; u0 += 64) {  // (uniform: the lanes of an IQ4_XS block exchange their sums)
            const bool live = u0 + lane < units;
            const int u = live ? u0 + lane : units - 1;
            uint32_t c[8];
            float scale;
            int scale_i;
            unit_codes<KIND>(row, u, c, scale, scale_i);
            const uint4 a0 = *reinterpret_cast<const uint4 *>(sq + u * 32), a1 = *reinterpret_cast<const uint4 *>(sq + u * 32 + 16);
            int isum = 0;
            isum = dot4(c[0], a0.x, isum);
            isum = dot4(c[1], a0.y, isum);
            isum = dot4(c[2], a0.z, isum);
            isum = dot4(c[3], a0.w, isum);
            isum = dot4(c[4], a1.x, isum);
            isum = dot4(c[5], a1.y, isum);
            isum = dot4(c[6], a1.z, isum);
            isum = dot4(c[7], a1.w, isum);
            if (KIND == FRK_KIND_IQ4_XS) {
                int t = live ? scale_i * isum : 0;  // |ls| <= 32, |s| <= 32 * 127 * 127: fits
                t += __shfl_xor(t, 1);
                t += __shfl_xor(t, 2);
                t += __shfl_xor(t, 4);
                if (live && (u & 7) == 0) acc += scale * sd[u >> 3] * (float)t;
            } else if (live) {
                acc += sd[u] * (scale * (float)isum);
            }
        }
        acc = part_sum<64>(acc);
        if (lane == 0) y[r] = acc;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();  // (the slot is rewritten at the top of the loop)
    }
}

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

bool is_unit_kind(int kind) { return kind == FRK_KIND_Q5_0 || kind == FRK_KIND_IQ4_XS || kind == FRK_KIND_MXFP4; }

int launch_dequant_units(const frk_weights *w, const int32_t *ids, size_t n_out, float *out, hipStream_t s) {
    const unsigned g = (unsigned)((n_out * (w->cols / 32) + 255) / 256);
    if (g == 0) return FRK_OK;
#define FRK_GO(KIND) \
    hipLaunchKernelGGL((dequant_units_kernel<KIND>), dim3(g), dim3(256), 0, s, w->dev, n_out, w->cols, w->layout.row_stride, ids, w->rows, out)
    if (w->kind == FRK_KIND_Q5_0) FRK_GO(FRK_KIND_Q5_0);
    else if (w->kind == FRK_KIND_IQ4_XS) FRK_GO(FRK_KIND_IQ4_XS);
    else FRK_GO(FRK_KIND_MXFP4);
#undef FRK_GO
    FRK_LAUNCH_CHECK("dequant_units");
    return FRK_OK;
}

// y = W x on dequantized weights and the f32 activation; rows of at most 16384 columns
int launch_gemv_units_f32(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    if (w->cols * 4 > 64 * 1024)
        return set_error(FRK_ERR_UNSUPPORTED, "the GEMV of quant kind %d takes rows of at most 16384 columns (%zu)", w->kind, w->cols);
    const size_t shmem = w->cols * 4;
    const unsigned grid = (unsigned)std::min<size_t>((w->rows + 7) / 8, 2048);
#define FRK_GO(KIND) \
    hipLaunchKernelGGL((gemv_units_f32_kernel<KIND>), dim3(grid), dim3(512), shmem, s, w->dev, w->layout.row_stride, (int)w->rows, (int)w->cols, x, y)
    if (w->kind == FRK_KIND_Q5_0) FRK_GO(FRK_KIND_Q5_0);
    else if (w->kind == FRK_KIND_IQ4_XS) FRK_GO(FRK_KIND_IQ4_XS);
    else FRK_GO(FRK_KIND_MXFP4);
#undef FRK_GO
    FRK_LAUNCH_CHECK("gemv_units_f32");
    return FRK_OK;
}

// y = W x on the integer tier: aq / ad are the activation's Q8_0 blocks (Q5_0, MXFP4) or its Q8_K quants and
// block scales (IQ4_XS)
size_t gemv_units_int_lds(const frk_weights *w) {
    const size_t nd = w->kind == FRK_KIND_IQ4_XS ? w->cols / QK_K : w->cols / 32;
    return ((w->cols + nd * 4 + 15) & ~(size_t)15) + 8 * w->layout.row_stride + 16;  // (16 bytes of slack behind the last slot)
}
bool gemv_units_int_fits(const frk_weights *w) { return gemv_units_int_lds(w) <= 160 * 1024 && w->layout.row_stride <= 12 * 1024; }
template <int KIND, int MAXP>
static int launch_gemv_units_int_as(const frk_weights *w, const int8_t *aq, const float *ad, float *y, hipStream_t s) {
    const size_t shmem = gemv_units_int_lds(w);
    static size_t sized = 0;  // a benign race: every thread raises the same attribute
    if (shmem > sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_units_int_kernel<KIND, MAXP>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(gemv units int): %s", hipGetErrorString(e));
        sized = 160 * 1024;
    }
    const unsigned grid = (unsigned)std::min<size_t>((w->rows + 7) / 8, 2048);
    hipLaunchKernelGGL((gemv_units_int_kernel<KIND, MAXP>), dim3(grid), dim3(512), shmem, s, w->dev, w->layout.row_stride, (int)w->rows,
                       (int)w->cols, aq, ad, y, UnitsJobs{nullptr, 0, 0, 1, nullptr, nullptr, 0});
    FRK_LAUNCH_CHECK("gemv_units_int");
    return FRK_OK;
}
template <int KIND, int MAXP>
static int launch_gemv_units_jobs_as(const frk_weights *w, const frk_weights *w2, size_t rows_e, int n_experts, const int32_t *ids,
                                     size_t n_jobs, int act_div, const int8_t *aq, const float *ad, float *y, float *y2, hipStream_t s) {
    const size_t shmem = gemv_units_int_lds(w);
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_units_int_kernel<KIND, MAXP, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(gemv units jobs): %s", hipGetErrorString(e));
        sized = true;
    }
    const unsigned gx = (unsigned)std::min<size_t>((rows_e + 7) / 8, 2048);
    if (w2 && 2 * n_jobs <= 65535) {  // both stacks in one launch
        hipLaunchKernelGGL((gemv_units_int_kernel<KIND, MAXP, true>), dim3(gx, (unsigned)(2 * n_jobs)), dim3(512), shmem, s, w->dev,
                           w->layout.row_stride, (int)rows_e, (int)w->cols, aq, ad, y,
                           UnitsJobs{ids, n_experts, 0, act_div, w2->dev, y2, (int)n_jobs});
        FRK_LAUNCH_CHECK("gemv_units_int (jobs, two stacks)");
        return FRK_OK;
    }
    for (int m = 0; m < (w2 ? 2 : 1); m++) {
        const frk_weights *wm = m ? w2 : w;
        for (size_t j0 = 0; j0 < n_jobs; j0 += 32768) {  // (the grid's second dimension holds 65535)
            const unsigned gy = (unsigned)std::min<size_t>(n_jobs - j0, 32768);
            hipLaunchKernelGGL((gemv_units_int_kernel<KIND, MAXP, true>), dim3(gx, gy), dim3(512), shmem, s, wm->dev, wm->layout.row_stride,
                               (int)rows_e, (int)wm->cols, aq, ad, m ? y2 : y, UnitsJobs{ids, n_experts, (int)j0, act_div, nullptr, nullptr, 0});
            FRK_LAUNCH_CHECK("gemv_units_int (jobs)");
        }
    }
    return FRK_OK;
}
template <int KIND>
static int launch_gemv_units_jobs_kind(const frk_weights *w, const frk_weights *w2, size_t rows_e, int n_experts, const int32_t *ids,
                                       size_t n_jobs, int act_div, const int8_t *aq, const float *ad, float *y, float *y2, hipStream_t s) {
    const size_t per_lane = (w->layout.row_stride / 16 + 63) / 64;
    if (per_lane <= 3) return launch_gemv_units_jobs_as<KIND, 3>(w, w2, rows_e, n_experts, ids, n_jobs, act_div, aq, ad, y, y2, s);
    if (per_lane <= 6) return launch_gemv_units_jobs_as<KIND, 6>(w, w2, rows_e, n_experts, ids, n_jobs, act_div, aq, ad, y, y2, s);
    return launch_gemv_units_jobs_as<KIND, 12>(w, w2, rows_e, n_experts, ids, n_jobs, act_div, aq, ad, y, y2, s);
}
// y[job][rows_e] = W[expert ids[job]] . activation row job / act_div, on the integer tier; w stacks the experts.
// With w2 (a stack of the same kind and shape: gate and up), y2 the same over w2, in the same launch where the grid
// holds both.
int launch_gemv_units_int_jobs(const frk_weights *w, const frk_weights *w2, size_t rows_e, int n_experts, const int32_t *ids,
                               size_t n_jobs, int act_div, const int8_t *aq, const float *ad, float *y, float *y2, hipStream_t s) {
    if (!gemv_units_int_fits(w))
        return set_error(FRK_ERR_UNSUPPORTED, "the integer GEMV of quant kind %d does not take rows of %zu columns", w->kind, w->cols);
    if (w2 && (w2->kind != w->kind || w2->rows != w->rows || w2->cols != w->cols || w2->layout.row_stride != w->layout.row_stride))
        return set_error(FRK_ERR_SHAPE, "two stacks in one launch must agree in kind and shape");
    if (w->kind == FRK_KIND_Q5_0)
        return launch_gemv_units_jobs_kind<FRK_KIND_Q5_0>(w, w2, rows_e, n_experts, ids, n_jobs, act_div, aq, ad, y, y2, s);
    if (w->kind == FRK_KIND_IQ4_XS)
        return launch_gemv_units_jobs_kind<FRK_KIND_IQ4_XS>(w, w2, rows_e, n_experts, ids, n_jobs, act_div, aq, ad, y, y2, s);
    return launch_gemv_units_jobs_kind<FRK_KIND_MXFP4>(w, w2, rows_e, n_experts, ids, n_jobs, act_div, aq, ad, y, y2, s);
}
template <int KIND>
static int launch_gemv_units_int_kind(const frk_weights *w, const int8_t *aq, const float *ad, float *y, hipStream_t s) {
    const size_t per_lane = (w->layout.row_stride / 16 + 63) / 64;
    if (per_lane <= 3) return launch_gemv_units_int_as<KIND, 3>(w, aq, ad, y, s);
    if (per_lane <= 6) return launch_gemv_units_int_as<KIND, 6>(w, aq, ad, y, s);
    return launch_gemv_units_int_as<KIND, 12>(w, aq, ad, y, s);
}
int launch_gemv_units_int(const frk_weights *w, const int8_t *aq, const float *ad, float *y, hipStream_t s) {
    if (!gemv_units_int_fits(w))
        return set_error(FRK_ERR_UNSUPPORTED, "the integer GEMV of quant kind %d takes rows of at most %d bytes (%zu columns)", w->kind,
                         12 * 1024, w->cols);
    if (w->kind == FRK_KIND_Q5_0) return launch_gemv_units_int_kind<FRK_KIND_Q5_0>(w, aq, ad, y, s);
    if (w->kind == FRK_KIND_IQ4_XS) return launch_gemv_units_int_kind<FRK_KIND_IQ4_XS>(w, aq, ad, y, s);
    return launch_gemv_units_int_kind<FRK_KIND_MXFP4>(w, aq, ad, y, s);
}

// ---- the batched integer path of Q5_0 / MXFP4: the codes as signed bytes and the scales as f16, in the planar
// form the Q8_0 matrix-core GEMM reads (one v_mfma_i32_32x32x32_i8 per block, the scales' outer product by an f16
// MFMA).  Q5_0's scale is an f16 already; MXFP4's halved E8M0 scale 2^(e - 128) is one for e in 104..143. ----
template <int KIND>
__global__ __launch_bounds__(256) void units_to_q8_0_planar_kernel(const uint8_t *__restrict__ W, size_t row_stride, size_t rows,
                                                                  size_t units, uint8_t *__restrict__ dst, size_t dst_stride,
                                                                  size_t off_d) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * units) return;
    const size_t r = i / units, u = i % units;
    uint32_t c[8];
    float scale;
    int scale_i;
    unit_codes<KIND>(W + r * row_stride, (int)u, c, scale, scale_i);
    uint4 *q = reinterpret_cast<uint4 *>(dst + r * dst_stride + u * 32);
    q[0] = make_uint4(c[0], c[1], c[2], c[3]);
    q[1] = make_uint4(c[4], c[5], c[6], c[7]);
    reinterpret_cast<uint16_t *>(dst + r * dst_stride + off_d)[u] = f2h_bits(scale);
}
int launch_units_to_q8_0_planar(const frk_weights *w, uint8_t *dst, size_t dst_stride, size_t off_d, hipStream_t s) {
    const size_t units = w->cols / 32;
    const unsigned g = (unsigned)((w->rows * units + 255) / 256);
    if (w->kind == FRK_KIND_Q5_0)
        hipLaunchKernelGGL((units_to_q8_0_planar_kernel<FRK_KIND_Q5_0>), dim3(g), dim3(256), 0, s, w->dev, w->layout.row_stride, w->rows,
                           units, dst, dst_stride, off_d);
    else if (w->kind == FRK_KIND_MXFP4)
        hipLaunchKernelGGL((units_to_q8_0_planar_kernel<FRK_KIND_MXFP4>), dim3(g), dim3(256), 0, s, w->dev, w->layout.row_stride, w->rows,
                           units, dst, dst_stride, off_d);
    else
        return set_error(FRK_ERR_UNSUPPORTED, "quant kind %d has no Q8_0 planar form", w->kind);
    FRK_LAUNCH_CHECK("units_to_q8_0_planar");
    return FRK_OK;
}

// IQ4_XS into the form the sub-scaled matrix-core GEMM reads: the codebook's signed bytes [cols], then per block of
// 256 a 16-byte slot -- the eight block scales ls - 32 as signed bytes, the f16 d, zeros.
__global__ __launch_bounds__(256) void iq4_xs_to_sub_planar_kernel(const uint8_t *__restrict__ W, size_t row_stride, size_t rows,
                                                                  size_t units, uint8_t *__restrict__ dst, size_t dst_stride,
                                                                  size_t off_d) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * units) return;
    const size_t r = i / units, u = i % units;
    uint32_t c[8];
    float scale;
    int scale_i;
    unit_codes<FRK_KIND_IQ4_XS>(W + r * row_stride, (int)u, c, scale, scale_i);
    uint4 *q = reinterpret_cast<uint4 *>(dst + r * dst_stride + u * 32);
    q[0] = make_uint4(c[0], c[1], c[2], c[3]);
    q[1] = make_uint4(c[4], c[5], c[6], c[7]);
    uint8_t *slot = dst + r * dst_stride + off_d + (u >> 3) * 16;
    slot[u & 7] = (uint8_t)(int8_t)scale_i;
    if ((u & 7) == 0) {
        reinterpret_cast<uint16_t *>(slot)[4] = f2h_bits(scale);  // (d is an f16 value: the bits it came from)
        reinterpret_cast<uint16_t *>(slot)[5] = 0;
        reinterpret_cast<uint32_t *>(slot)[3] = 0;
    }
}
int launch_iq4_xs_to_sub_planar(const frk_weights *w, uint8_t *dst, size_t dst_stride, size_t off_d, hipStream_t s) {
    if (w->kind != FRK_KIND_IQ4_XS) return set_error(FRK_ERR_UNSUPPORTED, "quant kind %d has no sub-scaled planar form", w->kind);
    const size_t units = w->cols / 32;
    const unsigned g = (unsigned)((w->rows * units + 255) / 256);
    hipLaunchKernelGGL(iq4_xs_to_sub_planar_kernel, dim3(g), dim3(256), 0, s, w->dev, w->layout.row_stride, w->rows, units, dst,
                       dst_stride, off_d);
    FRK_LAUNCH_CHECK("iq4_xs_to_sub_planar");
    return FRK_OK;
}

__global__ __launch_bounds__(256) void mxfp4_scale_range_kernel(const uint8_t *__restrict__ W, size_t row_stride, size_t rows, size_t units,
                                                               int *__restrict__ range) {
    int lo = 255, hi = 0;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < rows * units; i += (size_t)gridDim.x * 256) {
        const int e = W[(i / units) * row_stride + (i % units) * MXFP4_BYTES];
        lo = min(lo, e);
        hi = max(hi, e);
    }
    for (int m = 32; m > 0; m >>= 1) {
        lo = min(lo, __shfl_xor(lo, m));
        hi = max(hi, __shfl_xor(hi, m));
    }
    if ((threadIdx.x & 63) == 0) {
        atomicMin(&range[0], lo);
        atomicMax(&range[1], hi);
    }
}
int mxfp4_scale_range(const frk_weights *w, int *e_min, int *e_max, hipStream_t s) {
    int *range = nullptr;
    FRK_HIP_TRY(hipMalloc((void **)&range, 8));
    int h[2] = {255, 0};
    hipError_t e = hipMemcpyAsync(range, h, 8, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) {
        const size_t units = w->cols / 32;
        const unsigned g = (unsigned)std::min<size_t>((w->rows * units + 255) / 256, 4096);
        hipLaunchKernelGGL(mxfp4_scale_range_kernel, dim3(g), dim3(256), 0, s, w->dev, w->layout.row_stride, w->rows, units, range);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(h, range, 8, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)hipFree(range);
    if (e != hipSuccess) return set_error(FRK_ERR_HIP, "mxfp4 scale range: %s", hipGetErrorString(e));
    *e_min = h[0];
    *e_max = h[1];
    return FRK_OK;
}

bool units_have_planar_form(const frk_weights *w) {
    return w->kind == FRK_KIND_Q5_0 || w->kind == FRK_KIND_IQ4_XS ||
           (w->kind == FRK_KIND_MXFP4 && w->e8m0_min >= 104 && w->e8m0_max <= 143);
}
size_t units_planar_bytes(size_t rows, size_t cols) { return round_up(layout_for(FRK_KIND_Q8_0, cols).row_stride * rows + 256, 256); }
int launch_units_decode(const frk_weights *w, uint8_t *dst, hipStream_t s) {
    const Layout planar = layout_for(FRK_KIND_Q8_0, w->cols);
    return w->kind == FRK_KIND_IQ4_XS ? launch_iq4_xs_to_sub_planar(w, dst, planar.row_stride, planar.off_a, s)
                                      : launch_units_to_q8_0_planar(w, dst, planar.row_stride, planar.off_a, s);
}
int units_decoded(const frk_weights *w, uint8_t *room, hipStream_t s, const uint8_t **out) {
    if (const uint8_t *kept = w->decoded.load(std::memory_order_acquire)) {
        *out = kept;
        return FRK_OK;
    }
    *out = room;
    return launch_units_decode(w, room, s);
}

}  // namespace frk
