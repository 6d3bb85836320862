// Q5_0, IQ4_XS and MXFP4 (GGUF block form): dequantizer / row gather and the decode GEMV on the f32
// activation -- the kinds behind the reference's per-kind seam that the Q4_K_M model family does not use
// (crates/frink-cuda/src/mul_mm.rs:146-205; CPU forms dequant_q5_0 / dot_q5_0_f32,
// crates/frink-quant/src/lib.rs:4356-4418, dequant_iq4_xs / dot_iq4_xs_f32 :4860-4934, the E8M0 x E2M1
// arithmetic of dequant_mxfp4_row / dot_mxfp4_row_f32 :4947-5040 over 17-byte GGUF blocks :5560-5570).
// The resident copy keeps the GGUF bytes of a row in place (rows start 16-byte aligned); a weight is the
// dequantizer's value bit for bit.  The GEMV is the f32 dot of the reference's decode path: a wavefront
// per row, a lane per unit of 32 weights, the activation staged in LDS; the integer tier of these kinds
// (Q8_0 / Q8_K activations, crates/frink-quant/src/legacy_q8.rs, iq4_xs_q8.rs) is not built.
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

}  // namespace frk
