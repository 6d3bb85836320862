// Decode GEMV of the K-quants as the reference's default x86 decode path computes it: every weight
// dequantized and multiplied by the f32 activation, no activation quantization (WeightMatrix::dot,
// crates/frink-core/src/weight_matrix.rs:2044-2048 -> dot_q4_k_f32 / dot_q5_k_f32 / dot_q6_k_f32,
// crates/frink-quant/src/lib.rs:370-415, 461-515, 558-605).  A weight is the dequantizer's value bit for
// bit (d * sc * q - dmin * m, rounded where the reference rounds); the products are summed per lane and
// then across the wavefront, which is not the reference's left-to-right order: results agree with it
// within float summation order.
//
// A wavefront per weight row, a lane per unit of 32 weights (a sub-block of Q4_K / Q5_K, two 16-weight
// groups of Q6_K), units 64 apart; the activation (cols floats, up to 64 KB) is staged in LDS once per
// workgroup of eight rows at a time.  The work is a stream over the weights like the integer GEMVs, at
// four times the arithmetic; it is here for the path's numerics, not as the fast path.
#include "frk_device.hpp"

namespace frk {

template <int KIND>
__device__ __forceinline__ float unit_dot_f32(const uint8_t *__restrict__ row, const Layout &lay, int u, const float *__restrict__ xs) {
    const int b = u >> 3, sub = u & 7;
    const float4 *x4 = reinterpret_cast<const float4 *>(xs + (size_t)u * 32);
    float acc = 0.0f;
    if (KIND == FRK_KIND_Q4_K || KIND == FRK_KIND_Q5_K) {
        constexpr int BB = KIND == FRK_KIND_Q4_K ? Q4_K_BYTES : Q5_K_BYTES;
        constexpr int QS = KIND == FRK_KIND_Q4_K ? 16 : 48;
        const uint8_t *blk = row + (size_t)b * BB;
        const uint4 h = *reinterpret_cast<const uint4 *>(blk);
        const uint8_t *s = reinterpret_cast<const uint8_t *>(&h) + 4;
        int sc, m;
        if (sub < 4) {
            sc = s[sub] & 63;
            m = s[sub + 4] & 63;
        } else {
            sc = (s[sub + 4] & 0x0F) | ((s[sub - 4] >> 6) << 4);
            m = (s[sub + 4] >> 4) | ((s[sub] >> 6) << 4);
        }
        const float d1 = h2f(h.x & 0xffffu) * (float)sc, min1 = h2f(h.x >> 16) * (float)m;
        const uint4 qa = *reinterpret_cast<const uint4 *>(blk + QS + (sub >> 1) * 32);
        const uint4 qb = *reinterpret_cast<const uint4 *>(blk + QS + (sub >> 1) * 32 + 16);
        uint4 fa = make_uint4(0, 0, 0, 0), fb = fa;
        if (KIND == FRK_KIND_Q5_K) {  // the fifth bits: bit `sub` of qh[within]
            fa = *reinterpret_cast<const uint4 *>(blk + 16);
            fb = *reinterpret_cast<const uint4 *>(blk + 32);
        }
        const uint32_t qw[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const uint32_t fw[8] = {fa.x, fa.y, fa.z, fa.w, fb.x, fb.y, fb.z, fb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t nib = ((sub & 1) ? (qw[i] >> 4) : qw[i]) & 0x0f0f0f0fu;
            const uint32_t code = KIND == FRK_KIND_Q5_K ? nib | (((fw[i] >> sub) & 0x01010101u) << 4) : nib;
            const float4 xv = x4[i];
            acc = fmaf(__fsub_rn(__fmul_rn(d1, (float)(code & 0xff)), min1), xv.x, acc);
            acc = fmaf(__fsub_rn(__fmul_rn(d1, (float)((code >> 8) & 0xff)), min1), xv.y, acc);
            acc = fmaf(__fsub_rn(__fmul_rn(d1, (float)((code >> 16) & 0xff)), min1), xv.z, acc);
            acc = fmaf(__fsub_rn(__fmul_rn(d1, (float)(code >> 24)), min1), xv.w, acc);
        }
    } else {  // Q6_K, planar resident layout: elements 32 sub .. 32 sub + 31 of block b
        const int half = sub >> 2, quarter = sub & 3;
        const uint8_t *ql = row + (size_t)b * 128 + half * 64 + (quarter & 1) * 32;
        const uint8_t *qh = row + lay.off_a + (size_t)b * 64 + half * 32;
        const uint4 la = *reinterpret_cast<const uint4 *>(ql), lb = *reinterpret_cast<const uint4 *>(ql + 16);
        const uint4 ha = *reinterpret_cast<const uint4 *>(qh), hb = *reinterpret_cast<const uint4 *>(qh + 16);
        const uint16_t scw = *reinterpret_cast<const uint16_t *>(row + lay.off_b + (size_t)b * 16 + sub * 2);
        const float d = h2f(*reinterpret_cast<const uint16_t *>(row + lay.off_c + (size_t)b * 2));
        const float ds0 = __fmul_rn(d, (float)(int)(int8_t)(scw & 0xff)), ds1 = __fmul_rn(d, (float)(int)(int8_t)(scw >> 8));
        const uint32_t lw[8] = {la.x, la.y, la.z, la.w, lb.x, lb.y, lb.z, lb.w};
        const uint32_t hw[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t lo = ((quarter & 2) ? (lw[i] >> 4) : lw[i]) & 0x0f0f0f0fu;
            const uint32_t code = lo | (((hw[i] >> (2 * quarter)) & 0x03030303u) << 4);
            const float ds = i < 4 ? ds0 : ds1;  // (the group of 16 the element belongs to)
            const float4 xv = x4[i];
            acc = fmaf(__fmul_rn(ds, (float)((int)(code & 0xff) - 32)), xv.x, acc);
            acc = fmaf(__fmul_rn(ds, (float)((int)((code >> 8) & 0xff) - 32)), xv.y, acc);
            acc = fmaf(__fmul_rn(ds, (float)((int)((code >> 16) & 0xff) - 32)), xv.z, acc);
            acc = fmaf(__fmul_rn(ds, (float)((int)(code >> 24) - 32)), xv.w, acc);
        }
    }
    return acc;
}

template <int KIND>
__global__ __launch_bounds__(512) void gemv_kquant_f32_kernel(const uint8_t *__restrict__ W, Layout lay, int rows, int cols,
                                                             const float *__restrict__ x, float *__restrict__ y) {
    extern __shared__ uint4 smem_f32dot[];
    float *xs = reinterpret_cast<float *>(smem_f32dot);
    for (int i = threadIdx.x; i < cols / 4; i += 512) reinterpret_cast<float4 *>(xs)[i] = reinterpret_cast<const float4 *>(x)[i];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int units = cols / 32;
    for (int r = (int)blockIdx.x * 8 + wave; r < rows; r += (int)gridDim.x * 8) {
        const uint8_t *row = W + (size_t)r * lay.row_stride;
        float acc = 0.0f;
        for (int u = lane; u < units; u += 64) acc += unit_dot_f32<KIND>(row, lay, u, xs);
        acc = part_sum<64>(acc);
        if (lane == 0) y[r] = acc;
    }
}

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

bool kquant_f32_gemv_fits(const frk_weights *w) {
    return (w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K || w->kind == FRK_KIND_Q6_K) && w->cols * 4 <= 64 * 1024;
}

template <int KIND>
static int launch_kquant_f32(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const size_t shmem = w->cols * 4;
    const unsigned grid = (unsigned)std::min<size_t>((w->rows + 7) / 8, 2048);
    hipLaunchKernelGGL((gemv_kquant_f32_kernel<KIND>), dim3(grid), dim3(512), shmem, s, w->dev, w->layout, (int)w->rows, (int)w->cols,
                       x, y);
    FRK_LAUNCH_CHECK("gemv_kquant_f32");
    return FRK_OK;
}

// y = W x with dequantized weights and the f32 activation (rows of at most 16384 columns)
int launch_gemv_kquant_f32(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    if (w->kind == FRK_KIND_Q4_K) return launch_kquant_f32<FRK_KIND_Q4_K>(w, x, y, s);
    if (w->kind == FRK_KIND_Q5_K) return launch_kquant_f32<FRK_KIND_Q5_K>(w, x, y, s);
    return launch_kquant_f32<FRK_KIND_Q6_K>(w, x, y, s);
}

}  // namespace frk
