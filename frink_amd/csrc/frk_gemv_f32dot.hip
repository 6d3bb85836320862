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
// four times the arithmetic; it is here for the path's numerics, not as the fast path (Q4_K 14336x4096: 16 us
// against 8 on the integer path).
#include "frk_device.hpp"

namespace frk {

// A unit's bytes as they come from memory: Q4_K / Q5_K -- the block's header, the 32 bytes that hold the
// sub-block's nibbles (Q5_K: and the block's 32 bytes of fifth bits); Q6_K -- 32 bytes of low nibbles, 32 of
// high bits, the two group scales and the block scale.
template <int KIND>
struct UnitRaw {
    uint4 h, qa, qb, fa, fb;
    uint32_t scw, dbits;
};
template <int KIND>
__device__ __forceinline__ void unit_load(UnitRaw<KIND> &R, const uint8_t *__restrict__ row, const Layout &lay, int u) {
    const int b = u >> 3, sub = u & 7;
    if (KIND == FRK_KIND_Q4_K || KIND == FRK_KIND_Q5_K) {
        constexpr int BB = KIND == FRK_KIND_Q4_K ? Q4_K_BYTES : Q5_K_BYTES;
        constexpr int QS = KIND == FRK_KIND_Q4_K ? 16 : 48;
        const uint8_t *blk = row + (size_t)b * BB;
        R.h = *reinterpret_cast<const uint4 *>(blk);
        R.qa = *reinterpret_cast<const uint4 *>(blk + QS + (sub >> 1) * 32);
        R.qb = *reinterpret_cast<const uint4 *>(blk + QS + (sub >> 1) * 32 + 16);
        if (KIND == FRK_KIND_Q5_K) {  // the fifth bits: bit `sub` of qh[within]
            R.fa = *reinterpret_cast<const uint4 *>(blk + 16);
            R.fb = *reinterpret_cast<const uint4 *>(blk + 32);
        }
    } else {  // Q6_K, planar resident layout: elements 32 sub .. 32 sub + 31 of block b
        const int half = sub >> 2, quarter = sub & 3;
        const uint8_t *ql = row + (size_t)b * 128 + half * 64 + (quarter & 1) * 32;
        const uint8_t *qh = row + lay.off_a + (size_t)b * 64 + half * 32;
        R.qa = *reinterpret_cast<const uint4 *>(ql), R.qb = *reinterpret_cast<const uint4 *>(ql + 16);
        R.fa = *reinterpret_cast<const uint4 *>(qh), R.fb = *reinterpret_cast<const uint4 *>(qh + 16);
        R.scw = *reinterpret_cast<const uint16_t *>(row + lay.off_b + (size_t)b * 16 + sub * 2);
        R.dbits = *reinterpret_cast<const uint16_t *>(row + lay.off_c + (size_t)b * 2);
    }
}
// The unit's 32 weights, each the dequantizer's value bit for bit, times the unit's 32 activations x4[0..7].
template <int KIND, class X4>
__device__ __forceinline__ float unit_dot_loaded(const UnitRaw<KIND> &R, int u, X4 x4) {
    const int sub = u & 7;
    float acc0 = 0.0f, acc1 = 0.0f, acc2 = 0.0f, acc3 = 0.0f;  // four chains: one would wait for itself 32 times
    if (KIND == FRK_KIND_Q4_K || KIND == FRK_KIND_Q5_K) {
        const uint4 h = R.h;
        // q4_k_scale_min (crates/frink-quant/src/lib.rs:321-330) on the twelve scale bytes h.y | h.z | h.w, by shifts
        // (indexing the bytes of a register by `sub` would put the header in scratch memory)
        const int sh = 8 * (sub & 3);
        const uint32_t by = (h.y >> sh) & 0xff, bz = (h.z >> sh) & 0xff, bw = (h.w >> sh) & 0xff;
        const int sc = sub < 4 ? (int)(by & 63) : (int)((bw & 0x0F) | ((by >> 6) << 4));
        const int m = sub < 4 ? (int)(bz & 63) : (int)((bw >> 4) | ((bz >> 6) << 4));
        const float d1 = h2f(h.x & 0xffffu) * (float)sc, min1 = h2f(h.x >> 16) * (float)m;
        const uint32_t qw[8] = {R.qa.x, R.qa.y, R.qa.z, R.qa.w, R.qb.x, R.qb.y, R.qb.z, R.qb.w};
        const uint32_t fw[8] = {R.fa.x, R.fa.y, R.fa.z, R.fa.w, R.fb.x, R.fb.y, R.fb.z, R.fb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t nib = ((sub & 1) ? (qw[i] >> 4) : qw[i]) & 0x0f0f0f0fu;
            const uint32_t code = KIND == FRK_KIND_Q5_K ? nib | (((fw[i] >> sub) & 0x01010101u) << 4) : nib;
            const float4 xv = x4[i];
            acc0 = fmaf(__fsub_rn(__fmul_rn(d1, (float)(code & 0xff)), min1), xv.x, acc0);
            acc1 = fmaf(__fsub_rn(__fmul_rn(d1, (float)((code >> 8) & 0xff)), min1), xv.y, acc1);
            acc2 = fmaf(__fsub_rn(__fmul_rn(d1, (float)((code >> 16) & 0xff)), min1), xv.z, acc2);
            acc3 = fmaf(__fsub_rn(__fmul_rn(d1, (float)(code >> 24)), min1), xv.w, acc3);
        }
    } else {
        const int quarter = sub & 3;
        const float d = h2f(R.dbits);
        const float ds0 = __fmul_rn(d, (float)(int)(int8_t)(R.scw & 0xff)), ds1 = __fmul_rn(d, (float)(int)(int8_t)(R.scw >> 8));
        const uint32_t lw[8] = {R.qa.x, R.qa.y, R.qa.z, R.qa.w, R.qb.x, R.qb.y, R.qb.z, R.qb.w};
        const uint32_t hw[8] = {R.fa.x, R.fa.y, R.fa.z, R.fa.w, R.fb.x, R.fb.y, R.fb.z, R.fb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t lo = ((quarter & 2) ? (lw[i] >> 4) : lw[i]) & 0x0f0f0f0fu;
            const uint32_t code = lo | (((hw[i] >> (2 * quarter)) & 0x03030303u) << 4);
            const float ds = i < 4 ? ds0 : ds1;  // (the group of 16 the element belongs to)
            const float4 xv = x4[i];
            acc0 = fmaf(__fmul_rn(ds, (float)((int)(code & 0xff) - 32)), xv.x, acc0);
            acc1 = fmaf(__fmul_rn(ds, (float)((int)((code >> 8) & 0xff) - 32)), xv.y, acc1);
            acc2 = fmaf(__fmul_rn(ds, (float)((int)((code >> 16) & 0xff) - 32)), xv.z, acc2);
            acc3 = fmaf(__fmul_rn(ds, (float)((int)(code >> 24) - 32)), xv.w, acc3);
        }
    }
    return (acc0 + acc1) + (acc2 + acc3);
}
template <int KIND>
__device__ __forceinline__ float unit_dot_f32(const uint8_t *__restrict__ row, const Layout &lay, int u, const float *__restrict__ xs) {
    UnitRaw<KIND> R;
    unit_load<KIND>(R, row, lay, u);
    return unit_dot_loaded<KIND>(R, u, reinterpret_cast<const float4 *>(xs + (size_t)u * 32));
}

// The same with the columns split between the wavefronts of a workgroup: wavefront w takes units 64w .. 64w+63
// (2048 columns) of the workgroup's R rows, a lane keeps its unit's 32 activations in registers (read straight from
// global memory: no copy in LDS, no barrier between the requests and the arithmetic) and all its rows' bytes are
// requested before the first is multiplied; the wavefronts' partial sums of a row meet in LDS at the end.
template <int KIND, int R>
__global__ __launch_bounds__(1024) void gemv_kquant_f32_cols_kernel(const uint8_t *__restrict__ W, Layout lay, int rows, int cols,
                                                                   const float *__restrict__ x, float *__restrict__ y) {
    extern __shared__ uint4 smem_f32dot[];
    float *parts = reinterpret_cast<float *>(smem_f32dot);  // [wavefront][row]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int units = cols / 32;
    const bool live = wave * 64 + lane < units;
    const int u = min(wave * 64 + lane, units - 1);  // (a lane past the end: the last unit again, not added)
    const int r0 = (int)blockIdx.x * R;
    float4 xv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) xv[i] = reinterpret_cast<const float4 *>(x + (size_t)u * 32)[i];
    UnitRaw<KIND> raw[R];
#pragma unroll
    for (int k = 0; k < R; k++) unit_load<KIND>(raw[k], W + (size_t)min(r0 + k, rows - 1) * lay.row_stride, lay, u);
#pragma unroll
    for (int k = 0; k < R; k++) {
        const float v = part_sum<64>(live ? unit_dot_loaded<KIND>(raw[k], u, xv) : 0.0f);
        if (lane == 0) parts[wave * R + k] = v;
    }
    __syncthreads();
    if ((int)threadIdx.x < R && r0 + (int)threadIdx.x < rows) {
        float v = 0.0f;
        for (int w = 0; w < waves; w++) v += parts[w * R + threadIdx.x];
        y[r0 + threadIdx.x] = v;
    }
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
    // Q4_K: the column form, four rows to a workgroup (14336x4096 16.2 us against 18.7, 4096x14336 16.9 / 19.0; Q5_K and
    // Q6_K, whose units are more registers and fit two rows, are behind the kernel below: 20.9 / 19.5 and 24.0 / 20.6)
    if (KIND == FRK_KIND_Q4_K) {
        constexpr int R = KIND == FRK_KIND_Q4_K ? 4 : 2;
        const int waves = (int)((w->cols / 32 + 63) / 64);
        hipLaunchKernelGGL((gemv_kquant_f32_cols_kernel<KIND, R>), dim3((unsigned)((w->rows + R - 1) / R)), dim3(64 * waves),
                           (size_t)waves * R * 4, s, w->dev, w->layout, (int)w->rows, (int)w->cols, x, y);
        FRK_LAUNCH_CHECK("gemv_kquant_f32_cols");
        return FRK_OK;
    }
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
