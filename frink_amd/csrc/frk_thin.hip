// Thin batched GEMM (2..8 activation rows, batched decode): y[b][r] = sum_k W[r][k] * x[b][k].
//
// Still bandwidth-bound: the weights are read from HBM once for the whole batch, unpacked once per
// 64-weight unit, and multiplied against each of the NB quantized activation rows, which live in
// LDS (NB * cols bytes of quants plus their sums and scales).  Arithmetic per (row, activation) is
// exactly the decode GEMV's (dot_q4_k_q8 / dot_q6_k_q8, crates/frink-quant/src/lib.rs:822-869,
// 1069-1110), so a batch row's result equals the GEMV of that row.  This is the shape the
// reference runs as `batch` separate matvecs (crates/frink-core/src/weight_matrix.rs:2636-2652).
// Workgroups are 16 wavefronts so that one copy of the activations serves 16 weight rows at a time.
#include "frk_device.hpp"

namespace frk {

constexpr int THIN_THREADS = 1024;

// Stages NB Q8_K activation rows in LDS: quants | sums over GROUP*16 quants (as int) | block scales.
// Rows past `batch` repeat the last one (their results are not stored).
template <int NB, int SUMS_PER_BLOCK>
__device__ __forceinline__ void stage_acts(uint4 *smem, int nb, int batch, const int8_t *aq, const float *ad,
                                           const int16_t *absums, int8_t *&sq, int *&sbs, float *&sd) {
    sq = reinterpret_cast<int8_t *>(smem);
    sbs = reinterpret_cast<int *>(sq + (size_t)NB * nb * 256);
    sd = reinterpret_cast<float *>(sbs + (size_t)NB * nb * SUMS_PER_BLOCK);
    constexpr int FOLD = 16 / SUMS_PER_BLOCK;  // bsums folded per stored sum
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const int src = min(b, batch - 1);
        const uint4 *q4 = reinterpret_cast<const uint4 *>(aq + (size_t)src * nb * 256);
        for (int i = threadIdx.x; i < nb * 16; i += THIN_THREADS) smem[(size_t)b * nb * 16 + i] = q4[i];
        const int16_t *bs = absums + (size_t)src * nb * 16;
        for (int i = threadIdx.x; i < nb * SUMS_PER_BLOCK; i += THIN_THREADS) {
            int v = 0;
#pragma unroll
            for (int f = 0; f < FOLD; f++) v += (int)bs[FOLD * i + f];
            sbs[(size_t)b * nb * SUMS_PER_BLOCK + i] = v;
        }
        for (int i = threadIdx.x; i < nb; i += THIN_THREADS) sd[(size_t)b * nb + i] = ad[(size_t)src * nb + i];
    }
    __syncthreads();
}

template <int LPR, int NB>
__global__ __launch_bounds__(THIN_THREADS) void thin_q4_k_kernel(const uint8_t *__restrict__ W, size_t row_stride,
                                                                 int rows, int nb, int batch,
                                                                 const int8_t *__restrict__ aq,
                                                                 const float *__restrict__ ad,
                                                                 const int16_t *__restrict__ absums,
                                                                 float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    int8_t *sq;
    int *sbs;
    float *sd;
    stage_acts<NB, 8>(smem, nb, batch, aq, ad, absums, sq, sbs, sd);

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 4;
    const long n_waves = (long)gridDim.x * (THIN_THREADS / 64);
    for (long r0 = ((long)blockIdx.x * (THIN_THREADS / 64) + (threadIdx.x >> 6)) * PARTS; r0 < rows;
         r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) acc[b] = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * row_stride;
            for (int u = l; u < units; u += LPR) {
                const int blk_i = u >> 2, p = u & 3;
                const uint4 *blk = reinterpret_cast<const uint4 *>(row + (size_t)blk_i * Q4_K_BYTES);
                const uint4 h = blk[0];
                const uint4 qa = blk[1 + 2 * p], qb = blk[2 + 2 * p];
                // 6-bit scales and mins of sub-blocks 2p and 2p+1 (q4_k_scale_min, lib.rs:321-330)
                uint32_t scw, mw;
                if (p < 2) {
                    scw = h.y & 0x3f3f3f3fu;
                    mw = h.z & 0x3f3f3f3fu;
                } else {
                    scw = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);
                    mw = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
                }
                const int sh = (p & 1) * 16;
                const int sc1 = (scw >> sh) & 0xff, sc2 = (scw >> (sh + 8)) & 0xff;
                const int m1 = (mw >> sh) & 0xff, m2 = (mw >> (sh + 8)) & 0xff;
                const float d = h2f(h.x & 0xffffu), dmin = h2f(h.x >> 16);
                const uint32_t lo[8] = {qa.x & 0x0f0f0f0fu, qa.y & 0x0f0f0f0fu, qa.z & 0x0f0f0f0fu, qa.w & 0x0f0f0f0fu,
                                        qb.x & 0x0f0f0f0fu, qb.y & 0x0f0f0f0fu, qb.z & 0x0f0f0f0fu, qb.w & 0x0f0f0f0fu};
                const uint32_t hi[8] = {(qa.x >> 4) & 0x0f0f0f0fu, (qa.y >> 4) & 0x0f0f0f0fu, (qa.z >> 4) & 0x0f0f0f0fu,
                                        (qa.w >> 4) & 0x0f0f0f0fu, (qb.x >> 4) & 0x0f0f0f0fu, (qb.y >> 4) & 0x0f0f0f0fu,
                                        (qb.z >> 4) & 0x0f0f0f0fu, (qb.w >> 4) & 0x0f0f0f0fu};
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    const uint4 *a = reinterpret_cast<const uint4 *>(sq + ((size_t)b * nb + blk_i) * 256 + p * 64);
                    const uint4 a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
                    int is1 = 0, is2 = 0;
                    is1 = dot4(lo[0], a0.x, is1);
                    is1 = dot4(lo[1], a0.y, is1);
                    is1 = dot4(lo[2], a0.z, is1);
                    is1 = dot4(lo[3], a0.w, is1);
                    is1 = dot4(lo[4], a1.x, is1);
                    is1 = dot4(lo[5], a1.y, is1);
                    is1 = dot4(lo[6], a1.z, is1);
                    is1 = dot4(lo[7], a1.w, is1);
                    is2 = dot4(hi[0], a2.x, is2);
                    is2 = dot4(hi[1], a2.y, is2);
                    is2 = dot4(hi[2], a2.z, is2);
                    is2 = dot4(hi[3], a2.w, is2);
                    is2 = dot4(hi[4], a3.x, is2);
                    is2 = dot4(hi[5], a3.y, is2);
                    is2 = dot4(hi[6], a3.z, is2);
                    is2 = dot4(hi[7], a3.w, is2);
                    const int *bs = sbs + ((size_t)b * nb + blk_i) * 8 + 2 * p;
                    const int s1 = __mul24(sc1, is1) + __mul24(sc2, is2);
                    const int s2 = __mul24(m1, bs[0]) + __mul24(m2, bs[1]);
                    const float da = sd[(size_t)b * nb + blk_i];
                    acc[b] += (d * da) * (float)s1 - (dmin * da) * (float)s2;
                }
            }
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float v = part_sum<LPR>(acc[b]);
            if (l == 0 && r < rows && b < batch) y[(size_t)b * rows + r] = v;
        }
    }
}

template <int LPR, int NB>
__global__ __launch_bounds__(THIN_THREADS) void thin_q6_k_kernel(const uint8_t *__restrict__ W, Layout lay, int rows,
                                                                 int nb, int batch, const int8_t *__restrict__ aq,
                                                                 const float *__restrict__ ad,
                                                                 const int16_t *__restrict__ absums,
                                                                 float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    int8_t *sq;
    int *sbs;
    float *sd;
    stage_acts<NB, 16>(smem, nb, batch, aq, ad, absums, sq, sbs, sd);

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 4;
    const long n_waves = (long)gridDim.x * (THIN_THREADS / 64);
    for (long r0 = ((long)blockIdx.x * (THIN_THREADS / 64) + (threadIdx.x >> 6)) * PARTS; r0 < rows;
         r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) acc[b] = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * lay.row_stride;
            for (int u = l; u < units; u += LPR) {
                // unit = (block, half h, 16-lane column t), as in the decode GEMV
                const int blk_i = u >> 2, h = (u >> 1) & 1, t = u & 1;
                const uint4 qla = *reinterpret_cast<const uint4 *>(row + (size_t)blk_i * 128 + h * 64 + t * 16);
                const uint4 qlb = *reinterpret_cast<const uint4 *>(row + (size_t)blk_i * 128 + h * 64 + 32 + t * 16);
                const uint4 qh = *reinterpret_cast<const uint4 *>(row + lay.off_a + (size_t)blk_i * 64 + h * 32 + t * 16);
                const uint2 scv = *reinterpret_cast<const uint2 *>(row + lay.off_b + (size_t)blk_i * 16 + h * 8);
                const float d = h2f(*reinterpret_cast<const uint16_t *>(row + lay.off_c + (size_t)blk_i * 2));
                uint32_t w1[4], w2[4], w3[4], w4[4];  // the four 16-weight groups, 6-bit codes (0..63)
#define FRK_Q6_UNPACK(i, c)                                            \
    w1[i] = (qla.c & 0x0f0f0f0fu) | ((qh.c << 4) & 0x30303030u);        \
    w2[i] = (qlb.c & 0x0f0f0f0fu) | ((qh.c << 2) & 0x30303030u);        \
    w3[i] = ((qla.c >> 4) & 0x0f0f0f0fu) | (qh.c & 0x30303030u);        \
    w4[i] = ((qlb.c >> 4) & 0x0f0f0f0fu) | ((qh.c >> 2) & 0x30303030u);
                FRK_Q6_UNPACK(0, x)
                FRK_Q6_UNPACK(1, y)
                FRK_Q6_UNPACK(2, z)
                FRK_Q6_UNPACK(3, w)
#undef FRK_Q6_UNPACK
                const uint32_t slo = t ? (scv.x >> 8) : scv.x, shi = t ? (scv.y >> 8) : scv.y;
                const int s1 = (int)(int8_t)(slo & 0xff), s2 = (int)(int8_t)((slo >> 16) & 0xff);
                const int s3 = (int)(int8_t)(shi & 0xff), s4 = (int)(int8_t)((shi >> 16) & 0xff);
                const int g = h * 8 + t;
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    const int8_t *abase = sq + ((size_t)b * nb + blk_i) * 256 + h * 128 + t * 16;
                    const uint4 a0 = *reinterpret_cast<const uint4 *>(abase);
                    const uint4 a1 = *reinterpret_cast<const uint4 *>(abase + 32);
                    const uint4 a2 = *reinterpret_cast<const uint4 *>(abase + 64);
                    const uint4 a3 = *reinterpret_cast<const uint4 *>(abase + 96);
                    int d1 = 0, d2 = 0, d3 = 0, d4 = 0;
                    d1 = dot4(w1[0], a0.x, d1);
                    d1 = dot4(w1[1], a0.y, d1);
                    d1 = dot4(w1[2], a0.z, d1);
                    d1 = dot4(w1[3], a0.w, d1);
                    d2 = dot4(w2[0], a1.x, d2);
                    d2 = dot4(w2[1], a1.y, d2);
                    d2 = dot4(w2[2], a1.z, d2);
                    d2 = dot4(w2[3], a1.w, d2);
                    d3 = dot4(w3[0], a2.x, d3);
                    d3 = dot4(w3[1], a2.y, d3);
                    d3 = dot4(w3[2], a2.z, d3);
                    d3 = dot4(w3[3], a2.w, d3);
                    d4 = dot4(w4[0], a3.x, d4);
                    d4 = dot4(w4[1], a3.y, d4);
                    d4 = dot4(w4[2], a3.z, d4);
                    d4 = dot4(w4[3], a3.w, d4);
                    // the -32 of the 6-bit code folded as -32 * (sum of the 16 activation quants)
                    const int *bs = sbs + ((size_t)b * nb + blk_i) * 16 + g;
                    const int isum = s1 * (d1 - 32 * bs[0]) + s2 * (d2 - 32 * bs[2]) + s3 * (d3 - 32 * bs[4]) +
                                     s4 * (d4 - 32 * bs[6]);
                    acc[b] += (d * sd[(size_t)b * nb + blk_i]) * (float)isum;
                }
            }
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float v = part_sum<LPR>(acc[b]);
            if (l == 0 && r < rows && b < batch) y[(size_t)b * rows + r] = v;
        }
    }
}

// ------------------------------------------------------------------ launchers

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

static int thin_lanes_per_row(int units) { return units > 32 ? 64 : units > 16 ? 32 : 16; }

static unsigned thin_grid(size_t rows, int lpr) {
    const size_t rows_per_wg = (THIN_THREADS / 64) * (size_t)(64 / lpr);
    size_t g = (rows + rows_per_wg - 1) / rows_per_wg;
    if (g > 512) g = 512;  // two workgroups per CU at most; wavefronts loop over rows
    return (unsigned)(g < 1 ? 1 : g);
}

constexpr size_t THIN_LDS_LIMIT = 150 * 1024;

template <int LPR, int NB>
static int launch_thin_one(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    const bool q4 = w->kind == FRK_KIND_Q4_K;
    const size_t shmem = (size_t)NB * nb * (256 + (q4 ? 8 : 16) * 4 + 4);
    const unsigned grid = thin_grid(w->rows, LPR);
    if (q4) {
        static bool sized = false;
        if (shmem > 65536 && !sized) {
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_q4_k_kernel<LPR, NB>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)THIN_LDS_LIMIT));
            sized = true;
        }
        hipLaunchKernelGGL((thin_q4_k_kernel<LPR, NB>), dim3(grid), dim3(THIN_THREADS), shmem, s, w->dev,
                           w->layout.row_stride, (int)w->rows, nb, batch, a.q, a.d, a.bsums, y);
    } else {
        static bool sized = false;
        if (shmem > 65536 && !sized) {
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_q6_k_kernel<LPR, NB>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)THIN_LDS_LIMIT));
            sized = true;
        }
        hipLaunchKernelGGL((thin_q6_k_kernel<LPR, NB>), dim3(grid), dim3(THIN_THREADS), shmem, s, w->dev, w->layout,
                           (int)w->rows, nb, batch, a.q, a.d, a.bsums, y);
    }
    FRK_LAUNCH_CHECK("thin gemm");
    return FRK_OK;
}

template <int NB>
static int launch_thin_nb(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const int lpr = thin_lanes_per_row((int)(w->cols / QK_K) * 4);
    if (lpr == 64) return launch_thin_one<64, NB>(w, batch, a, y, s);
    if (lpr == 32) return launch_thin_one<32, NB>(w, batch, a, y, s);
    return launch_thin_one<16, NB>(w, batch, a, y, s);
}

// Largest number of activation rows one launch can take for this matrix (LDS), at most 8.
int thin_gemm_max_batch(const frk_weights *w) {
    const size_t per_row = (w->cols / QK_K) * (256 + (w->kind == FRK_KIND_Q4_K ? 8 : 16) * 4 + 4);
    for (int nbatch = 8; nbatch >= 2; nbatch /= 2)
        if (per_row * nbatch <= THIN_LDS_LIMIT) return nbatch;
    return 0;
}

// y[batch][rows] for 1 <= batch <= thin_gemm_max_batch(w) quantized activation rows (K-quants).
int launch_thin_gemm(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    if (batch > 4) return launch_thin_nb<8>(w, batch, a, y, s);
    if (batch > 2) return launch_thin_nb<4>(w, batch, a, y, s);
    return launch_thin_nb<2>(w, batch, a, y, s);
}

}  // namespace frk
