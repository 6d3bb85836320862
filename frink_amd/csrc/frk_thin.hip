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

// Where the 16-byte granule g of an activation row goes in LDS.  A lane reads four granules per unit
// and 64 lanes read 64 consecutive units, so granules are stored [piece k of a unit][unit]: the lanes
// of one read then touch consecutive 16-byte slots (reading them in place, 64 bytes apart, would be
// a four-way bank conflict).
//   Q4_K unit u = granules 4u .. 4u+3                            -> piece k = g & 3, unit = g >> 2
//   Q6_K unit u = (block, half h, column t): granules 16*block + 8h + t + {0, 2, 4, 6}
template <bool Q6>
__device__ __forceinline__ int granule_slot(int g, int units) {
    if (!Q6) return (g & 3) * units + (g >> 2);
    const int blk = g >> 4, h = (g >> 3) & 1, k = (g >> 1) & 3, t = g & 1;
    return k * units + (blk * 4 + h * 2 + t);
}

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
        for (int i = threadIdx.x; i < nb * 16; i += THIN_THREADS)
            smem[(size_t)b * nb * 16 + granule_slot<SUMS_PER_BLOCK == 16>(i, nb * 4)] = q4[i];
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

// Both kernels: LPR lanes share R consecutive weight rows (a wavefront works on 64/LPR such row
// groups at once) and walk them in units of 64 weights; a lane multiplies its unit of all R rows
// against the same slice of each activation row, so that slice is read from LDS once per R rows.

template <int LPR, int NB, int R>
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
    for (long g0 = ((long)blockIdx.x * (THIN_THREADS / 64) + (threadIdx.x >> 6)) * PARTS; g0 * R < rows;
         g0 += n_waves * PARTS) {
        const long r0 = (g0 + part) * R;  // this lane's first row of the group
        float acc[R][NB];
#pragma unroll
        for (int k = 0; k < R; k++)
#pragma unroll
            for (int b = 0; b < NB; b++) acc[k][b] = 0.0f;
        if (r0 < rows) {
            for (int u = l; u < units; u += LPR) {
                const int blk_i = u >> 2, p = u & 3;
                uint4 h[R], qa[R], qb[R];
#pragma unroll
                for (int k = 0; k < R; k++) {  // rows past the end repeat the last one; their results are dropped
                    const uint4 *blk = reinterpret_cast<const uint4 *>(
                        W + (size_t)min(r0 + k, (long)rows - 1) * row_stride + (size_t)blk_i * Q4_K_BYTES);
                    h[k] = blk[0];
                    qa[k] = blk[1 + 2 * p];
                    qb[k] = blk[2 + 2 * p];
                }
                const int sh = (p & 1) * 16;
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    const uint4 *a = smem + (size_t)b * nb * 16 + u;  // pieces k at [k][unit]
                    const uint4 a0 = a[0], a1 = a[units], a2 = a[2 * units], a3 = a[3 * units];
                    const int *bs = sbs + ((size_t)b * nb + blk_i) * 8 + 2 * p;
                    const int bs0 = bs[0], bs1 = bs[1];
                    const float da = sd[(size_t)b * nb + blk_i];
#pragma unroll
                    for (int k = 0; k < R; k++) {
                        // 6-bit scales and mins of sub-blocks 2p and 2p+1 (q4_k_scale_min, lib.rs:321-330)
                        uint32_t scw, mw;
                        if (p < 2) {
                            scw = h[k].y & 0x3f3f3f3fu;
                            mw = h[k].z & 0x3f3f3f3fu;
                        } else {
                            scw = (h[k].w & 0x0f0f0f0fu) | (((h[k].y >> 6) & 0x03030303u) << 4);
                            mw = ((h[k].w >> 4) & 0x0f0f0f0fu) | (((h[k].z >> 6) & 0x03030303u) << 4);
                        }
                        const int sc1 = (scw >> sh) & 0xff, sc2 = (scw >> (sh + 8)) & 0xff;
                        const int m1 = (mw >> sh) & 0xff, m2 = (mw >> (sh + 8)) & 0xff;
                        int is1 = 0, is2 = 0;
                        is1 = dot4(qa[k].x & 0x0f0f0f0fu, a0.x, is1);
                        is1 = dot4(qa[k].y & 0x0f0f0f0fu, a0.y, is1);
                        is1 = dot4(qa[k].z & 0x0f0f0f0fu, a0.z, is1);
                        is1 = dot4(qa[k].w & 0x0f0f0f0fu, a0.w, is1);
                        is1 = dot4(qb[k].x & 0x0f0f0f0fu, a1.x, is1);
                        is1 = dot4(qb[k].y & 0x0f0f0f0fu, a1.y, is1);
                        is1 = dot4(qb[k].z & 0x0f0f0f0fu, a1.z, is1);
                        is1 = dot4(qb[k].w & 0x0f0f0f0fu, a1.w, is1);
                        is2 = dot4((qa[k].x >> 4) & 0x0f0f0f0fu, a2.x, is2);
                        is2 = dot4((qa[k].y >> 4) & 0x0f0f0f0fu, a2.y, is2);
                        is2 = dot4((qa[k].z >> 4) & 0x0f0f0f0fu, a2.z, is2);
                        is2 = dot4((qa[k].w >> 4) & 0x0f0f0f0fu, a2.w, is2);
                        is2 = dot4((qb[k].x >> 4) & 0x0f0f0f0fu, a3.x, is2);
                        is2 = dot4((qb[k].y >> 4) & 0x0f0f0f0fu, a3.y, is2);
                        is2 = dot4((qb[k].z >> 4) & 0x0f0f0f0fu, a3.z, is2);
                        is2 = dot4((qb[k].w >> 4) & 0x0f0f0f0fu, a3.w, is2);
                        const int s1 = __mul24(sc1, is1) + __mul24(sc2, is2);
                        const int s2 = __mul24(m1, bs0) + __mul24(m2, bs1);
                        const float d = h2f(h[k].x & 0xffffu), dmin = h2f(h[k].x >> 16);
                        acc[k][b] += (d * da) * (float)s1 - (dmin * da) * (float)s2;
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < R; k++)
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const float v = part_sum<LPR>(acc[k][b]);
                if (l == 0 && r0 + k < rows && b < batch) y[(size_t)b * rows + r0 + k] = v;
            }
    }
}

template <int LPR, int NB, int R>
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
    for (long g0 = ((long)blockIdx.x * (THIN_THREADS / 64) + (threadIdx.x >> 6)) * PARTS; g0 * R < rows;
         g0 += n_waves * PARTS) {
        const long r0 = (g0 + part) * R;
        float acc[R][NB];
#pragma unroll
        for (int k = 0; k < R; k++)
#pragma unroll
            for (int b = 0; b < NB; b++) acc[k][b] = 0.0f;
        if (r0 < rows) {
            for (int u = l; u < units; u += LPR) {
                // unit = (block, half h, 16-lane column t), as in the decode GEMV
                const int blk_i = u >> 2, h = (u >> 1) & 1, t = u & 1;
                uint32_t w1[R][4], w2[R][4], w3[R][4], w4[R][4];  // four 16-weight groups, 6-bit codes (0..63)
                int s1[R], s2[R], s3[R], s4[R];
                float d[R];
#pragma unroll
                for (int k = 0; k < R; k++) {
                    const uint8_t *row = W + (size_t)min(r0 + k, (long)rows - 1) * lay.row_stride;
                    const uint4 qla = *reinterpret_cast<const uint4 *>(row + (size_t)blk_i * 128 + h * 64 + t * 16);
                    const uint4 qlb = *reinterpret_cast<const uint4 *>(row + (size_t)blk_i * 128 + h * 64 + 32 + t * 16);
                    const uint4 qh = *reinterpret_cast<const uint4 *>(row + lay.off_a + (size_t)blk_i * 64 + h * 32 + t * 16);
                    const uint2 scv = *reinterpret_cast<const uint2 *>(row + lay.off_b + (size_t)blk_i * 16 + h * 8);
                    d[k] = h2f(*reinterpret_cast<const uint16_t *>(row + lay.off_c + (size_t)blk_i * 2));
#define FRK_Q6_UNPACK(i, c)                                               \
    w1[k][i] = (qla.c & 0x0f0f0f0fu) | ((qh.c << 4) & 0x30303030u);        \
    w2[k][i] = (qlb.c & 0x0f0f0f0fu) | ((qh.c << 2) & 0x30303030u);        \
    w3[k][i] = ((qla.c >> 4) & 0x0f0f0f0fu) | (qh.c & 0x30303030u);        \
    w4[k][i] = ((qlb.c >> 4) & 0x0f0f0f0fu) | ((qh.c >> 2) & 0x30303030u);
                    FRK_Q6_UNPACK(0, x)
                    FRK_Q6_UNPACK(1, y)
                    FRK_Q6_UNPACK(2, z)
                    FRK_Q6_UNPACK(3, w)
#undef FRK_Q6_UNPACK
                    const uint32_t slo = t ? (scv.x >> 8) : scv.x, shi = t ? (scv.y >> 8) : scv.y;
                    s1[k] = (int)(int8_t)(slo & 0xff);
                    s2[k] = (int)(int8_t)((slo >> 16) & 0xff);
                    s3[k] = (int)(int8_t)(shi & 0xff);
                    s4[k] = (int)(int8_t)((shi >> 16) & 0xff);
                }
                const int g = h * 8 + t;
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    const uint4 *a = smem + (size_t)b * nb * 16 + u;  // pieces k at [k][unit]
                    const uint4 a0 = a[0], a1 = a[units], a2 = a[2 * units], a3 = a[3 * units];
                    // the -32 of the 6-bit code folded as -32 * (sum of the 16 activation quants)
                    const int *bs = sbs + ((size_t)b * nb + blk_i) * 16 + g;
                    const int o1 = 32 * bs[0], o2 = 32 * bs[2], o3 = 32 * bs[4], o4 = 32 * bs[6];
                    const float da = sd[(size_t)b * nb + blk_i];
#pragma unroll
                    for (int k = 0; k < R; k++) {
                        int d1 = 0, d2 = 0, d3 = 0, d4 = 0;
                        d1 = dot4(w1[k][0], a0.x, d1);
                        d1 = dot4(w1[k][1], a0.y, d1);
                        d1 = dot4(w1[k][2], a0.z, d1);
                        d1 = dot4(w1[k][3], a0.w, d1);
                        d2 = dot4(w2[k][0], a1.x, d2);
                        d2 = dot4(w2[k][1], a1.y, d2);
                        d2 = dot4(w2[k][2], a1.z, d2);
                        d2 = dot4(w2[k][3], a1.w, d2);
                        d3 = dot4(w3[k][0], a2.x, d3);
                        d3 = dot4(w3[k][1], a2.y, d3);
                        d3 = dot4(w3[k][2], a2.z, d3);
                        d3 = dot4(w3[k][3], a2.w, d3);
                        d4 = dot4(w4[k][0], a3.x, d4);
                        d4 = dot4(w4[k][1], a3.y, d4);
                        d4 = dot4(w4[k][2], a3.z, d4);
                        d4 = dot4(w4[k][3], a3.w, d4);
                        const int isum = s1[k] * (d1 - o1) + s2[k] * (d2 - o2) + s3[k] * (d3 - o3) + s4[k] * (d4 - o4);
                        acc[k][b] += (d[k] * da) * (float)isum;
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < R; k++)
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const float v = part_sum<LPR>(acc[k][b]);
                if (l == 0 && r0 + k < rows && b < batch) y[(size_t)b * rows + r0 + k] = v;
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

static unsigned thin_grid(size_t rows, int lpr, int r) {
    const size_t rows_per_wg = (THIN_THREADS / 64) * (size_t)(64 / lpr) * (size_t)r;
    size_t g = (rows + rows_per_wg - 1) / rows_per_wg;
    if (g > 256) g = 256;  // a workgroup per CU; wavefronts loop over rows, so the activations are staged once
    return (unsigned)(g < 1 ? 1 : g);
}

constexpr size_t THIN_LDS_LIMIT = 150 * 1024;

template <int LPR, int NB>
static int launch_thin_one(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    const bool q4 = w->kind == FRK_KIND_Q4_K;
    const size_t shmem = (size_t)NB * nb * (256 + (q4 ? 8 : 16) * 4 + 4);
    constexpr int R4 = 1, R6 = 1;  // more rows per lane spill at 128 registers and were measured slower  // weight rows per lane and unit
    const unsigned grid = thin_grid(w->rows, LPR, q4 ? R4 : R6);
    if (q4) {
        static bool sized = false;
        if (shmem > 65536 && !sized) {
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_q4_k_kernel<LPR, NB, R4>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)THIN_LDS_LIMIT));
            sized = true;
        }
        hipLaunchKernelGGL((thin_q4_k_kernel<LPR, NB, R4>), dim3(grid), dim3(THIN_THREADS), shmem, s, w->dev,
                           w->layout.row_stride, (int)w->rows, nb, batch, a.q, a.d, a.bsums, y);
    } else {
        static bool sized = false;
        if (shmem > 65536 && !sized) {
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_q6_k_kernel<LPR, NB, R6>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)THIN_LDS_LIMIT));
            sized = true;
        }
        hipLaunchKernelGGL((thin_q6_k_kernel<LPR, NB, R6>), dim3(grid), dim3(THIN_THREADS), shmem, s, w->dev, w->layout,
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
