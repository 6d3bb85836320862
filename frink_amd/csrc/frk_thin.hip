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
// Rows past `batch` repeat the last one (their results are not stored).  All of a thread's loads
// are issued before the first LDS write: a load, its wait and its write in turn, once per row,
// made the staging cost as much as the arithmetic.
template <int NB, int SUMS_PER_BLOCK>
__device__ __forceinline__ void stage_acts(uint4 *smem, int nb, int batch, const int8_t *aq, const float *ad,
                                           const int16_t *absums, int8_t *&sq, int *&sbs, float *&sd) {
    sq = reinterpret_cast<int8_t *>(smem);
    sbs = reinterpret_cast<int *>(sq + (size_t)NB * nb * 256);
    sd = reinterpret_cast<float *>(sbs + (size_t)NB * nb * SUMS_PER_BLOCK);
    constexpr int FOLD = 16 / SUMS_PER_BLOCK;  // bsums folded per stored sum
    constexpr int CHUNK = 4;
    const int tid = threadIdx.x;
    const int row_g = nb * 16, row_s = nb * SUMS_PER_BLOCK;
    for (int base = 0; base < NB * row_g; base += CHUNK * THIN_THREADS) {
        uint4 v[CHUNK];
#pragma unroll
        for (int j = 0; j < CHUNK; j++) {  // (past the end: a valid address, the value is not written)
            const int idx = min(base + j * THIN_THREADS + tid, NB * row_g - 1);
            const int b = idx / row_g, i = idx - b * row_g;
            v[j] = reinterpret_cast<const uint4 *>(aq + (size_t)min(b, batch - 1) * nb * 256)[i];
        }
#pragma unroll
        for (int j = 0; j < CHUNK; j++) {
            const int idx = base + j * THIN_THREADS + tid;
            if (idx < NB * row_g) {
                const int b = idx / row_g, i = idx - b * row_g;
                smem[(size_t)b * row_g + granule_slot<SUMS_PER_BLOCK == 16>(i, nb * 4)] = v[j];
            }
        }
    }
    for (int base = 0; base < NB * row_s; base += CHUNK * THIN_THREADS) {
        int v[CHUNK];
#pragma unroll
        for (int j = 0; j < CHUNK; j++) {
            const int idx = base + j * THIN_THREADS + tid;
            v[j] = 0;
            {
                const int idc = min(idx, NB * row_s - 1);
                const int b = idc / row_s, i = idc - b * row_s;
                const int16_t *bs = absums + (size_t)min(b, batch - 1) * nb * 16;
#pragma unroll
                for (int f = 0; f < FOLD; f++) v[j] += (int)bs[FOLD * i + f];
            }
        }
#pragma unroll
        for (int j = 0; j < CHUNK; j++) {
            const int idx = base + j * THIN_THREADS + tid;
            if (idx < NB * row_s) sbs[idx] = v[j];
        }
    }
    for (int idx = tid; idx < NB * nb; idx += THIN_THREADS) {
        const int b = idx / nb, i = idx - b * nb;
        sd[idx] = ad[(size_t)min(b, batch - 1) * nb + i];
    }
    __syncthreads();
}

// Both kernels: LPR lanes share a weight row (a wavefront works on 64/LPR rows at once) and walk it
// in units of 64 weights; a lane unpacks its unit once and multiplies it against the same slice of
// each activation row.  A wavefront's (row, unit) steps form one sequence, and the weights of step
// i+1 are requested before step i is computed: with one workgroup per CU there is nothing else to
// hide the load latency behind.

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
    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 4, upl = (units + LPR - 1) / LPR;  // steps per row
    const int wave_id = blockIdx.x * (THIN_THREADS / 64) + (threadIdx.x >> 6), n_waves = gridDim.x * (THIN_THREADS / 64);
    const int n_groups = (rows + PARTS - 1) / PARTS;
    const int my_groups = wave_id < n_groups ? (n_groups - wave_id + n_waves - 1) / n_waves : 0;

    struct Unit {
        uint4 h, qa, qb;
    };
    // the unit of step (group gi, pass ui); past the end of a row or of the matrix it repeats a
    // valid one, whose product is not used
    auto load_unit = [&](int gi, int ui, Unit &U) {
        const int row = min((wave_id + gi * n_waves) * PARTS + part, rows - 1);
        const int u = min(l + ui * LPR, units - 1);
        const uint4 *blk = reinterpret_cast<const uint4 *>(W + (size_t)row * row_stride + (size_t)(u >> 2) * Q4_K_BYTES);
        U.h = blk[0];
        U.qa = blk[1 + 2 * (u & 3)];
        U.qb = blk[2 + 2 * (u & 3)];
    };
    Unit cur;
    if (my_groups > 0) load_unit(0, 0, cur);  // in flight while the activations are staged
    stage_acts<NB, 8>(smem, nb, batch, aq, ad, absums, sq, sbs, sd);

    float acc[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) acc[b] = 0.0f;
    int gi = 0, ui = 0;
    for (int it = 0; it < my_groups * upl; it++) {
        int gn = gi, un = ui + 1;
        if (un == upl) {
            un = 0;
            gn++;
        }
        Unit nxt = cur;
        if (gn < my_groups) load_unit(gn, un, nxt);

        const int u = l + ui * LPR;
        const int row = (wave_id + gi * n_waves) * PARTS + part;
        if (u < units && row < rows) {
            const int blk_i = u >> 2, p = u & 3;
            // 6-bit scales and mins of sub-blocks 2p and 2p+1 (q4_k_scale_min, lib.rs:321-330)
            uint32_t scw, mw;
            if (p < 2) {
                scw = cur.h.y & 0x3f3f3f3fu;
                mw = cur.h.z & 0x3f3f3f3fu;
            } else {
                scw = (cur.h.w & 0x0f0f0f0fu) | (((cur.h.y >> 6) & 0x03030303u) << 4);
                mw = ((cur.h.w >> 4) & 0x0f0f0f0fu) | (((cur.h.z >> 6) & 0x03030303u) << 4);
            }
            const int sh = (p & 1) * 16;
            const int sc1 = (scw >> sh) & 0xff, sc2 = (scw >> (sh + 8)) & 0xff;
            const int m1 = (mw >> sh) & 0xff, m2 = (mw >> (sh + 8)) & 0xff;
            const float d = h2f(cur.h.x & 0xffffu), dmin = h2f(cur.h.x >> 16);
            const uint32_t la[4] = {cur.qa.x & 0x0f0f0f0fu, cur.qa.y & 0x0f0f0f0fu, cur.qa.z & 0x0f0f0f0fu, cur.qa.w & 0x0f0f0f0fu};
            const uint32_t lb[4] = {cur.qb.x & 0x0f0f0f0fu, cur.qb.y & 0x0f0f0f0fu, cur.qb.z & 0x0f0f0f0fu, cur.qb.w & 0x0f0f0f0fu};
            const uint32_t ha[4] = {(cur.qa.x >> 4) & 0x0f0f0f0fu, (cur.qa.y >> 4) & 0x0f0f0f0fu, (cur.qa.z >> 4) & 0x0f0f0f0fu,
                                    (cur.qa.w >> 4) & 0x0f0f0f0fu};
            const uint32_t hb[4] = {(cur.qb.x >> 4) & 0x0f0f0f0fu, (cur.qb.y >> 4) & 0x0f0f0f0fu, (cur.qb.z >> 4) & 0x0f0f0f0fu,
                                    (cur.qb.w >> 4) & 0x0f0f0f0fu};
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const uint4 *a = smem + (size_t)b * nb * 16 + u;  // pieces k at [k][unit]
                const uint4 a0 = a[0], a1 = a[units], a2 = a[2 * units], a3 = a[3 * units];
                const int *bs = sbs + ((size_t)b * nb + blk_i) * 8 + 2 * p;
                const int bs0 = bs[0], bs1 = bs[1];
                const float da = sd[(size_t)b * nb + blk_i];
                int is1 = 0, is2 = 0;
                is1 = dot4(la[0], a0.x, is1);
                is1 = dot4(la[1], a0.y, is1);
                is1 = dot4(la[2], a0.z, is1);
                is1 = dot4(la[3], a0.w, is1);
                is1 = dot4(lb[0], a1.x, is1);
                is1 = dot4(lb[1], a1.y, is1);
                is1 = dot4(lb[2], a1.z, is1);
                is1 = dot4(lb[3], a1.w, is1);
                is2 = dot4(ha[0], a2.x, is2);
                is2 = dot4(ha[1], a2.y, is2);
                is2 = dot4(ha[2], a2.z, is2);
                is2 = dot4(ha[3], a2.w, is2);
                is2 = dot4(hb[0], a3.x, is2);
                is2 = dot4(hb[1], a3.y, is2);
                is2 = dot4(hb[2], a3.z, is2);
                is2 = dot4(hb[3], a3.w, is2);
                const int s1 = __mul24(sc1, is1) + __mul24(sc2, is2);
                const int s2 = __mul24(m1, bs0) + __mul24(m2, bs1);
                acc[b] += (d * da) * (float)s1 - (dmin * da) * (float)s2;
            }
        }
        if (ui == upl - 1) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const float v = part_sum<LPR>(acc[b]);
                if (l == 0 && row < rows && b < batch) y[(size_t)b * rows + row] = v;
                acc[b] = 0.0f;
            }
        }
        cur = nxt;
        gi = gn;
        ui = un;
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

// ------------------------------------------------------------------ thin GEMM on the matrix cores (Q4_K)
//
// Up to 16 activation rows against 16 weight rows per wavefront with v_mfma_i32_16x16x32_i8: one
// MFMA is the integer dot of one 32-weight sub-block for all 16 x 16 (activation, weight row) pairs,
// so the eight sub-block dots of a block cost eight short MFMAs instead of 16 dot4 per activation,
// and the 6-bit scale multiplies each MFMA's four results (one v_mul_i32_i24 each: the weight row,
// hence the scale, is the lane's own).  Integers are exactly dot_q4_k_q8's
// (crates/frink-quant/src/lib.rs:822-869); the min term sum_j m_j * bsum_j is one f16 MFMA (both
// factors and all sums exact); per block the float step is the batched GEMM's
// acc += da * (d * S1 - dmin * S2).
// Operand layout (checked on the device): lane l holds row/column l % 16 and the eight k
// 8*(l/16) .. +7 (four for the K=16 f16 form); result register r is D[4*(l/16) + r][l % 16].  A =
// activations, B = weights: a lane's four results are four activation rows of its own weight row.
//
// Data movement.  An MFMA lane wants 8 bytes of ITS row, so loading operands straight from memory
// touches 16 rows per instruction, and the address unit then costs more than the data (measured:
// 20 us, with or without the weights streaming).  Instead:
//   * the quantized activations (acts x cols bytes, plus sums as f16 and scales) are staged in LDS
//     once per workgroup with contiguous loads;
//   * each wavefront streams the raw blocks of its 16 rows (16 x 144 bytes, contiguous per row) with
//     ordinary 16-byte loads, TM_AHEAD blocks ahead in registers, and turns a block into the per-row
//     view through a 2.25 KB LDS area of its own: a wavefront reads only what it wrote, in order,
//     so after the staging there is no barrier in the loop.  (global_load_lds would save the
//     registers, but it moved a KB per 60 to 100 clocks and CU here, a quarter of what the
//     ordinary loads do.)
// A workgroup is 8 wavefronts = RG groups of 16 rows x KS splits of the blocks (block kb goes to split
// kb % KS); the splits add up through LDS in order at the end.
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef _Float16 v4h_t __attribute__((ext_vector_type(4)));

constexpr int TM_WAVES = 8;
constexpr int TM_AHEAD = 4;                    // blocks of a wavefront in flight
// one block of 16 rows: 2304 bytes of Q4_K, 2816 of Q5_K
__host__ __device__ constexpr int tm_wblock(bool q5) { return 16 * (q5 ? Q5_K_BYTES : Q4_K_BYTES); }
// LDS rows of the activations are padded so that the 16 rows a read touches fall in different banks
__host__ __device__ constexpr int tm_q_stride(int cols) { return cols + 16; }
__host__ __device__ constexpr int tm_bs_stride(int cols) { return cols / 8 + 8; }  // f16 sums, bytes
__host__ __device__ inline size_t tm_lds_bytes(int acts, int cols, bool q5) {
    return (size_t)acts * (tm_q_stride(cols) + tm_bs_stride(cols)) + (size_t)(cols / QK_K) * 64 +
           (size_t)TM_WAVES * tm_wblock(q5);
}

// (at most 4 wavefronts per SIMD: without the bound the compiler aims for 7, with 72 registers,
// and keeps the ring in scratch memory)
// Q5: the weights are Q5_K -- the same super-block with 32 bytes of fifth bits between the header and
// the nibbles (11 sixteen-byte pieces a row instead of 9); byte l of them serves weight l of every
// sub-block, sub-block j through bit j (dot_q5_k_q8, crates/frink-quant/src/lib.rs:886-938).
template <int RG, int ACTS, bool Q5>
__global__ __launch_bounds__(64 * TM_WAVES) __attribute__((amdgpu_waves_per_eu(2, 4))) void thin_mfma_q4_k_kernel(const uint8_t *__restrict__ W, size_t row_stride,
                                                                        int rows, int nb, int batch,
                                                                        const int8_t *__restrict__ aq,
                                                                        const float *__restrict__ ad,
                                                                        const int16_t *__restrict__ absums,
                                                                        float *__restrict__ y) {
    constexpr int KS = TM_WAVES / RG;
    // a batch wider than ACTS is a grid of groups of ACTS activation rows: blockIdx.y picks the group
    // (every group streams the weights again, out of L2 after the first)
    aq += (size_t)blockIdx.y * ACTS * nb * QK_K;
    ad += (size_t)blockIdx.y * ACTS * nb;
    absums += (size_t)blockIdx.y * ACTS * nb * 16;
    y += (size_t)blockIdx.y * ACTS * rows;
    batch = min(ACTS, batch - (int)blockIdx.y * ACTS);
    constexpr int BB = Q5 ? Q5_K_BYTES : Q4_K_BYTES;  // bytes of a block
    constexpr int PR = BB / 16, NP = 16 * PR;         // 16-byte pieces of a row's block, of 16 rows' blocks
    constexpr int QS = Q5 ? 48 : 16;                  // where the nibbles start
    constexpr int WBLOCK = tm_wblock(Q5);
    extern __shared__ uint4 smem[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
    const int cols = nb * QK_K;
    const int q_stride = tm_q_stride(cols), bs_stride = tm_bs_stride(cols);
    uint8_t *lds_q = lds;                                     // [ACTS][q_stride]
    uint8_t *lds_bs = lds_q + (size_t)ACTS * q_stride;        // [ACTS][bs_stride] f16
    float *lds_d = reinterpret_cast<float *>(lds_bs + (size_t)ACTS * bs_stride);  // [nb][16]
    uint8_t *lds_w = reinterpret_cast<uint8_t *>(lds_d + (size_t)nb * 16);        // [wave][WBLOCK]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int rgrp = wave % RG, ksp = wave / RG;
    const int row0 = (blockIdx.x * RG + rgrp) * 16;
    const int my_blocks = nb > ksp ? (nb - ksp + KS - 1) / KS : 0;

    // ---- this wavefront's weight stream: piece p = 64*c + lane of chunk c is row p/PR, piece p%PR ----
    const uint8_t *w_src[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        const int p = min(64 * c + lane, NP - 1);
        w_src[c] = W + (size_t)min(row0 + p / PR, rows - 1) * row_stride + (p % PR) * 16 + (size_t)ksp * BB;
    }
    struct Raw {
        uint4 a, b, c;
    };
    auto fetch_block = [&](int i) {  // (past the last block: the last one again, never used)
        const size_t off = (size_t)KS * max(min(i, my_blocks - 1), 0) * BB;
        Raw R;
        R.a = *reinterpret_cast<const uint4 *>(w_src[0] + off);
        R.b = *reinterpret_cast<const uint4 *>(w_src[1] + off);
        R.c = *reinterpret_cast<const uint4 *>(w_src[2] + off);  // lanes NP-128.. repeat the last piece
        return R;
    };
    static_assert(TM_AHEAD == 4, "the ring is four named buffers");
    // (named values handed around by value: an array, or structs passed by reference, end up in memory)
    Raw R0, R1, R2, R3;

    // ---- the activations, once per workgroup ----
    // A wavefront's loads complete in order.  The staging loads (four per thread and array in a
    // round; one round is the whole of it at the usual sizes) therefore go out first and the
    // weight ring right behind them: the staging is over after one trip to the L2, and the first
    // blocks are multiplied while the rest of the matrix is still streaming in.
    {
        constexpr int T = 64 * TM_WAVES;
        const int row_g = cols / 16;   // 16-byte granules of quants per row
        const int row_s4 = cols / 64;  // sums per row, four at a time
        auto load_q = [&](int base, int u) {  // (past the end: a valid address, the value is not written)
            const int idx = min(base + u * T + tid, ACTS * row_g - 1);
            const int a = idx / row_g, i = idx - a * row_g;
            return reinterpret_cast<const uint4 *>(aq + (size_t)min(a, batch - 1) * cols)[i];
        };
        auto store_q = [&](int base, int u, uint4 v) {
            const int idx = base + u * T + tid;
            if (idx < ACTS * row_g) {
                const int a = idx / row_g, i = idx - a * row_g;
                *reinterpret_cast<uint4 *>(lds_q + (size_t)a * q_stride + i * 16) = v;
            }
        };
        auto load_s = [&](int base, int u) {
            const int idx = min(base + u * T + tid, ACTS * row_s4 - 1);
            const int a = idx / row_s4, i = idx - a * row_s4;
            return reinterpret_cast<const uint2 *>(absums + (size_t)min(a, batch - 1) * row_s4 * 4)[i];
        };
        auto store_s = [&](int base, int u, uint2 v) {
            const int idx = base + u * T + tid;
            if (idx < ACTS * row_s4) {
                const int a = idx / row_s4, i = idx - a * row_s4;
                const v4h_t h = {(_Float16)(int)(int16_t)(v.x & 0xffff), (_Float16)(int)(int16_t)(v.x >> 16),
                                 (_Float16)(int)(int16_t)(v.y & 0xffff), (_Float16)(int)(int16_t)(v.y >> 16)};
                *reinterpret_cast<v4h_t *>(lds_bs + (size_t)a * bs_stride + i * 8) = h;
            }
        };
        auto load_d = [&](int idx) {
            idx = min(idx, nb * 16 - 1);
            return ad[(size_t)min(idx & 15, batch - 1) * nb + (idx >> 4)];
        };
        const uint4 q0 = load_q(0, 0), q1 = load_q(0, 1), q2 = load_q(0, 2), q3 = load_q(0, 3);
        const uint2 s0 = load_s(0, 0), s1 = load_s(0, 1), s2 = load_s(0, 2), s3 = load_s(0, 3);
        const float d0 = load_d(tid);
        R0 = fetch_block(0);
        R1 = fetch_block(1);
        R2 = fetch_block(2);
        R3 = fetch_block(3);
        store_q(0, 0, q0);
        store_q(0, 1, q1);
        store_q(0, 2, q2);
        store_q(0, 3, q3);
        store_s(0, 0, s0);
        store_s(0, 1, s1);
        store_s(0, 2, s2);
        store_s(0, 3, s3);
        if (tid < nb * 16) lds_d[tid] = d0;
        // what one round does not cover (long rows): behind the ring, at the ring's pace
        for (int base = 4 * T; base < ACTS * row_g; base += 4 * T)
#pragma unroll
            for (int u = 0; u < 4; u++) store_q(base, u, load_q(base, u));
        for (int base = 4 * T; base < ACTS * row_s4; base += 4 * T)
#pragma unroll
            for (int u = 0; u < 4; u++) store_s(base, u, load_s(base, u));
        for (int idx = T + tid; idx < nb * 16; idx += T) lds_d[idx] = load_d(idx);
    }
    __syncthreads();

    // ---- the loop: no barrier; a wavefront writes its block to its own area and reads it back by row ----
    const int act = min(j, ACTS - 1);  // rows past the staged ones repeat the last; their results are not stored
    const uint8_t *a_q = lds_q + (size_t)act * q_stride + 8 * g;
    const uint8_t *a_bs = lds_bs + (size_t)act * bs_stride + 8 * g;
    const float *a_d = lds_d + 4 * g;
    uint8_t *area = lds_w + (size_t)wave * WBLOCK;
    const uint8_t *a_w = area + j * BB;
    auto as_long = [](uint2 v) { return (long)(((unsigned long)v.y << 32) | v.x); };
    v4f_t acc = {0.f, 0.f, 0.f, 0.f};
    auto multiply_block = [&](int i, Raw R) {  // returns the block that takes this one's place in the ring
        const int kb = ksp + KS * i;
        reinterpret_cast<uint4 *>(area)[lane] = R.a;
        reinterpret_cast<uint4 *>(area)[64 + lane] = R.b;
        if (lane < NP - 128) reinterpret_cast<uint4 *>(area)[128 + lane] = R.c;
        R = fetch_block(i + TM_AHEAD);  // the registers are free again
        const uint4 h = *reinterpret_cast<const uint4 *>(a_w);
        // 6-bit scales and mins (q4_k_scale_min, lib.rs:321-330): bytes of sc_lo/m_lo are sub-blocks
        // 0..3, of sc_hi/m_hi sub-blocks 4..7
        const uint32_t sc_lo = h.y & 0x3f3f3f3fu, m_lo = h.z & 0x3f3f3f3fu;
        const uint32_t sc_hi = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);
        const uint32_t m_hi = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
        v4i_t s1 = {0, 0, 0, 0};
        const v4i_t zero = {0, 0, 0, 0};
        const uint8_t *aq_k = a_q + (size_t)kb * QK_K;
        // Q5_K: the fifth bits of this lane's eight weights, of every sub-block
        const uint2 f = Q5 ? *reinterpret_cast<const uint2 *>(a_w + 16 + 8 * g) : make_uint2(0u, 0u);
#pragma unroll
        for (int c = 0; c < 4; c++) {  // sub-blocks 2c (low nibbles) and 2c+1 (high)
            const uint2 q = *reinterpret_cast<const uint2 *>(a_w + QS + 32 * c + 8 * g);
            const uint2 alo = *reinterpret_cast<const uint2 *>(aq_k + 64 * c);
            const uint2 ahi = *reinterpret_cast<const uint2 *>(aq_k + 64 * c + 32);
            const uint32_t scw = (c < 2 ? sc_lo : sc_hi) >> (16 * (c & 1));
            const int sc0 = scw & 0xff, sc1 = (scw >> 8) & 0xff;
            uint2 lo = make_uint2(q.x & 0x0f0f0f0fu, q.y & 0x0f0f0f0fu);
            uint2 hi = make_uint2((q.x >> 4) & 0x0f0f0f0fu, (q.y >> 4) & 0x0f0f0f0fu);
            if (Q5) {
                lo.x |= ((f.x >> (2 * c)) & 0x01010101u) << 4, lo.y |= ((f.y >> (2 * c)) & 0x01010101u) << 4;
                hi.x |= ((f.x >> (2 * c + 1)) & 0x01010101u) << 4, hi.y |= ((f.y >> (2 * c + 1)) & 0x01010101u) << 4;
            }
            const v4i_t t0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(alo), as_long(lo), zero, 0, 0, 0);
            const v4i_t t1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(ahi), as_long(hi), zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; r++) s1[r] += __mul24(sc0, t0[r]) + __mul24(sc1, t1[r]);
        }
        // mins of the 16-wide groups 4g..4g+3, i.e. of sub-blocks 2g and 2g+1, against the sums
        const uint32_t mw = (g < 2 ? m_lo : m_hi) >> (16 * (g & 1));
        const _Float16 m0 = (_Float16)(int)(mw & 0xff), m1 = (_Float16)(int)((mw >> 8) & 0xff);
        const v4h_t mh = {m0, m0, m1, m1};
        const v4h_t bh = *reinterpret_cast<const v4h_t *>(a_bs + (size_t)kb * 32);
        const v4f_t da = *reinterpret_cast<const v4f_t *>(a_d + (size_t)kb * 16);
        const v4f_t zf = {0.f, 0.f, 0.f, 0.f};
        const v4f_t s2 = __builtin_amdgcn_mfma_f32_16x16x16f16(bh, mh, zf, 0, 0, 0);
        const float d = h2f(h.x & 0xffffu), ndmin = -h2f(h.x >> 16);
#pragma unroll
        for (int r = 0; r < 4; r++) acc[r] = fmaf(da[r], fmaf(ndmin, s2[r], d * (float)s1[r]), acc[r]);
        return R;
    };
    // the ring's buffers take turns by position, so no buffer is ever copied into another (a copy
    // would wait for the loads in flight)
    for (int i = 0; i < my_blocks; i += TM_AHEAD) {
        R0 = multiply_block(i, R0);
        if (i + 1 < my_blocks) R1 = multiply_block(i + 1, R1);
        if (i + 2 < my_blocks) R2 = multiply_block(i + 2, R2);
        if (i + 3 < my_blocks) R3 = multiply_block(i + 3, R3);
    }

    if (KS > 1) {  // add the splits up in order, through the (now idle) activation area
        __syncthreads();
        float *red = reinterpret_cast<float *>(lds);
        if (ksp > 0) {
#pragma unroll
            for (int r = 0; r < 4; r++) red[(((ksp - 1) * RG + rgrp) * 4 + r) * 64 + lane] = acc[r];
        }
        __syncthreads();
        if (ksp > 0) return;
#pragma unroll
        for (int k = 0; k < KS - 1; k++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += red[((k * RG + rgrp) * 4 + r) * 64 + lane];
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int b = 4 * g + r;
        if (b < batch && row0 + j < rows) y[(size_t)b * rows + row0 + j] = acc[r];
    }
}

// ------------------------------------------------------------------ thin GEMM on the matrix cores (Q6_K)
//
// Same plan as the Q4_K kernel above, for up to 8 activation rows.  Q6_K scales sixteen weights at
// a time, and a K=32 MFMA would add up two such groups.  So the 16 rows of the MFMA's activation
// operand hold the (at most 8) activation rows twice: rows 0..7 with only the first sixteen k of
// every 32 (the rest zero), rows 8..15 with only the second sixteen.  One MFMA then returns, for
// each (activation, weight row), the two 16-wide dots side by side -- in the lanes of k-groups 0..1
// and 2..3, which multiply them by their own group's int8 scale; the two halves of a result meet
// once, at the end.  The 6-bit codes go in as signed bytes q - 32 (one add and one xor per four
// codes), so there is no "-32 * sum of the activations" term to carry: the integers are
// dot_q6_k_q8's (crates/frink-quant/src/lib.rs:1069-1110), split in two partial sums per block.
// Weights are the resident planar form (ql | qh | sc | d per row); in LDS a row of a block is
// [ql 128 | qh 64 | sc 16 | d 2], 240 bytes apart so that the 16 rows of a read fall in
// different banks.
constexpr int T6_ROW = 240;
constexpr int T6_WBLOCK = 16 * T6_ROW;  // 3840
__host__ __device__ inline size_t t6_lds_bytes(int acts, int cols) {
    return (size_t)acts * tm_q_stride(cols) + (size_t)(cols / QK_K) * 32 + (size_t)TM_WAVES * T6_WBLOCK;
}

template <int RG, int ACTS>
__global__ __launch_bounds__(64 * TM_WAVES) __attribute__((amdgpu_waves_per_eu(2, 4))) void thin_mfma_q6_k_kernel(
    const uint8_t *__restrict__ W, Layout lay, int rows, int nb, int batch, const int8_t *__restrict__ aq,
    const float *__restrict__ ad, float *__restrict__ y) {
    constexpr int KS = TM_WAVES / RG;
    extern __shared__ uint4 smem[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
    const int cols = nb * QK_K;
    // a batch wider than ACTS is a grid of groups of ACTS activation rows: blockIdx.y picks the group
    // (every group streams the matrix again; the groups after the first find it in the caches)
    aq += (size_t)blockIdx.y * ACTS * cols;
    ad += (size_t)blockIdx.y * ACTS * nb;
    y += (size_t)blockIdx.y * ACTS * rows;
    batch = min(ACTS, batch - (int)blockIdx.y * ACTS);
    const int q_stride = tm_q_stride(cols);
    uint8_t *lds_q = lds;                                                         // [ACTS][q_stride]
    float *lds_d = reinterpret_cast<float *>(lds_q + (size_t)ACTS * q_stride);    // [nb][8]
    uint8_t *lds_w = reinterpret_cast<uint8_t *>(lds_d + (size_t)nb * 8);         // [wave][3840]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int rgrp = wave % RG, ksp = wave / RG;
    const int row0 = (blockIdx.x * RG + rgrp) * 16;
    const int my_blocks = nb > ksp ? (nb - ksp + KS - 1) / KS : 0;

    // ---- this wavefront's weight stream: the four planes of its 16 rows, 16-byte pieces ----
    // ql: piece p = 64*c + lane (c = 0, 1) is row p/8, piece p%8; qh: piece lane is row lane/4, piece
    // lane%4; sc: lanes 0..15, one piece per row; d: lanes 0..15, two bytes per row
    auto row_ptr = [&](int r) { return W + (size_t)min(row0 + r, rows - 1) * lay.row_stride; };
    const uint8_t *src_ql0 = row_ptr(lane >> 3) + (lane & 7) * 16 + (size_t)ksp * 128;
    const uint8_t *src_ql1 = row_ptr(8 + (lane >> 3)) + (lane & 7) * 16 + (size_t)ksp * 128;
    const uint8_t *src_qh = row_ptr(lane >> 2) + lay.off_a + (lane & 3) * 16 + (size_t)ksp * 64;
    const uint8_t *src_sc = row_ptr(lane & 15) + lay.off_b + (size_t)ksp * 16;
    const uint8_t *src_d = row_ptr(lane & 15) + lay.off_c + (size_t)ksp * 2;
    struct Raw {
        uint4 ql0, ql1, qh, sc;
        uint32_t d;
    };
    auto fetch_block = [&](int i) {  // (past the last block: the last one again, never used)
        const size_t k = (size_t)KS * max(min(i, my_blocks - 1), 0);
        Raw R;
        R.ql0 = *reinterpret_cast<const uint4 *>(src_ql0 + k * 128);
        R.ql1 = *reinterpret_cast<const uint4 *>(src_ql1 + k * 128);
        R.qh = *reinterpret_cast<const uint4 *>(src_qh + k * 64);
        R.sc = *reinterpret_cast<const uint4 *>(src_sc + k * 16);  // lanes 16.. repeat rows 0..15
        R.d = *reinterpret_cast<const uint16_t *>(src_d + k * 2);
        return R;
    };
    static_assert(TM_AHEAD == 4, "the ring is four named buffers");
    Raw R0, R1, R2, R3;

    // ---- the activations, once per workgroup: staging loads first, the weight ring behind them ----
    {
        constexpr int T = 64 * TM_WAVES;
        const int row_g = cols / 16;  // 16-byte granules of quants per row
        auto load_q = [&](int base, int u) {  // (past the end: a valid address, the value is not written)
            const int idx = min(base + u * T + tid, ACTS * row_g - 1);
            const int a = idx / row_g, i = idx - a * row_g;
            return reinterpret_cast<const uint4 *>(aq + (size_t)min(a, batch - 1) * cols)[i];
        };
        auto store_q = [&](int base, int u, uint4 v) {
            const int idx = base + u * T + tid;
            if (idx < ACTS * row_g) {
                const int a = idx / row_g, i = idx - a * row_g;
                *reinterpret_cast<uint4 *>(lds_q + (size_t)a * q_stride + i * 16) = v;
            }
        };
        auto load_d = [&](int idx) {
            idx = min(idx, nb * 8 - 1);
            return ad[(size_t)min(idx & 7, batch - 1) * nb + (idx >> 3)];
        };
        const uint4 q0 = load_q(0, 0), q1 = load_q(0, 1), q2 = load_q(0, 2), q3 = load_q(0, 3);
        const float d0 = load_d(tid);
        R0 = fetch_block(0);
        R1 = fetch_block(1);
        R2 = fetch_block(2);
        R3 = fetch_block(3);
        store_q(0, 0, q0);
        store_q(0, 1, q1);
        store_q(0, 2, q2);
        store_q(0, 3, q3);
        if (tid < nb * 8) lds_d[tid] = d0;
        // what one round does not cover (long rows): behind the ring, at the ring's pace
        for (int base = 4 * T; base < ACTS * row_g; base += 4 * T)
#pragma unroll
            for (int u = 0; u < 4; u++) store_q(base, u, load_q(base, u));
        for (int idx = T + tid; idx < nb * 8; idx += T) lds_d[idx] = load_d(idx);
    }
    __syncthreads();

    // ---- the loop ----
    // activation operand row j: activation j % 8, and only the k-groups of its half are real
    const bool real = (j < 8) == (g < 2);
    const uint8_t *a_q = lds_q + (size_t)min(j & 7, ACTS - 1) * q_stride + 8 * g;
    const float *a_d = lds_d + 4 * (g & 1);
    uint8_t *area = lds_w + (size_t)wave * T6_WBLOCK;
    const uint8_t *a_w = area + j * T6_ROW;
    auto as_long = [](uint2 v) { return (long)(((unsigned long)v.y << 32) | v.x); };
    v4f_t acc = {0.f, 0.f, 0.f, 0.f};
    auto multiply_block = [&](int i, Raw R) {  // returns the block that takes this one's place in the ring
        const int kb = ksp + KS * i;
        *reinterpret_cast<uint4 *>(area + (lane >> 3) * T6_ROW + (lane & 7) * 16) = R.ql0;
        *reinterpret_cast<uint4 *>(area + (8 + (lane >> 3)) * T6_ROW + (lane & 7) * 16) = R.ql1;
        *reinterpret_cast<uint4 *>(area + (lane >> 2) * T6_ROW + 128 + (lane & 3) * 16) = R.qh;
        if (lane < 16) {
            *reinterpret_cast<uint4 *>(area + lane * T6_ROW + 192) = R.sc;
            *reinterpret_cast<uint32_t *>(area + lane * T6_ROW + 208) = R.d;
        }
        R = fetch_block(i + TM_AHEAD);  // the registers are free again
        const uint4 scv = *reinterpret_cast<const uint4 *>(a_w + 192);
        const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
        const float d = h2f(*reinterpret_cast<const uint32_t *>(a_w + 208) & 0xffffu);
        const v4i_t zero = {0, 0, 0, 0};
        v4i_t isum = {0, 0, 0, 0};
        const uint8_t *aq_k = a_q + (size_t)kb * QK_K;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint2 qla = *reinterpret_cast<const uint2 *>(a_w + h * 64 + 8 * g);
            const uint2 qlb = *reinterpret_cast<const uint2 *>(a_w + h * 64 + 32 + 8 * g);
            const uint2 qh = *reinterpret_cast<const uint2 *>(a_w + 128 + h * 32 + 8 * g);
#pragma unroll
            for (int v = 0; v < 4; v++) {  // weights h*128 + 32*v + l, l = 8g .. 8g+7
                const uint2 ql = (v & 1) ? qlb : qla;
                auto code = [&](uint32_t lo, uint32_t hi) {  // four 6-bit codes, as signed bytes q - 32
                    const uint32_t nib = (v >= 2 ? lo >> 4 : lo) & 0x0f0f0f0fu;
                    const uint32_t top = ((hi >> (2 * v)) & 0x03030303u) << 4;
                    return ((nib | top) + 0x60606060u) ^ 0x80808080u;
                };
                const uint2 wq = make_uint2(code(ql.x, qh.x), code(ql.y, qh.y));
                uint2 a = *reinterpret_cast<const uint2 *>(aq_k + h * 128 + 32 * v);
                if (!real) a = make_uint2(0u, 0u);
                const v4i_t t = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(a), as_long(wq), zero, 0, 0, 0);
                // the scale of this lane's 16-wide group: sc[h*8 + 2*v + g/2]
                const int si = h * 8 + 2 * v + (g >> 1);
                const int sc = (int)(int8_t)((scw[si >> 2] >> (8 * (si & 3))) & 0xff);
#pragma unroll
                for (int r = 0; r < 4; r++) isum[r] += __mul24(sc, t[r]);
            }
        }
        const v4f_t da = *reinterpret_cast<const v4f_t *>(a_d + (size_t)kb * 8);
#pragma unroll
        for (int r = 0; r < 4; r++) acc[r] += (d * da[r]) * (float)isum[r];
        return R;
    };
    for (int i = 0; i < my_blocks; i += TM_AHEAD) {
        R0 = multiply_block(i, R0);
        if (i + 1 < my_blocks) R1 = multiply_block(i + 1, R1);
        if (i + 2 < my_blocks) R2 = multiply_block(i + 2, R2);
        if (i + 3 < my_blocks) R3 = multiply_block(i + 3, R3);
    }
    // the two 16-wide halves of every result sit 32 lanes apart
#pragma unroll
    for (int r = 0; r < 4; r++) acc[r] += __shfl_xor(acc[r], 32);

    if (KS > 1) {  // add the splits up in order, through the (now idle) activation area
        __syncthreads();
        float *red = reinterpret_cast<float *>(lds);
        if (ksp > 0) {
#pragma unroll
            for (int r = 0; r < 4; r++) red[(((ksp - 1) * RG + rgrp) * 4 + r) * 64 + lane] = acc[r];
        }
        __syncthreads();
        if (ksp > 0) return;
#pragma unroll
        for (int k = 0; k < KS - 1; k++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += red[((k * RG + rgrp) * 4 + r) * 64 + lane];
    }
    if (g < 2) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int b = 4 * g + r;
            if (b < batch && row0 + j < rows) y[(size_t)b * rows + row0 + j] = acc[r];
        }
    }
}

// ------------------------------------------------------------------ thin GEMM over whole spans (Q4_K)
//
// The kernel above walks a row group's blocks one after the other, four in flight: at 14336x4096 a
// wavefront's sixteen blocks are a chain of sixteen round trips, and its 144-byte pieces of sixteen
// rows cost the CU's L1 two line look-ups for every line of data.  Here a wavefront owns 16 rows x 4
// blocks = 16 contiguous pieces of 576 bytes, requests them all at once and into LDS without passing
// registers (ten global_load_lds: a row's 36 sixteen-byte pieces back to back and a 37th of padding,
// so that rows, 592 bytes apart, fall in different banks for the MFMA's reads), and multiplies when
// they have landed.  The quantized activations come in slices of four blocks (a KB a row, with the
// slice's sums and scales), moved by global_load_lds as well.  The arithmetic is the kernel's above,
// block by block, all LDS reads and MFMAs of the four blocks issued before the first integer multiply.
// A workgroup is one row group, its wavefronts the row's groups of four blocks (rows of up to 32
// blocks); all slices of the activations are staged, and the wavefronts' sums are added in the order
// of the blocks through LDS.  Small workgroups, two to a CU: one streams while the other multiplies.
// Measured at 14336x4096, 8 rows: 12.0 us against the kernel above's 12.1 (the data movement alone
// takes 7.5 us: what is left is the multiplication, which two workgroups a CU overlap too little);
// at 4096x4096 6.0 us against 6.9.  (Rows split between workgroups, one slice each, with the
// partial sums added by whichever workgroup finishes last, were tried for longer rows: the three
// trips to memory at the end cost 3 us, more than the split gains.)
constexpr int TS_ROW_PIECES = 37;
constexpr int TS_ROW_BYTES = TS_ROW_PIECES * 16;   // 592
constexpr int TS_SLOT = 16 * TS_ROW_BYTES;         // 9472
constexpr int TS_Q_STRIDE = 1024 + 16;             // a row of an activation slice (padded: 16 rows, 16 banks apart)
template <int ACTS>
struct SpanLds {
    static constexpr int OFF_BS = ACTS * TS_Q_STRIDE;  // int16 sums [ACTS][4 blocks][16]
    static constexpr int OFF_D = OFF_BS + ACTS * 128;  // f32 scales [4 blocks][16 rows]
    static constexpr int SLICE = OFF_D + 256;
    static constexpr size_t bytes(int slices, int waves) { return (size_t)slices * SLICE + (size_t)waves * TS_SLOT; }
};

template <int ACTS>
__global__ __launch_bounds__(512) void thin_span_q4_k_kernel(const uint8_t *__restrict__ W, size_t row_stride, int rows, int nb,
                                                            int batch, const int8_t *__restrict__ aq,
                                                            const float *__restrict__ ad, const int16_t *__restrict__ absums,
                                                            float *__restrict__ y) {
    using L = SpanLds<ACTS>;
    extern __shared__ uint4 smem[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
    const uint32_t lds0 = lds_address(lds);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = (int)blockDim.x >> 6;
    const int kg = wave, slices = waves;  // a wavefront per group of four blocks
    const int row0 = (int)blockIdx.x * 16;
    const int cols = nb * QK_K;
    uint8_t *const lds_w = lds + slices * L::SLICE;

    // ---- the activations: a wavefront fetches the slice it multiplies, so that it waits for nobody ----
#pragma unroll
    for (int piece = 0; piece < ACTS + 2; piece++) {
        const int sl = wave;
        const int k = sl;
        const uint32_t base = lds0 + (uint32_t)sl * L::SLICE;
        if (piece < ACTS) {
            dma16(base + piece * TS_Q_STRIDE, aq + (size_t)min(piece, batch - 1) * cols + (size_t)k * 1024, (uint32_t)lane * 16);
        } else if (piece == ACTS) {  // the 64 sums of a row's slice are 128 bytes: eight rows an instruction
#pragma unroll
            for (int h = 0; h < ACTS / 8; h++) {
                const int tok = min(h * 8 + (lane >> 3), batch - 1);
                dma16(base + L::OFF_BS + h * 1024, reinterpret_cast<const uint8_t *>(absums) + (size_t)k * 128,
                      (uint32_t)tok * (uint32_t)nb * 32u + (uint32_t)(lane & 7) * 16u);
            }
        } else {  // the scales, [block][row]
            const int tok = min(lane & 15, batch - 1);
            dma4(base + L::OFF_D, ad + (size_t)k * 4, ((uint32_t)tok * (uint32_t)nb + (uint32_t)(lane >> 4)) * 4u);
        }
    }
    // ---- this wavefront's 16 rows x 4 blocks: slot piece s = 64 c + lane is row s / 37, piece s % 37 ----
    {
        const int rbase = min(row0, rows - 1);  // (a wavefront past the matrix reads its last row and stores nothing)
        const uint8_t *src = W + (size_t)rbase * row_stride + (size_t)kg * 576;
        const uint32_t slot = lds_address(lds_w) + (uint32_t)wave * TS_SLOT;
#pragma unroll
        for (int c = 0; c < 10; c++) {
            const int sl = 64 * c + lane;
            const int r = min(sl / TS_ROW_PIECES, 15), q = min(sl % TS_ROW_PIECES, 35);  // (the 37th piece: the 36th again)
            const uint32_t off = (uint32_t)(min(row0 + r, rows - 1) - rbase) * (uint32_t)row_stride + (uint32_t)q * 16u;
            if (c < 9) dma16(slot + c * 1024, src, off);
            else if (lane < 16 * TS_ROW_PIECES - 576) dma16(slot + 9 * 1024, src, off);
        }
    }
    // Nothing is shared before the sums: a wavefront multiplies as soon as ITS slice and ITS rows have landed.
    // (With the slices' pieces dealt round the wavefronts there was a barrier here, reached only once the
    // memory pipeline had taken every wavefront's requests.)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    const int j = lane & 15, g = lane >> 4;
    const int act = min(j, ACTS - 1);  // (rows past the staged ones repeat the last; their results are not stored)
    const uint8_t *slice = lds + wave * L::SLICE;
    const uint8_t *a_q = slice + act * TS_Q_STRIDE + 8 * g;
    const uint8_t *a_bs = slice + L::OFF_BS + act * 128 + 8 * g;
    const float *a_d = reinterpret_cast<const float *>(slice + L::OFF_D) + 4 * g;
    uint8_t *const my_slot = lds_w + wave * TS_SLOT;
    const uint8_t *a_w = my_slot + j * TS_ROW_BYTES;
    auto as_long = [](uint2 v) { return (long)(((unsigned long)v.y << 32) | v.x); };
    v4f_t acc = {0.f, 0.f, 0.f, 0.f};
    // Everything the four blocks need is read from LDS first: with two wavefronts to a SIMD there is nothing
    // else to hide a block's chain of LDS reads, MFMAs and integer multiplies behind but the other blocks.
    uint4 hd[4];
    uint2 wq[4][4], alo[4][4], ahi[4][4], bsw[4];
    v4f_t da[4];
#pragma unroll
    for (int blk = 0; blk < 4; blk++) {
        hd[blk] = *reinterpret_cast<const uint4 *>(a_w + blk * Q4_K_BYTES);
#pragma unroll
        for (int c = 0; c < 4; c++) {
            wq[blk][c] = *reinterpret_cast<const uint2 *>(a_w + blk * Q4_K_BYTES + 16 + 32 * c + 8 * g);
            alo[blk][c] = *reinterpret_cast<const uint2 *>(a_q + blk * QK_K + 64 * c);
            ahi[blk][c] = *reinterpret_cast<const uint2 *>(a_q + blk * QK_K + 64 * c + 32);
        }
        bsw[blk] = *reinterpret_cast<const uint2 *>(a_bs + blk * 32);
        da[blk] = *reinterpret_cast<const v4f_t *>(a_d + blk * 16);
    }
    const v4i_t zero = {0, 0, 0, 0};
    v4i_t t0[4][4], t1[4][4];
#pragma unroll
    for (int blk = 0; blk < 4; blk++)
#pragma unroll
        for (int c = 0; c < 4; c++) {  // sub-blocks 2c (low nibbles) and 2c+1 (high)
            const uint2 q = wq[blk][c];
            const uint2 lo = make_uint2(q.x & 0x0f0f0f0fu, q.y & 0x0f0f0f0fu);
            const uint2 hi = make_uint2((q.x >> 4) & 0x0f0f0f0fu, (q.y >> 4) & 0x0f0f0f0fu);
            t0[blk][c] = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(alo[blk][c]), as_long(lo), zero, 0, 0, 0);
            t1[blk][c] = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(ahi[blk][c]), as_long(hi), zero, 0, 0, 0);
        }
#pragma unroll
    for (int blk = 0; blk < 4; blk++) {
        const uint4 h = hd[blk];
        const uint32_t sc_lo = h.y & 0x3f3f3f3fu, m_lo = h.z & 0x3f3f3f3fu;
        const uint32_t sc_hi = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);
        const uint32_t m_hi = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
        v4i_t s1 = {0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t scw = (c < 2 ? sc_lo : sc_hi) >> (16 * (c & 1));
            const int sc0 = scw & 0xff, sc1 = (scw >> 8) & 0xff;
#pragma unroll
            for (int r = 0; r < 4; r++) s1[r] += __mul24(sc0, t0[blk][c][r]) + __mul24(sc1, t1[blk][c][r]);
        }
        const uint32_t mw = (g < 2 ? m_lo : m_hi) >> (16 * (g & 1));
        const _Float16 m0 = (_Float16)(int)(mw & 0xff), m1 = (_Float16)(int)((mw >> 8) & 0xff);
        const v4h_t mh = {m0, m0, m1, m1};
        const v4h_t bh = {(_Float16)(int)(int16_t)(bsw[blk].x & 0xffff), (_Float16)(int)(int16_t)(bsw[blk].x >> 16),
                          (_Float16)(int)(int16_t)(bsw[blk].y & 0xffff), (_Float16)(int)(int16_t)(bsw[blk].y >> 16)};
        const v4f_t zf = {0.f, 0.f, 0.f, 0.f};
        const v4f_t s2 = __builtin_amdgcn_mfma_f32_16x16x16f16(bh, mh, zf, 0, 0, 0);
        const float d = h2f(h.x & 0xffffu), ndmin = -h2f(h.x >> 16);
#pragma unroll
        for (int r = 0; r < 4; r++) acc[r] = fmaf(da[blk][r], fmaf(ndmin, s2[r], d * (float)s1[r]), acc[r]);
    }

    const int row = row0 + j;
    // the row's groups of four blocks meet in LDS (every wavefront's own slot, which it has read for the
    // last time) and the first wavefront adds them in their order
    if (waves > 1) {
        if (wave > 0) *reinterpret_cast<v4f_t *>(my_slot + lane * 16) = acc;
        __syncthreads();
        if (wave > 0) return;
        for (int k = 1; k < waves; k++) {
            const v4f_t o = *reinterpret_cast<const v4f_t *>(lds_w + k * TS_SLOT + lane * 16);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += o[r];
        }
    }
#pragma unroll
    for (int r = 0; r < 4; r++)
        if (4 * g + r < batch && row < rows) y[(size_t)(4 * g + r) * rows + row] = acc[r];
}

// ------------------------------------------------------------------ thin GEMM streamed in chunks (Q6_K)
//
// The Q6_K kernel above loads a block's planes into registers with five gather-like loads per lane (sixteen
// rows an instruction) and walks a row group's blocks as a chain of round trips.  Here a workgroup is ONE row
// group of 16 rows and its wavefronts split the row's blocks; a wavefront moves a chunk -- S6_CB blocks of its 16
// rows, and the same blocks of the (at most 8) quantized activation rows -- into an LDS buffer of its own with
// global_load_lds (a lane names its own 16-byte piece: the LDS image is the rows back to back,
// [ql CB x 128 | qh CB x 64 | sc CB x 16 | the 16 bytes around the chunk's d] a row; the activations CB x 16 pieces a
// row and one of padding, so that the rows of a read fall in different banks), and multiplies the chunk when it
// has landed; with two buffers the next chunk travels meanwhile.  Nothing is shared before the sums: no barrier in
// the loop.  The arithmetic is the kernel's above.  (The longer a chunk, the longer the contiguous runs the
// planar rows give the memory system: a block's run is 128 bytes.)
// Measured at 4096 x 14336, 8 rows, from quantized activations (us): chunks of 2 blocks, one buffer, 14 wavefronts 16.3;
// 2 blocks, two buffers, 7 wavefronts 16.7 - 17.1; one block, two to four buffers, 6 to 13 wavefronts 17.8 - 20.0; chunks of 4
// blocks 23 and more; the kernel above 19.7.  More wavefronts beat deeper buffers: a wavefront issues one instruction
// in five clocks or so, and a chunk is some 600 of them.
constexpr int S6_CB = 2;                                // blocks of a chunk (2 or 4: the chunk's d sit in one aligned 16 bytes)
constexpr int S6_BUFS = 1;                              // 1 or 2
constexpr int S6_MAX_WAVES = 14;
constexpr int S6_WPIECES = 13 * S6_CB + 1;              // 27 / 53: odd, rows 8 banks apart
constexpr int S6_WROW = S6_WPIECES * 16;
constexpr int S6_WBUF = 16 * S6_WROW;
constexpr int S6_APIECES = 16 * S6_CB + 1;
constexpr int S6_AROW = S6_APIECES * 16;
constexpr int S6_ABUF = 8 * S6_AROW + S6_CB * 32;       // quants of 8 rows, then the scales [CB blocks][8 rows]
constexpr int S6_BUF = S6_WBUF + S6_ABUF;
constexpr int S6_WREQ = (16 * S6_WPIECES + 63) / 64, S6_AREQ = (8 * S6_APIECES + 63) / 64;
constexpr int S6_REQUESTS = S6_WREQ + S6_AREQ + 1;      // requests of a chunk
static_assert(S6_BUF % 16 == 0 && (size_t)S6_MAX_WAVES * S6_BUFS * S6_BUF <= 160 * 1024 && S6_REQUESTS < 64, "LDS of a CU; vmcnt");

__global__ __launch_bounds__(64 * S6_MAX_WAVES) void thin_stream_q6_k_kernel(const uint8_t *__restrict__ W, Layout lay, int rows, int nb,
                                                                           int batch, const int8_t *__restrict__ aq,
                                                                           const float *__restrict__ ad, float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
    const int cols = nb * QK_K;
    // a batch wider than 8 is a grid of groups of 8 activation rows: blockIdx.y picks the group
    aq += (size_t)blockIdx.y * 8 * cols;
    ad += (size_t)blockIdx.y * 8 * nb;
    y += (size_t)blockIdx.y * 8 * rows;
    batch = min(8, batch - (int)blockIdx.y * 8);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = (int)blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int row0 = (int)blockIdx.x * 16;
    const int chunks = nb / S6_CB;  // (nb is a multiple of S6_CB)
    const int c_begin = chunks * wave / waves, c_end = chunks * (wave + 1) / waves;
    uint8_t *const my_lds = lds + (size_t)wave * S6_BUFS * S6_BUF;
    const uint32_t my_lds_a = lds_address(my_lds);

    // ---- what a lane fetches of a chunk: fixed pieces, the chunk number moves the addresses ----
    // weights: slot piece s = 64 i + lane is row s / S6_WPIECES, piece s % S6_WPIECES of that row's image
    const int rbase = min(row0, rows - 1);  // (rows past the matrix read its last row and store nothing)
    const uint8_t *w_base = (const uint8_t *)scalar_pointer(W + (size_t)rbase * lay.row_stride);
    uint32_t w_off[S6_WREQ], w_step[S6_WREQ];
    bool w_is_d[S6_WREQ];
#pragma unroll
    for (int i = 0; i < S6_WREQ; i++) {
        const int sidx = min(64 * i + lane, 16 * S6_WPIECES - 1);
        const int r = sidx / S6_WPIECES, p = sidx % S6_WPIECES;
        const uint32_t ro = (uint32_t)(min(row0 + r, rows - 1) - rbase) * (uint32_t)lay.row_stride;
        w_is_d[i] = p == 13 * S6_CB;
        if (p < 8 * S6_CB) w_off[i] = ro + (uint32_t)p * 16, w_step[i] = 128 * S6_CB;
        else if (p < 12 * S6_CB) w_off[i] = ro + (uint32_t)lay.off_a + (uint32_t)(p - 8 * S6_CB) * 16, w_step[i] = 64 * S6_CB;
        else if (p < 13 * S6_CB) w_off[i] = ro + (uint32_t)lay.off_b + (uint32_t)(p - 12 * S6_CB) * 16, w_step[i] = 16 * S6_CB;
        else w_off[i] = ro + (uint32_t)lay.off_c, w_step[i] = 16;  // the aligned 16 bytes that hold the chunk's scales d
    }
    // quants: piece s = 64 i + lane is activation row s / S6_APIECES, piece s % S6_APIECES (the last: the one before again)
    uint32_t a_off[S6_AREQ];
#pragma unroll
    for (int i = 0; i < S6_AREQ; i++) {
        const int sidx = min(64 * i + lane, 8 * S6_APIECES - 1);
        const int a = min(sidx / S6_APIECES, batch - 1), p = min(sidx % S6_APIECES, 16 * S6_CB - 1);
        a_off[i] = (uint32_t)a * (uint32_t)cols + (uint32_t)p * 16;
    }
    const uint32_t d_off = ((uint32_t)min(lane & 7, batch - 1) * (uint32_t)nb + (uint32_t)((lane >> 3) % S6_CB)) * 4u;  // [block][row]
    auto fetch_chunk = [&](int c, int buf) {  // S6_REQUESTS requests
        const uint32_t base = my_lds_a + (uint32_t)buf * S6_BUF;
#pragma unroll
        for (int i = 0; i < S6_WREQ; i++) {
            const uint32_t off = w_off[i] + (w_is_d[i] ? (uint32_t)(c * S6_CB >> 3) : (uint32_t)c) * w_step[i];
            if (i < S6_WREQ - 1 || lane < 16 * S6_WPIECES - (S6_WREQ - 1) * 64) dma16(base + i * 1024, w_base, off);
        }
        const int8_t *q_base = aq + (size_t)c * (S6_CB * QK_K);
#pragma unroll
        for (int i = 0; i < S6_AREQ; i++)
            if (i < S6_AREQ - 1 || lane < 8 * S6_APIECES - (S6_AREQ - 1) * 64) dma16(base + S6_WBUF + i * 1024, q_base, a_off[i]);
        if (lane < 8 * S6_CB) dma4(base + S6_WBUF + 8 * S6_AROW, ad + (size_t)c * S6_CB, d_off);
    };

    // activation operand row j of the MFMA: activation j % 8, and only the k-groups of its half are real
    const bool real = (j < 8) == (g < 2);
    auto as_long = [](uint2 v) { return (long)(((unsigned long)v.y << 32) | v.x); };
    v4f_t acc = {0.f, 0.f, 0.f, 0.f};
    auto multiply_chunk = [&](int c, int buf) {
        const uint8_t *wb = my_lds + (size_t)buf * S6_BUF + j * S6_WROW;
        const uint8_t *ab = my_lds + (size_t)buf * S6_BUF + S6_WBUF;
        const uint8_t *a_q = ab + (size_t)(j & 7) * S6_AROW + 8 * g;
        const float *a_d = reinterpret_cast<const float *>(ab + 8 * S6_AROW) + 4 * (g & 1);
#pragma unroll
        for (int b = 0; b < S6_CB; b++) {
            const uint4 scv = *reinterpret_cast<const uint4 *>(wb + 192 * S6_CB + 16 * b);
            const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
            const float d = h2f(*reinterpret_cast<const uint16_t *>(wb + 208 * S6_CB + (((S6_CB * c + b) * 2) & 15)));
            const v4i_t zero = {0, 0, 0, 0};
            v4i_t isum = {0, 0, 0, 0};
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const uint2 qla = *reinterpret_cast<const uint2 *>(wb + 128 * b + h * 64 + 8 * g);
                const uint2 qlb = *reinterpret_cast<const uint2 *>(wb + 128 * b + h * 64 + 32 + 8 * g);
                const uint2 qh = *reinterpret_cast<const uint2 *>(wb + 128 * S6_CB + 64 * b + h * 32 + 8 * g);
#pragma unroll
                for (int v = 0; v < 4; v++) {  // weights h*128 + 32*v + l, l = 8g .. 8g+7
                    const uint2 ql = (v & 1) ? qlb : qla;
                    auto code = [&](uint32_t lo, uint32_t hi) {  // four 6-bit codes, as signed bytes q - 32
                        const uint32_t nib = (v >= 2 ? lo >> 4 : lo) & 0x0f0f0f0fu;
                        const uint32_t top = ((hi >> (2 * v)) & 0x03030303u) << 4;
                        return ((nib | top) + 0x60606060u) ^ 0x80808080u;
                    };
                    const uint2 wq = make_uint2(code(ql.x, qh.x), code(ql.y, qh.y));
                    uint2 a = *reinterpret_cast<const uint2 *>(a_q + b * QK_K + h * 128 + 32 * v);
                    if (!real) a = make_uint2(0u, 0u);
                    const v4i_t t = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(a), as_long(wq), zero, 0, 0, 0);
                    const int si = h * 8 + 2 * v + (g >> 1);  // the scale of this lane's 16-wide group
                    const int sc = (int)(int8_t)((scw[si >> 2] >> (8 * (si & 3))) & 0xff);
#pragma unroll
                    for (int r = 0; r < 4; r++) isum[r] += __mul24(sc, t[r]);
                }
            }
            const v4f_t da = *reinterpret_cast<const v4f_t *>(a_d + b * 8);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += (d * da[r]) * (float)isum[r];
        }
    };

    // requests complete in order, so "all but the youngest chunk's requests" means the older chunk has landed
    if (c_begin < c_end) fetch_chunk(c_begin, 0);
    for (int c = c_begin; c < c_end; c++) {
        const int buf = S6_BUFS > 1 ? (c - c_begin) & 1 : 0;
        if (S6_BUFS > 1 && c + 1 < c_end) {
            fetch_chunk(c + 1, buf ^ 1);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S6_REQUESTS) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        multiply_chunk(c, buf);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the buffer has been read: a later chunk may land in it
        if (S6_BUFS == 1 && c + 1 < c_end) fetch_chunk(c + 1, 0);
    }
    // the two 16-wide halves of every result sit 32 lanes apart
#pragma unroll
    for (int r = 0; r < 4; r++) acc[r] += __shfl_xor(acc[r], 32);
    if (waves > 1) {  // the wavefronts' shares of the row meet in LDS and are added in their order
        __syncthreads();
        float *red = reinterpret_cast<float *>(lds);
        if (wave > 0) {
#pragma unroll
            for (int r = 0; r < 4; r++) red[((wave - 1) * 4 + r) * 64 + lane] = acc[r];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int k = 0; k < waves - 1; k++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += red[(k * 4 + r) * 64 + lane];
    }
    if (g < 2) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int b = 4 * g + r;
            if (b < batch && row0 + j < rows) y[(size_t)b * rows + row0 + j] = acc[r];
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
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_q4_k_kernel<LPR, NB>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)THIN_LDS_LIMIT));
            sized = true;
        }
        hipLaunchKernelGGL((thin_q4_k_kernel<LPR, NB>), dim3(grid), dim3(THIN_THREADS), shmem, s, w->dev,
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

constexpr size_t TM_LDS_LIMIT = 160 * 1024;


template <int RG, int ACTS, bool Q5>
static int launch_thin_mfma_kind(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const size_t shmem = tm_lds_bytes(ACTS, (int)w->cols, Q5);
    static bool sized = false;
    if (!sized) {
        FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_mfma_q4_k_kernel<RG, ACTS, Q5>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)TM_LDS_LIMIT));
        sized = true;
    }
    const size_t groups = (w->rows + 15) / 16;
    hipLaunchKernelGGL((thin_mfma_q4_k_kernel<RG, ACTS, Q5>), dim3((unsigned)((groups + RG - 1) / RG), (unsigned)((batch + ACTS - 1) / ACTS)),
                       dim3(64 * TM_WAVES),
                       shmem, s, w->dev, w->layout.row_stride, (int)w->rows, (int)(w->cols / QK_K), batch, a.q, a.d,
                       a.bsums, y);
    FRK_LAUNCH_CHECK("thin mfma gemm");
    return FRK_OK;
}
template <int RG, int ACTS>
static int launch_thin_mfma(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    return w->kind == FRK_KIND_Q5_K ? launch_thin_mfma_kind<RG, ACTS, true>(w, batch, a, y, s)
                                    : launch_thin_mfma_kind<RG, ACTS, false>(w, batch, a, y, s);
}
// rows of activations the matrix-core kernel can stage for this Q4_K or Q5_K matrix (16, 8, 4 or 0)
static int thin_mfma_acts(const frk_weights *w) {
    for (int acts = 16; acts >= 4; acts /= 2)
        if (tm_lds_bytes(acts, (int)w->cols, w->kind == FRK_KIND_Q5_K) <= TM_LDS_LIMIT) return acts;
    return 0;
}
template <int ACTS>
static int launch_thin_mfma_rg(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    // row groups per workgroup: as many as still give (nearly) every CU a workgroup -- one per CU was
    // measured faster than two, the activations being staged half as often; the rest of the 8
    // wavefronts split the blocks, four or more each
    const size_t groups = (w->rows + 15) / 16, nb = w->cols / QK_K;
    int rg = 8;
    while (rg > 1 && ((groups + rg - 1) / rg < 224 && (size_t)(TM_WAVES / rg) * 4 <= nb)) rg /= 2;
    switch (rg) {
        case 8: return launch_thin_mfma<8, ACTS>(w, batch, a, y, s);
        case 4: return launch_thin_mfma<4, ACTS>(w, batch, a, y, s);
        case 2: return launch_thin_mfma<2, ACTS>(w, batch, a, y, s);
        default: return launch_thin_mfma<1, ACTS>(w, batch, a, y, s);
    }
}

template <int RG, int ACTS>
static int launch_thin_mfma6(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const size_t shmem = t6_lds_bytes(ACTS, (int)w->cols);
    static bool sized = false;
    if (!sized) {
        FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_mfma_q6_k_kernel<RG, ACTS>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)TM_LDS_LIMIT));
        sized = true;
    }
    const size_t groups = (w->rows + 15) / 16;
    hipLaunchKernelGGL((thin_mfma_q6_k_kernel<RG, ACTS>), dim3((unsigned)((groups + RG - 1) / RG), (unsigned)((batch + ACTS - 1) / ACTS)),
                       dim3(64 * TM_WAVES), shmem, s, w->dev, w->layout, (int)w->rows, (int)(w->cols / QK_K), batch, a.q, a.d, y);
    FRK_LAUNCH_CHECK("thin mfma gemm");
    return FRK_OK;
}
// rows of activations the Q6_K matrix-core kernel can stage for this matrix (8, 4 or 0)
static int thin_mfma6_acts(const frk_weights *w) {
    for (int acts = 8; acts >= 4; acts /= 2)
        if (t6_lds_bytes(acts, (int)w->cols) <= TM_LDS_LIMIT) return acts;
    return 0;
}
template <int ACTS>
static int launch_thin_mfma6_rg(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const size_t groups = (w->rows + 15) / 16, nb = w->cols / QK_K;
    int rg = 8;
    while (rg > 1 && ((groups + rg - 1) / rg < 224 && (size_t)(TM_WAVES / rg) * 4 <= nb)) rg /= 2;
    switch (rg) {
        case 8: return launch_thin_mfma6<8, ACTS>(w, batch, a, y, s);
        case 4: return launch_thin_mfma6<4, ACTS>(w, batch, a, y, s);
        case 2: return launch_thin_mfma6<2, ACTS>(w, batch, a, y, s);
        default: return launch_thin_mfma6<1, ACTS>(w, batch, a, y, s);
    }
}

// ---- the streamed Q6_K kernel: rows of whole chunks of blocks, groups of 8 activation rows ----
static bool thin_stream6_fits(const frk_weights *w) {
    const size_t nb = w->cols / QK_K;
    return w->kind == FRK_KIND_Q6_K && nb >= S6_CB && nb % S6_CB == 0 && (uint64_t)w->layout.row_stride * 16 < (1ull << 32) &&
           (uint64_t)w->cols * 8 < (1ull << 32);
}
static int launch_thin_stream6(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const size_t groups = (w->rows + 15) / 16, chunks = w->cols / QK_K / S6_CB;
    // a wavefront per four chunks or so, as many as LDS holds buffers for
    const int waves = (int)std::max<size_t>(1, std::min<size_t>(S6_MAX_WAVES, (chunks + 3) / 4));
    const size_t shmem = (size_t)waves * S6_BUFS * S6_BUF;
    static bool sized = false;
    if (!sized) {
        FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_stream_q6_k_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)TM_LDS_LIMIT));
        sized = true;
    }
    hipLaunchKernelGGL(thin_stream_q6_k_kernel, dim3((unsigned)groups, (unsigned)((batch + 7) / 8)), dim3(64 * waves), shmem, s, w->dev,
                       w->layout, (int)w->rows, (int)(w->cols / QK_K), batch, a.q, a.d, y);
    FRK_LAUNCH_CHECK("thin stream gemm (Q6_K)");
    return FRK_OK;
}

// ---- the span kernel: Q4_K rows of 4, 8, .. 32 blocks (a wavefront per four), up to 16 activation rows ----
static bool thin_span_fits(const frk_weights *w, int batch) {
    const size_t nb = w->cols / QK_K, n_kg = nb / 4;
    if (w->kind != FRK_KIND_Q4_K || nb % 4 || n_kg > 8 || batch < 1 || batch > 16) return false;
    if (nb * Q4_K_BYTES > w->layout.row_stride) return false;
    const size_t lds = batch > 8 ? SpanLds<16>::bytes((int)n_kg, (int)n_kg) : SpanLds<8>::bytes((int)n_kg, (int)n_kg);
    return lds <= TM_LDS_LIMIT;
}
template <int ACTS>
static int launch_thin_span(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    const size_t groups = (w->rows + 15) / 16;
    const int waves = (int)(w->cols / QK_K / 4);
    const size_t shmem = SpanLds<ACTS>::bytes(waves, waves);
    static bool sized = false;
    if (!sized) {
        FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&thin_span_q4_k_kernel<ACTS>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)TM_LDS_LIMIT));
        sized = true;
    }
    hipLaunchKernelGGL((thin_span_q4_k_kernel<ACTS>), dim3((unsigned)groups), dim3(64 * waves), shmem, s, w->dev,
                       w->layout.row_stride, (int)w->rows, (int)(w->cols / QK_K), batch, a.q, a.d, a.bsums, y);
    FRK_LAUNCH_CHECK("thin span gemm");
    return FRK_OK;
}

// Largest number of activation rows one launch can take for this matrix: up to 16 on the
// matrix-core path (Q4_K), else what fits LDS, at most 8.
int thin_gemm_max_batch(const frk_weights *w) {
    if ((w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K) && thin_mfma_acts(w) > 0) return thin_mfma_acts(w);
    if (w->kind == FRK_KIND_Q5_K) return 0;  // (no other batched kernel for Q5_K)
    const size_t per_row = (w->cols / QK_K) * (256 + (w->kind == FRK_KIND_Q4_K ? 8 : 16) * 4 + 4);
    for (int nbatch = 8; nbatch >= 2; nbatch /= 2)
        if (per_row * nbatch <= THIN_LDS_LIMIT) return nbatch;
    return 0;
}

// A batch of any width in one launch, where the kind has a kernel that takes one (Q6_K and Q5_K on the
// matrix cores: a grid of 8- and 16-row groups); 0 rows = no such kernel for this matrix.
int thin_gemm_wide_rows(const frk_weights *w) {
    if (w->kind == FRK_KIND_Q5_K && thin_mfma_acts(w) >= 16) return 65535 * 16;  // (groups of 16 rows)
    return (w->kind == FRK_KIND_Q6_K && thin_mfma6_acts(w) >= 8) ? 65535 * 8 : 0;
}
int launch_thin_gemm_wide(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    // Q5_K: many groups of activation rows fill the chip whatever the matrix, so a workgroup takes eight row groups
    if (w->kind == FRK_KIND_Q5_K) return launch_thin_mfma<8, 16>(w, batch, a, y, s);
    if (thin_stream6_fits(w)) return launch_thin_stream6(w, batch, a, y, s);
    return launch_thin_mfma6_rg<8>(w, batch, a, y, s);
}

// y[batch][rows] for 1 <= batch <= thin_gemm_max_batch(w) quantized activation rows (K-quants).
int launch_thin_gemm(const frk_weights *w, int batch, Q8KActs a, float *y, hipStream_t s) {
    if (batch > 2 && thin_span_fits(w, batch))
        return batch > 8 ? launch_thin_span<16>(w, batch, a, y, s) : launch_thin_span<8>(w, batch, a, y, s);
    // (two rows of Q4_K: the dot4 kernel is still ahead)
    if ((w->kind == FRK_KIND_Q4_K && thin_mfma_acts(w) > 0 && batch > 2) || w->kind == FRK_KIND_Q5_K) {
        // the fewest staged rows that hold the batch
        if (batch <= 4) return launch_thin_mfma_rg<4>(w, batch, a, y, s);
        if (batch <= 8) return launch_thin_mfma_rg<8>(w, batch, a, y, s);
        return launch_thin_mfma_rg<16>(w, batch, a, y, s);
    }
    if (w->kind == FRK_KIND_Q6_K && batch > 2 && thin_stream6_fits(w)) return launch_thin_stream6(w, batch, a, y, s);
    if (w->kind == FRK_KIND_Q6_K && batch > 2 && thin_mfma6_acts(w) >= (batch > 4 ? 8 : 4))
        return batch > 4 ? launch_thin_mfma6_rg<8>(w, batch, a, y, s) : launch_thin_mfma6_rg<4>(w, batch, a, y, s);
    if (batch > 4) return launch_thin_nb<8>(w, batch, a, y, s);
    if (batch > 2) return launch_thin_nb<4>(w, batch, a, y, s);
    return launch_thin_nb<2>(w, batch, a, y, s);
}

}  // namespace frk

