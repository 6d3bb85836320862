// Decode GEMV for Q6_K and Q8_0 with every load of a wavefront's share in flight at once.
//
// Two ways of cutting a matrix between wavefronts.  Rows: one wavefront owns one weight row; lane l owns units
// l, l+64, ... (a unit is 64 weights of Q6_K or 16 of Q8_0, the same units as the looping kernels in
// frk_gemv.hip); the activation is shared by the rows of a workgroup through LDS, or read by every lane from L2.
// Columns: a workgroup owns a few rows and wavefront w the same 64 units of every one of them, so that a lane's
// slice of the activation is loaded (Q6_K: quantized) once and kept in registers -- nothing is shared before the
// sums, and no barrier stands between the requests and the arithmetic.  All of a lane's loads -- its share of
// the activation first, because a wavefront's loads return in issue order and the activation comes from L2,
// then its weights from HBM -- are issued before any arithmetic, so a CU holds tens of kilobytes in flight
// instead of one loop iteration's worth.  Rows too long for either fall back to the looping kernels.
#include "frk_device.hpp"

namespace frk {

// ------------------------------------------------------------------ Q6_K x Q8_K
// dot_q6_k_q8 (crates/frink-quant/src/lib.rs:1069-1110) over the planar resident layout.
// Unit = (block b, half h, 16-lane column t): ql[64h+16t..], ql[64h+32+16t..], qh[32h+16t..]
// hold four 16-weight groups with scales sc[8h+t+{0,2,4,6}].  The -32 offset is folded as
// -32 * (sum of the 16 activation quants), which Q8_K's bsums already hold.
// FUSED: the workgroup (16 wavefronts, XB blocks of the activation each) quantizes the f32 activation
// to Q8_K into LDS itself, bit-exact with quantize_activations_q8_k, while its weight loads are in
// flight, and its 16 rows share that one copy (a row of this kind is shorter than the activation it
// multiplies, so per-lane reads of the activation from L2 would double the traffic); otherwise the
// quantized activation is read from global memory.
template <int U, int XB, bool FUSED>
__global__ __launch_bounds__(FUSED ? 1024 : 256) void gemv_q6_k_direct_kernel(
    const uint8_t *__restrict__ W, Layout lay, int rows, int nb, const float *__restrict__ x,
    const int8_t *__restrict__ aq, const float *__restrict__ ad, const int16_t *__restrict__ absums,
    float *__restrict__ y) {
    constexpr int WAVES = FUSED ? 16 : 4;
    extern __shared__ uint4 smem_direct[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = min((int)blockIdx.x * WAVES + wave, rows - 1);  // a wavefront past the end repeats the last row
    const bool store = (int)blockIdx.x * WAVES + wave < rows;
    const uint8_t *row = W + (size_t)r * lay.row_stride;
    const int units = nb * 4;

    // the activation's loads go out before the weights': a wavefront's loads return in issue order
    float4 xv[FUSED ? XB : 1];
    if (FUSED) {
#pragma unroll
        for (int i = 0; i < XB; i++) {
            const int b = min(wave + i * WAVES, nb - 1);
            xv[i] = reinterpret_cast<const float4 *>(x + (size_t)b * QK_K)[lane];
        }
    }
    uint4 a0[U], a1[U], a2[U], a3[U], bs[U];
    float da[U];
    if (!FUSED) {
#pragma unroll
        for (int j = 0; j < U; j++) {
            const int u = min(lane + 64 * j, units - 1);  // a lane past the end repeats the last unit, unused
            const int b = u >> 2, h = (u >> 1) & 1, t = u & 1;
            const int8_t *abase = aq + b * 256 + h * 128 + t * 16;
            a0[j] = *reinterpret_cast<const uint4 *>(abase);
            a1[j] = *reinterpret_cast<const uint4 *>(abase + 32);
            a2[j] = *reinterpret_cast<const uint4 *>(abase + 64);
            a3[j] = *reinterpret_cast<const uint4 *>(abase + 96);
            bs[j] = *reinterpret_cast<const uint4 *>(absums + b * 16 + h * 8);  // the half's eight 16-wide sums
            da[j] = ad[b];
        }
    }
    uint4 qla[U], qlb[U], qh[U];
    uint2 scv[U];
    uint32_t dbits[U];
#pragma unroll
    for (int j = 0; j < U; j++) {
        const int u = min(lane + 64 * j, units - 1);
        const int b = u >> 2, h = (u >> 1) & 1, t = u & 1;
        qla[j] = *reinterpret_cast<const uint4 *>(row + (size_t)b * 128 + h * 64 + t * 16);
        qlb[j] = *reinterpret_cast<const uint4 *>(row + (size_t)b * 128 + h * 64 + 32 + t * 16);
        qh[j] = *reinterpret_cast<const uint4 *>(row + lay.off_a + (size_t)b * 64 + h * 32 + t * 16);
        scv[j] = *reinterpret_cast<const uint2 *>(row + lay.off_b + (size_t)b * 16 + h * 8);
        dbits[j] = *reinterpret_cast<const uint16_t *>(row + lay.off_c + (size_t)b * 2);
    }
    if (FUSED) {
        int8_t *sq = reinterpret_cast<int8_t *>(smem_direct);
        int16_t *sbs = reinterpret_cast<int16_t *>(sq + (size_t)nb * 256);
        float *sd = reinterpret_cast<float *>(sbs + (size_t)nb * 16);
#pragma unroll
        for (int i = 0; i < XB; i++) {
            const int b = wave + i * WAVES;
            float d;
            int s16;
            const uint32_t packed = quantize_q8_k_lane(xv[i], d, s16);
            if (b < nb) {  // uniform across the wavefront
                reinterpret_cast<uint32_t *>(sq + b * QK_K)[lane] = packed;
                if ((lane & 3) == 0) sbs[b * 16 + (lane >> 2)] = (int16_t)s16;
                if (lane == 0) sd[b] = d;
            }
        }
        lds_barrier();  // publishes LDS, does not wait for the weight loads
    }

    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < U; j++) {
        const int t = lane & 1;  // (lane + 64*j) & 1
        if (FUSED) {  // this unit's slice of the activation, from the workgroup's copy
            const int8_t *sq = reinterpret_cast<const int8_t *>(smem_direct);
            const int16_t *sbs = reinterpret_cast<const int16_t *>(sq + (size_t)nb * 256);
            const float *sd = reinterpret_cast<const float *>(sbs + (size_t)nb * 16);
            const int u = min(lane + 64 * j, units - 1);
            const int b = u >> 2, h = (u >> 1) & 1;
            const int8_t *abase = sq + b * 256 + h * 128 + t * 16;
            a0[j] = *reinterpret_cast<const uint4 *>(abase);
            a1[j] = *reinterpret_cast<const uint4 *>(abase + 32);
            a2[j] = *reinterpret_cast<const uint4 *>(abase + 64);
            a3[j] = *reinterpret_cast<const uint4 *>(abase + 96);
            bs[j] = *reinterpret_cast<const uint4 *>(sbs + b * 16 + h * 8);
            da[j] = sd[b];
        }
        int d1 = 0, d2 = 0, d3 = 0, d4 = 0;
#define FRK_Q6_STEP(c)                                                                                   \
    d1 = dot4((qla[j].c & 0x0f0f0f0fu) | ((qh[j].c << 4) & 0x30303030u), a0[j].c, d1);                    \
    d2 = dot4((qlb[j].c & 0x0f0f0f0fu) | ((qh[j].c << 2) & 0x30303030u), a1[j].c, d2);                    \
    d3 = dot4(((qla[j].c >> 4) & 0x0f0f0f0fu) | (qh[j].c & 0x30303030u), a2[j].c, d3);                    \
    d4 = dot4(((qlb[j].c >> 4) & 0x0f0f0f0fu) | ((qh[j].c >> 2) & 0x30303030u), a3[j].c, d4);
        FRK_Q6_STEP(x)
        FRK_Q6_STEP(y)
        FRK_Q6_STEP(z)
        FRK_Q6_STEP(w)
#undef FRK_Q6_STEP
        const uint32_t slo = t ? (scv[j].x >> 8) : scv[j].x, shi = t ? (scv[j].y >> 8) : scv[j].y;
        const int s1 = (int)(int8_t)(slo & 0xff), s2 = (int)(int8_t)((slo >> 16) & 0xff);
        const int s3 = (int)(int8_t)(shi & 0xff), s4 = (int)(int8_t)((shi >> 16) & 0xff);
        // sums of groups t, t+2, t+4, t+6 of the half: 16-bit fields t, t+2 (x, y) and t+4, t+6 (z, w)
        const int sh = 16 * t;
        const int b1 = (int)(int16_t)(bs[j].x >> sh), b2 = (int)(int16_t)(bs[j].y >> sh);
        const int b3 = (int)(int16_t)(bs[j].z >> sh), b4 = (int)(int16_t)(bs[j].w >> sh);
        const int isum = s1 * (d1 - 32 * b1) + s2 * (d2 - 32 * b2) + s3 * (d3 - 32 * b3) + s4 * (d4 - 32 * b4);
        const float term = (h2f(dbits[j]) * da[j]) * (float)isum;
        acc += (lane + 64 * j < units) ? term : 0.0f;
    }
    acc = part_sum<64>(acc);
    if (lane == 0 && store) y[r] = acc;
}

// ------------------------------------------------------------------ Q6_K x f32, one launch, no barrier before the dots
// The same step -- quantize_activations_q8_k, then dot_q6_k_q8 per row -- with the work cut the other way:
// a workgroup takes 4 * U rows and wavefront w the columns of blocks 4w .. 4w+3 of all of them, the very
// blocks it quantizes itself.  A wavefront therefore waits for nobody before it multiplies: its slice of
// the activation goes through a corner of LDS that only it touches (quantized four values a lane, read
// back as this lane's 64 columns and kept in registers for every row), all its weight loads are in flight
// from the start, and the one workgroup barrier stands at the very end, where the wavefronts' sixteen
// partial sums a row meet.  (A barrier behind the weight loads, as in the kernel above, costs microseconds
// on long rows: a wavefront reaches it only once the memory pipeline has taken all its loads.)
// Round j of a wavefront covers rows 4j .. 4j+3 of the workgroup: lane = 16 * (row of the round) + unit,
// unit = (block of the slice, half, 16-byte column) as above.
constexpr int COLS_WAVE_LDS = 4 * (QK_K + 32 + 4);  // four blocks: quants, 16-wide sums, scale
template <int U, bool NT = false>
__global__ __launch_bounds__(1024) void gemv_q6_k_cols_kernel(const uint8_t *__restrict__ W, Layout lay, int rows, int nb,
                                                             const float *__restrict__ x, float *__restrict__ y) {
    typedef float xv_t __attribute__((ext_vector_type(4)));
    typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
    typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
    extern __shared__ uint4 smem_cols[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), waves = blockDim.x >> 6;
    uint8_t *mine = reinterpret_cast<uint8_t *>(smem_cols) + wave * COLS_WAVE_LDS;
    float *parts = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(smem_cols) + waves * COLS_WAVE_LDS);
    const int b0 = wave * 4, r0 = (int)blockIdx.x * 4 * U;

    // the activation's loads first: a wavefront's loads return in issue order
    xv_t xv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {  // (a block past the row's end: the last one again, not used)
        const float *src = x + (size_t)min(b0 + i, nb - 1) * QK_K + lane * 4;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xv[i]) : "v"(src) : "memory");
    }
    const int ul = lane & 15, bl = ul >> 2, h = (ul >> 1) & 1, t = ul & 1;
    const bool live = b0 + bl < nb;
    const int b = min(b0 + bl, nb - 1);
    u4_t qla[U], qlb[U], qh[U];
    u2_t scv[U];
    uint32_t dbits[U];
    auto request = [&](int j) {
        const int r = min(r0 + 4 * j + (lane >> 4), rows - 1);  // a row past the end: the last one again, not stored
        const uint8_t *row = W + (size_t)r * lay.row_stride;
        const uint8_t *p_l = row + (size_t)b * 128 + h * 64 + t * 16;
        const uint8_t *p_h = row + lay.off_a + (size_t)b * 64 + h * 32 + t * 16;
        const uint8_t *p_s = row + lay.off_b + (size_t)b * 16 + h * 8;
        const uint8_t *p_d = row + lay.off_c + (size_t)b * 2;
        if (NT) {  // (rows that start on a cache line: a wavefront's share of the two big planes is whole lines)
            asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(qla[j]) : "v"(p_l) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off offset:32 nt" : "=v"(qlb[j]) : "v"(p_l) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(qh[j]) : "v"(p_h) : "memory");
        } else {
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qla[j]) : "v"(p_l) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off offset:32" : "=v"(qlb[j]) : "v"(p_l) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qh[j]) : "v"(p_h) : "memory");
        }
        asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(scv[j]) : "v"(p_s) : "memory");
        asm volatile("global_load_ushort %0, %1, off" : "=v"(dbits[j]) : "v"(p_d) : "memory");
    };
    request(0);

    // ---- this wavefront's four blocks of the activation, through its own corner of LDS ----
    // (the other rounds are requested once the activation is here: behind twenty weight loads of each of
    // sixteen wavefronts, a late wavefront's activation came late)
    asm volatile("s_waitcnt vmcnt(5)" : "+v"(xv[0]), "+v"(xv[1]), "+v"(xv[2]), "+v"(xv[3]));
#pragma unroll
    for (int j = 1; j < U; j++) request(j);
    uint32_t *sq = reinterpret_cast<uint32_t *>(mine);
    int16_t *sbs = reinterpret_cast<int16_t *>(mine + 4 * QK_K);
    float *sd = reinterpret_cast<float *>(mine + 4 * QK_K + 4 * 32);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float d;
        int s16;
        const uint32_t packed = quantize_q8_k_lane<false>(make_float4(xv[i].x, xv[i].y, xv[i].z, xv[i].w), d, s16);
        sq[i * 64 + lane] = packed;
        if ((lane & 3) == 0) sbs[i * 16 + (lane >> 2)] = (int16_t)s16;
        if (lane == 0) sd[i] = d;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint8_t *abase = mine + bl * QK_K + h * 128 + t * 16;
    const uint4 a0 = *reinterpret_cast<const uint4 *>(abase), a1 = *reinterpret_cast<const uint4 *>(abase + 32);
    const uint4 a2 = *reinterpret_cast<const uint4 *>(abase + 64), a3 = *reinterpret_cast<const uint4 *>(abase + 96);
    const uint4 bs = *reinterpret_cast<const uint4 *>(sbs + bl * 16 + h * 8);  // the half's eight 16-wide sums
    const float da = sd[bl];
    // sums of groups t, t+2, t+4, t+6 of the half: 16-bit fields t, t+2 (x, y) and t+4, t+6 (z, w)
    const int sh = 16 * t;
    const int b1 = 32 * (int)(int16_t)(bs.x >> sh), b2 = 32 * (int)(int16_t)(bs.y >> sh);
    const int b3 = 32 * (int)(int16_t)(bs.z >> sh), b4 = 32 * (int)(int16_t)(bs.w >> sh);

    auto round = [&](const u4_t la, const u4_t lb, const u4_t hh, const u2_t sc, const uint32_t dbit) {
        int d1 = 0, d2 = 0, d3 = 0, d4 = 0;
#define FRK_Q6_STEP(c)                                                                     \
    d1 = dot4((la.c & 0x0f0f0f0fu) | ((hh.c << 4) & 0x30303030u), a0.c, d1);                \
    d2 = dot4((lb.c & 0x0f0f0f0fu) | ((hh.c << 2) & 0x30303030u), a1.c, d2);                \
    d3 = dot4(((la.c >> 4) & 0x0f0f0f0fu) | (hh.c & 0x30303030u), a2.c, d3);                \
    d4 = dot4(((lb.c >> 4) & 0x0f0f0f0fu) | ((hh.c >> 2) & 0x30303030u), a3.c, d4);
        FRK_Q6_STEP(x)
        FRK_Q6_STEP(y)
        FRK_Q6_STEP(z)
        FRK_Q6_STEP(w)
#undef FRK_Q6_STEP
        const uint32_t slo = t ? (sc.x >> 8) : sc.x, shi = t ? (sc.y >> 8) : sc.y;
        const int s1 = (int)(int8_t)(slo & 0xff), s2 = (int)(int8_t)((slo >> 16) & 0xff);
        const int s3 = (int)(int8_t)(shi & 0xff), s4 = (int)(int8_t)((shi >> 16) & 0xff);
        const int isum = s1 * (d1 - b1) + s2 * (d2 - b2) + s3 * (d3 - b3) + s4 * (d4 - b4);
        const float term = (h2f(dbit) * da) * (float)isum;
        return part_sum<16>(live ? term : 0.0f);
    };
    float sums[U];
#define FRK_COLS_ROUND(j)                                                                                            \
    if constexpr (U > j) {                                                                                           \
        asm volatile("s_waitcnt vmcnt(%5)"                                                                           \
                     : "+v"(qla[j]), "+v"(qlb[j]), "+v"(qh[j]), "+v"(scv[j]), "+v"(dbits[j])                         \
                     : "n"(5 * (U - 1 - j)));                                                                        \
        sums[j] = round(qla[j], qlb[j], qh[j], scv[j], dbits[j]);                                                    \
    }
    FRK_COLS_ROUND(0)
    FRK_COLS_ROUND(1)
    FRK_COLS_ROUND(2)
    FRK_COLS_ROUND(3)
    FRK_COLS_ROUND(4)
    FRK_COLS_ROUND(5)
#undef FRK_COLS_ROUND
#pragma unroll
    for (int j = 0; j < U; j++)
        if (ul == 0) parts[wave * (4 * U) + 4 * j + (lane >> 4)] = sums[j];
    lds_barrier();
    // a row's partial sums, in the order of the columns
    if ((int)threadIdx.x < 4 * U && r0 + (int)threadIdx.x < rows) {
        float v = 0.0f;
        for (int w = 0; w < waves; w++) v += parts[w * (4 * U) + threadIdx.x];
        y[r0 + threadIdx.x] = v;
    }
}

// ------------------------------------------------------------------ Q6_K experts, one job per (token, slot)
// The decode form of a mixture-of-experts down projection whose experts are Q6_K (run_expert,
// crates/frink-moe/src/lib.rs:1068-1165): job j multiplies expert ids[j]'s rows_e rows (the experts'
// matrices are stacked) by ITS activation x + j * x_stride, which the workgroup quantizes to Q8_K in
// LDS first (bit-exact with quantize_activations_q8_k).  Expert rows are short (768 columns = 12
// units in the usual case), so LPR lanes share a row and a wavefront takes 64 / LPR rows at a time,
// STEPS times, all of a lane's weight loads in flight before the activation is quantized.
// The arithmetic is dot_q6_k_q8's, as in the kernel above.  An id outside [0, n_experts) computes on
// expert 0 (the weighted sum leaves such a slot out).
template <int LPR, int STEPS>
__global__ __launch_bounds__(256) void gemv_q6_k_experts_kernel(const uint8_t *__restrict__ W, Layout lay, int rows_e, int nb,
                                                               int n_experts, const int32_t *__restrict__ ids,
                                                               const float *__restrict__ x, int x_stride,
                                                               float *__restrict__ y) {
    constexpr int PARTS = 64 / LPR, ROWS_WG = 4 * PARTS * STEPS;
    extern __shared__ uint4 smem_direct[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int part = lane / LPR, l = lane % LPR;
    const int job = blockIdx.y;
    int e = ids[job];
    if (e < 0 || e >= n_experts) e = 0;
    const int units = nb * 4;
    const int u = min(l, units - 1);  // (a lane past the row's units repeats the last, unused)
    const int b = u >> 2, h = (u >> 1) & 1, t = u & 1;
    const float *xj = x + (size_t)job * x_stride;

    constexpr int XB = 4;  // blocks of the activation a wavefront quantizes (nb <= 16)
    float4 xv[XB];
#pragma unroll
    for (int i = 0; i < XB; i++) xv[i] = reinterpret_cast<const float4 *>(xj + (size_t)min(wave + 4 * i, nb - 1) * QK_K)[lane];
    uint4 qla[STEPS], qlb[STEPS], qh[STEPS];
    uint2 scv[STEPS];
    uint32_t dbits[STEPS];
    int rr[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        rr[st] = (int)blockIdx.x * ROWS_WG + (st * 4 + wave) * PARTS + part;
        const uint8_t *row = W + ((size_t)e * rows_e + min(rr[st], rows_e - 1)) * lay.row_stride;
        qla[st] = *reinterpret_cast<const uint4 *>(row + (size_t)b * 128 + h * 64 + t * 16);
        qlb[st] = *reinterpret_cast<const uint4 *>(row + (size_t)b * 128 + h * 64 + 32 + t * 16);
        qh[st] = *reinterpret_cast<const uint4 *>(row + lay.off_a + (size_t)b * 64 + h * 32 + t * 16);
        scv[st] = *reinterpret_cast<const uint2 *>(row + lay.off_b + (size_t)b * 16 + h * 8);
        dbits[st] = *reinterpret_cast<const uint16_t *>(row + lay.off_c + (size_t)b * 2);
    }
    int8_t *sq = reinterpret_cast<int8_t *>(smem_direct);
    int16_t *sbs = reinterpret_cast<int16_t *>(sq + (size_t)nb * 256);
    float *sd = reinterpret_cast<float *>(sbs + (size_t)nb * 16);
#pragma unroll
    for (int i = 0; i < XB; i++) {
        const int bq = wave + 4 * i;
        float d;
        int s16;
        const uint32_t packed = quantize_q8_k_lane(xv[i], d, s16);
        if (bq < nb) {  // uniform across the wavefront
            reinterpret_cast<uint32_t *>(sq + bq * QK_K)[lane] = packed;
            if ((lane & 3) == 0) sbs[bq * 16 + (lane >> 2)] = (int16_t)s16;
            if (lane == 0) sd[bq] = d;
        }
    }
    lds_barrier();  // publishes LDS, does not wait for the weight loads

    const int8_t *abase = sq + b * 256 + h * 128 + t * 16;
    const uint4 a0 = *reinterpret_cast<const uint4 *>(abase), a1 = *reinterpret_cast<const uint4 *>(abase + 32);
    const uint4 a2 = *reinterpret_cast<const uint4 *>(abase + 64), a3 = *reinterpret_cast<const uint4 *>(abase + 96);
    const uint4 bs = *reinterpret_cast<const uint4 *>(sbs + b * 16 + h * 8);
    const float da = sd[b];
    const int sh = 16 * t;
    const int b1 = (int)(int16_t)(bs.x >> sh), b2 = (int)(int16_t)(bs.y >> sh);
    const int b3 = (int)(int16_t)(bs.z >> sh), b4 = (int)(int16_t)(bs.w >> sh);
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        int d1 = 0, d2 = 0, d3 = 0, d4 = 0;
#define FRK_Q6_STEP(c)                                                                                     \
    d1 = dot4((qla[st].c & 0x0f0f0f0fu) | ((qh[st].c << 4) & 0x30303030u), a0.c, d1);                       \
    d2 = dot4((qlb[st].c & 0x0f0f0f0fu) | ((qh[st].c << 2) & 0x30303030u), a1.c, d2);                       \
    d3 = dot4(((qla[st].c >> 4) & 0x0f0f0f0fu) | (qh[st].c & 0x30303030u), a2.c, d3);                       \
    d4 = dot4(((qlb[st].c >> 4) & 0x0f0f0f0fu) | ((qh[st].c >> 2) & 0x30303030u), a3.c, d4);
        FRK_Q6_STEP(x)
        FRK_Q6_STEP(y)
        FRK_Q6_STEP(z)
        FRK_Q6_STEP(w)
#undef FRK_Q6_STEP
        const uint32_t slo = t ? (scv[st].x >> 8) : scv[st].x, shi = t ? (scv[st].y >> 8) : scv[st].y;
        const int s1 = (int)(int8_t)(slo & 0xff), s2 = (int)(int8_t)((slo >> 16) & 0xff);
        const int s3 = (int)(int8_t)(shi & 0xff), s4 = (int)(int8_t)((shi >> 16) & 0xff);
        const int isum = s1 * (d1 - 32 * b1) + s2 * (d2 - 32 * b2) + s3 * (d3 - 32 * b3) + s4 * (d4 - 32 * b4);
        float acc = l < units ? (h2f(dbits[st]) * da) * (float)isum : 0.0f;
        acc = part_sum<LPR>(acc);
        if (l == 0 && rr[st] < rows_e) y[(size_t)job * rows_e + rr[st]] = acc;
    }
}

// ------------------------------------------------------------------ Q8_0 x f32
// dot_q8_0_f32 (crates/frink-quant/src/lib.rs:663-686) over the planar resident layout.
// Unit = 16 quants (half a block).
// A row to a wavefront, every load of the row in flight at once, the activation shared through LDS by the
// rows of the workgroup (rows of more than 16384 columns): a row of Q8_0 weights is a quarter of the bytes of
// the f32 activation it multiplies, so per-lane activation reads from L2 would be four times the weight
// traffic.  The activation goes global -> LDS with one
// global_load_lds per wavefront, laid out [piece k of a unit][unit] so that the lanes of a read are
// consecutive; LDS reads are inline assembly so that the compiler does not wait for the weight
// loads in front of them (it cannot tell the two apart from the global_load_lds).
typedef float v4f_t __attribute__((ext_vector_type(4)));
template <int U, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemv_q8_0_f32_shared_kernel(const uint8_t *__restrict__ W, Layout lay,
                                                                          int rows, int nb, const float *__restrict__ x,
                                                                          float *__restrict__ y) {
    extern __shared__ uint4 smem_direct[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = min((int)blockIdx.x * WAVES + wave, rows - 1);
    const bool store = (int)blockIdx.x * WAVES + wave < rows;
    const uint8_t *row = W + (size_t)r * lay.row_stride;
    const int units = nb * 2;
#pragma unroll
    for (int i = 0; i < (4 * U + WAVES - 1) / WAVES; i++) {  // the activation's 4 U KB at most: a KB a wavefront and round
        const int chunk = min(wave + i * WAVES, 4 * U - 1);  // (a wavefront past the end repeats the last chunk)
        const int slot = min(chunk * 64 + lane, 4 * units - 1);  // slots past the end repeat the last slot
        const int k = slot / units, u = slot - k * units;
        load_to_lds16(x + (size_t)(4 * u + k) * 4, reinterpret_cast<uint8_t *>(smem_direct) + chunk * 1024);
    }
    asm volatile("" ::: "memory");  // the weight loads below are issued after it: the wait counts on that
    uint4 qv[U];
    uint32_t dbits[U];
#pragma unroll
    for (int j = 0; j < U; j++) {
        const int u = min(lane + 64 * j, units - 1);
        qv[j] = stream_load16(row + (size_t)u * 16);
        dbits[j] = stream_load2(row + lay.off_a + (size_t)(u >> 1) * 2);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * U) : "memory");  // the activation piece has landed
    lds_barrier();
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)smem_direct;
#else
    const uint32_t base = 0;
#endif
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < U; j++) {
        const int u = min(lane + 64 * j, units - 1);
        v4f_t x0, x1, x2, x3;
        const uint32_t a0 = base + (uint32_t)u * 16, stride = (uint32_t)units * 16;
        asm volatile("ds_read_b128 %0, %1" : "=v"(x0) : "v"(a0));
        asm volatile("ds_read_b128 %0, %1" : "=v"(x1) : "v"(a0 + stride));
        asm volatile("ds_read_b128 %0, %1" : "=v"(x2) : "v"(a0 + 2 * stride));
        asm volatile("ds_read_b128 %0, %1" : "=v"(x3) : "v"(a0 + 3 * stride));
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));
        float s = 0.0f;
#define FRK_Q8_STEP(c, xx)                                         \
    s = fmaf((float)(int8_t)(qv[j].c & 0xff), xx.x, s);            \
    s = fmaf((float)(int8_t)((qv[j].c >> 8) & 0xff), xx.y, s);     \
    s = fmaf((float)(int8_t)((qv[j].c >> 16) & 0xff), xx.z, s);    \
    s = fmaf((float)(int8_t)(qv[j].c >> 24), xx.w, s);
        FRK_Q8_STEP(x, x0)
        FRK_Q8_STEP(y, x1)
        FRK_Q8_STEP(z, x2)
        FRK_Q8_STEP(w, x3)
#undef FRK_Q8_STEP
        const float term = s * h2f(dbits[j]);
        acc += (lane + 64 * j < units) ? term : 0.0f;
    }
    acc = part_sum<64>(acc);
    if (lane == 0 && store) y[r] = acc;
}

// The same product with the columns split between the wavefronts of a workgroup instead of the rows: wavefront w
// takes units 64w .. 64w+63 (1024 columns) of the workgroup's R rows, so a lane multiplies the same sixteen
// columns in every row and keeps its 64 bytes of the activation in registers, read straight from global memory
// -- no copy in LDS, hence no barrier between the requests and the arithmetic; the wavefronts' partial sums of a
// row meet in LDS at the end and are added in the order of the columns.
template <int R>
__global__ __launch_bounds__(1024) void gemv_q8_0_f32_cols_kernel(const uint8_t *__restrict__ W, Layout lay, int rows, int nb,
                                                                 const float *__restrict__ x, float *__restrict__ y) {
    extern __shared__ uint4 smem_direct[];
    float *parts = reinterpret_cast<float *>(smem_direct);  // [wavefront][row]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int units = nb * 2;
    const bool live = wave * 64 + lane < units;
    const int u = min(wave * 64 + lane, units - 1);  // (a lane past the end: the last unit again, not added)
    const int r0 = (int)blockIdx.x * R;
    const float4 *xp = reinterpret_cast<const float4 *>(x + (size_t)u * 16);
    const float4 x0 = xp[0], x1 = xp[1], x2 = xp[2], x3 = xp[3];
    uint4 qv[R];
    uint32_t dbits[R];
#pragma unroll
    for (int k = 0; k < R; k++) {
        const uint8_t *row = W + (size_t)min(r0 + k, rows - 1) * lay.row_stride;  // (a row past the end: the last again)
        qv[k] = stream_load16(row + (size_t)u * 16);
        dbits[k] = stream_load2(row + lay.off_a + (size_t)(u >> 1) * 2);
    }
#pragma unroll
    for (int k = 0; k < R; k++) {
        float s = 0.0f;
#define FRK_Q8_STEP(c, xx)                                         \
    s = fmaf((float)(int8_t)(qv[k].c & 0xff), xx.x, s);            \
    s = fmaf((float)(int8_t)((qv[k].c >> 8) & 0xff), xx.y, s);     \
    s = fmaf((float)(int8_t)((qv[k].c >> 16) & 0xff), xx.z, s);    \
    s = fmaf((float)(int8_t)(qv[k].c >> 24), xx.w, s);
        FRK_Q8_STEP(x, x0)
        FRK_Q8_STEP(y, x1)
        FRK_Q8_STEP(z, x2)
        FRK_Q8_STEP(w, x3)
#undef FRK_Q8_STEP
        const float v = part_sum<64>(live ? s * h2f(dbits[k]) : 0.0f);
        if (lane == 0) parts[wave * R + k] = v;
    }
    __syncthreads();
    if ((int)threadIdx.x < R && r0 + (int)threadIdx.x < rows) {
        float v = 0.0f;
        for (int w = 0; w < waves; w++) v += parts[w * R + threadIdx.x];
        y[r0 + threadIdx.x] = v;
    }
}

// Q4_0 x f32 the same way (dot_q4_0_f32, crates/frink-quant/src/lib.rs:4253-4276; blocks of 32 weights as 16 bytes of
// nibbles -- byte i: element i low, element i + 16 high -- in the quant plane and an f16 scale in the scale plane):
// wavefront w takes blocks 64w .. 64w+63 of the workgroup's R rows, a lane keeps its block's 32 activations and their
// sum in registers.  The sum is taken over the raw nibbles and eight times the block's sum of x comes off afterwards,
// as in gemv_q4_0_f32_kernel.
template <int R>
__global__ __launch_bounds__(1024) void gemv_q4_0_f32_cols_kernel(const uint8_t *__restrict__ W, Layout lay, int rows, int nb,
                                                                 const float *__restrict__ x, float *__restrict__ y) {
    extern __shared__ uint4 smem_direct[];
    float *parts = reinterpret_cast<float *>(smem_direct);  // [wavefront][row]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const bool live = wave * 64 + lane < nb;
    const int u = min(wave * 64 + lane, nb - 1);  // (a lane past the end: the last block again, not added)
    const int r0 = (int)blockIdx.x * R;
    const float4 *xp = reinterpret_cast<const float4 *>(x + (size_t)u * 32);
    float4 xv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) xv[i] = xp[i];
    uint4 qv[R];
    uint32_t dbits[R];
#pragma unroll
    for (int k = 0; k < R; k++) {
        const uint8_t *row = W + (size_t)min(r0 + k, rows - 1) * lay.row_stride;  // (a row past the end: the last again)
        qv[k] = stream_load16(row + (size_t)u * 16);
        dbits[k] = stream_load2(row + lay.off_a + (size_t)u * 2);
    }
    float xsum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) xsum += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
#pragma unroll
    for (int k = 0; k < R; k++) {
        float s = 0.0f;
#define FRK_Q4_STEP(c, kk)                                                       \
    {                                                                            \
        const float4 lo = xv[kk], hi = xv[4 + kk];                               \
        const uint32_t nl = qv[k].c & 0x0f0f0f0fu, nh = (qv[k].c >> 4) & 0x0f0f0f0fu; \
        s = fmaf((float)(nl & 0xff), lo.x, s);                                   \
        s = fmaf((float)(nh & 0xff), hi.x, s);                                   \
        s = fmaf((float)((nl >> 8) & 0xff), lo.y, s);                            \
        s = fmaf((float)((nh >> 8) & 0xff), hi.y, s);                            \
        s = fmaf((float)((nl >> 16) & 0xff), lo.z, s);                           \
        s = fmaf((float)((nh >> 16) & 0xff), hi.z, s);                           \
        s = fmaf((float)(nl >> 24), lo.w, s);                                    \
        s = fmaf((float)(nh >> 24), hi.w, s);                                    \
    }
        FRK_Q4_STEP(x, 0)
        FRK_Q4_STEP(y, 1)
        FRK_Q4_STEP(z, 2)
        FRK_Q4_STEP(w, 3)
#undef FRK_Q4_STEP
        const float v = part_sum<64>(live ? fmaf(-8.0f, xsum, s) * h2f(dbits[k]) : 0.0f);
        if (lane == 0) parts[wave * R + k] = v;
    }
    __syncthreads();
    if ((int)threadIdx.x < R && r0 + (int)threadIdx.x < rows) {
        float v = 0.0f;
        for (int w = 0; w < waves; w++) v += parts[w * R + threadIdx.x];
        y[r0 + threadIdx.x] = v;
    }
}

// ------------------------------------------------------------------ launchers

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

// rows of at most 64*4 units, and long enough that a wavefront per row is not mostly idle lanes
bool direct_gemv_fits(const frk_weights *w) {
    const size_t units = w->kind == FRK_KIND_Q6_K ? w->cols / QK_K * 4 : w->cols / Q8_0_ELEMS * 2;
    // (Q8_0: up to 16384 columns on the kernel whose wavefronts split the columns; up to 28672 -- 112 KB of activation
    // in LDS, one workgroup a CU -- where the rows are many enough for the kernel that gives a row to a wavefront)
    if (w->kind == FRK_KIND_Q8_0) return units > 32 && (units <= 1024 || (units <= 1792 && w->rows >= 1024));
    return w->kind == FRK_KIND_Q6_K && units > 32 && units <= 256;
}

int launch_gemv_q6_k_direct(const frk_weights *w, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    const int u = (nb * 4 + 63) / 64;
    const dim3 grid((unsigned)((w->rows + 3) / 4)), block(256);
#define FRK_GO(UU)                                                                                              \
    hipLaunchKernelGGL((gemv_q6_k_direct_kernel<UU, 1, false>), grid, block, 0, s, w->dev, w->layout, (int)w->rows, \
                       nb, (const float *)nullptr, a.q, a.d, a.bsums, y)
    if (u == 1) FRK_GO(1);
    else if (u == 2) FRK_GO(2);
    else if (u == 3) FRK_GO(3);
    else FRK_GO(4);
#undef FRK_GO
    FRK_LAUNCH_CHECK("gemv_q6_k_direct");
    return FRK_OK;
}

// Rows of 20 blocks and more, and rows too short for the kernel that gives a row to a wavefront: the column form.
bool q6_k_cols_form(const frk_weights *w) {
    const size_t nb = w->cols / QK_K;
    return w->kind == FRK_KIND_Q6_K && nb <= 64 && (nb >= 20 || nb <= 8);
}
static int compute_units_direct() {
    static const int n = [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
            v = 256;
        return v;
    }();
    return n;
}
// One launch: Q8_K quantization of x inside the kernel.  nb <= 64 (direct_gemv_fits).
int launch_gemv_q6_k_fused(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    if (q6_k_cols_form(w)) {  // the wavefronts split the columns, not the rows
        const int waves = (nb + 3) / 4;
        // Rows to a workgroup, 4 * U.  A CU's share of the launch costs about (its workgroups) x (4 * U rows + the
        // quantization of the activation, as much as five rows): the U with the smallest product, the larger of
        // equals.  (Measured at 1024 .. 32000 rows of 4 .. 56 blocks: within 4 % of the best U everywhere.)
        const int cus = compute_units_direct();
        int best_u = 1;
        size_t best = SIZE_MAX;
        for (int u = 1; u <= (waves == 1 ? 2 : 6); u++) {
            const size_t wgs = (w->rows + 4 * u - 1) / (4 * u);
            const size_t cost = (wgs + cus - 1) / cus * (4 * u + 5);
            if (cost <= best) best = cost, best_u = u;
        }
        const size_t lds = (size_t)waves * (COLS_WAVE_LDS + 4 * best_u * 4);
        const dim3 grid((unsigned)((w->rows + 4 * best_u - 1) / (4 * best_u))), block(64 * waves);
        const bool whole_lines = w->layout.row_stride % 128 == 0 && nb % 4 == 0;  // (every wavefront's four blocks of ql: 512 bytes)
#define FRK_GO_COLS(UU)                                                                                                              \
    if (whole_lines)                                                                                                                 \
        hipLaunchKernelGGL((gemv_q6_k_cols_kernel<UU, true>), grid, block, lds, s, w->dev, w->layout, (int)w->rows, nb, x, y);      \
    else                                                                                                                             \
        hipLaunchKernelGGL((gemv_q6_k_cols_kernel<UU, false>), grid, block, lds, s, w->dev, w->layout, (int)w->rows, nb, x, y)
        if (best_u == 1) FRK_GO_COLS(1);
        else if (best_u == 2) FRK_GO_COLS(2);
        else if (best_u == 3) FRK_GO_COLS(3);
        else if (best_u == 4) FRK_GO_COLS(4);
        else if (best_u == 5) FRK_GO_COLS(5);
        else FRK_GO_COLS(6);
#undef FRK_GO_COLS
        FRK_LAUNCH_CHECK("gemv_q6_k_cols");
        return FRK_OK;
    }
    const int u = (nb * 4 + 63) / 64;
    const dim3 grid((unsigned)((w->rows + 15) / 16)), block(1024);
    const size_t shmem = (size_t)nb * (256 + 32 + 4);
#define FRK_GO(UU, XX)                                                                                              \
    hipLaunchKernelGGL((gemv_q6_k_direct_kernel<UU, XX, true>), grid, block, shmem, s, w->dev, w->layout, (int)w->rows, \
                       nb, x, (const int8_t *)nullptr, (const float *)nullptr, (const int16_t *)nullptr, y)
    if (u == 1) FRK_GO(1, 1);       // nb <= 16
    else if (u == 2) FRK_GO(2, 2);  // nb <= 32
    else if (u == 3) FRK_GO(3, 3);  // nb <= 48
    else FRK_GO(4, 4);              // nb <= 64
#undef FRK_GO
    FRK_LAUNCH_CHECK("gemv_q6_k_fused");
    return FRK_OK;
}

// expert rows of at most 64 units (4096 columns), at most 16 blocks for the workgroup to quantize
bool q6_k_experts_gemv_fits(const frk_weights *w) {
    return w->kind == FRK_KIND_Q6_K && w->cols / QK_K * 4 <= 64;
}
// y[j][rows_e] = (rows of expert ids[j]) . (x + j * x_stride) for j < jobs
int launch_gemv_q6_k_experts(const frk_weights *w, int n_experts, size_t rows_e, const float *x, size_t x_stride,
                             const int32_t *ids, size_t jobs, float *y, hipStream_t s) {
    if (jobs > 65535) return set_error(FRK_ERR_SHAPE, "%zu expert jobs exceed the grid", jobs);
    const int nb = (int)(w->cols / QK_K), units = nb * 4;
    const size_t shmem = (size_t)nb * (256 + 32 + 4);
    constexpr int STEPS = 4;
#define FRK_GO(LPR)                                                                                                    \
    hipLaunchKernelGGL((gemv_q6_k_experts_kernel<LPR, STEPS>),                                                         \
                       dim3((unsigned)((rows_e + 4 * (64 / LPR) * STEPS - 1) / (4 * (64 / LPR) * STEPS)), (unsigned)jobs), \
                       dim3(256), shmem, s, w->dev, w->layout, (int)rows_e, nb, n_experts, ids, x, (int)x_stride, y)
    if (units <= 16) FRK_GO(16);
    else if (units <= 32) FRK_GO(32);
    else FRK_GO(64);
#undef FRK_GO
    FRK_LAUNCH_CHECK("gemv_q6_k_experts");
    return FRK_OK;
}

int launch_gemv_q8_0_f32_direct(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / Q8_0_ELEMS);
    const int u = (nb * 2 + 63) / 64;
    if (u <= 16) {  // rows of up to 16384 columns: the wavefronts of a workgroup split the columns
        // Eight rows to a workgroup; four where eight would leave a CU fewer than a dozen wavefronts.  (Measured
        // against the kernel below, which shares the activation through LDS: 4096x4096 5.6 against 5.7 us,
        // 14336x4096 13.2 / 14.0, 4096x8192 8.9 / 10.0, 4096x11008 11.3 / 12.9, 4096x14336 15.0 / 17.3; twelve and
        // sixteen rows to a workgroup are slower everywhere.)
        const bool four = (w->rows / 8) * (size_t)u < 12 * (size_t)compute_units_direct();
#define FRK_GO_COLS(RR)                                                                                                              \
    hipLaunchKernelGGL((gemv_q8_0_f32_cols_kernel<RR>), dim3((unsigned)((w->rows + RR - 1) / RR)), dim3(64 * u), (size_t)u * RR * 4, s, \
                       w->dev, w->layout, (int)w->rows, nb, x, y)
        if (four) FRK_GO_COLS(4);
        else FRK_GO_COLS(8);
#undef FRK_GO_COLS
        FRK_LAUNCH_CHECK("gemv_q8_0_f32_cols");
        return FRK_OK;
    }
    // longer rows (direct_gemv_fits: up to 28672 columns, at least 1024 rows): a row to a wavefront, the activation
    // through LDS, one workgroup to a CU
    constexpr int WAVES = 8;
    const dim3 grid((unsigned)((w->rows + WAVES - 1) / WAVES)), block(64 * WAVES);
// (more than 48 KB of LDS: the kernel is told once)
#define FRK_GO_BIG(UU)                                                                                                        \
    do {                                                                                                                      \
        static bool sized = false;                                                                                            \
        if (!sized) {                                                                                                         \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q8_0_f32_shared_kernel<UU, WAVES>),         \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 4096 * UU);                        \
            if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(gemv q8_0, LDS): %s", hipGetErrorString(e)); \
            sized = true;                                                                                                     \
        }                                                                                                                     \
        hipLaunchKernelGGL((gemv_q8_0_f32_shared_kernel<UU, WAVES>), grid, block, 4096 * UU, s, w->dev, w->layout, (int)w->rows, \
                           nb, x, y);                                                                                         \
    } while (0)
    if (u <= 20) FRK_GO_BIG(20);
    else if (u <= 24) FRK_GO_BIG(24);
    else FRK_GO_BIG(28);  // (2 * 28 loads in flight behind the activation's: vmcnt counts to 63)
#undef FRK_GO_BIG
    FRK_LAUNCH_CHECK("gemv_q8_0_f32_shared");
    return FRK_OK;
}

// Q4_0 rows of up to 32768 columns (1024 blocks: sixteen wavefronts).  Against gemv_q4_0_f32_kernel, which stages the
// activation in LDS behind a barrier (us): 4096x14336 12.3 / 18.5, 4096x11008 11.1 / 15.2, 4096x4096 5.3 / 5.9,
// 1024x4096 3.8 / 5.5, 32000x4096 20.6 / 22.7, 14336x4096 12.0 / 12.0.
bool q4_0_cols_form(const frk_weights *w) { return w->kind == FRK_KIND_Q4_0 && w->cols / Q8_0_ELEMS <= 1024; }
int launch_gemv_q4_0_f32_cols(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / Q8_0_ELEMS), waves = (nb + 63) / 64;
    const bool four = (w->rows / 8) * (size_t)waves < 12 * (size_t)compute_units_direct();
#define FRK_GO_COLS(RR)                                                                                                       \
    hipLaunchKernelGGL((gemv_q4_0_f32_cols_kernel<RR>), dim3((unsigned)((w->rows + RR - 1) / RR)), dim3(64 * waves),           \
                       (size_t)waves * RR * 4, s, w->dev, w->layout, (int)w->rows, nb, x, y)
    if (four) FRK_GO_COLS(4);
    else FRK_GO_COLS(8);
#undef FRK_GO_COLS
    FRK_LAUNCH_CHECK("gemv_q4_0_f32_cols");
    return FRK_OK;
}

}  // namespace frk
