// Decode GEMV over GGUF block formats: y[r] = sum_k W[r][k] * x[k], one activation vector.
//
// Bandwidth-bound: every weight byte is read once from HBM with 16-byte loads, the quantized
// activation lives in LDS, the integer products run on v_dot4_i32_i8 and a block's scale is
// applied once per 64 weights.  A wavefront (or an LPR-lane part of one, for short rows) owns a
// row; lanes walk the row in "units" of 64 weights.
#include "frk_device.hpp"

namespace frk {

// ------------------------------------------------------------------ Q4_K x Q8_K
// dot_q4_k_q8 (crates/frink-quant/src/lib.rs:822-869).  Unit = (block b, pair p): the 32 bytes
// qs[32p..32p+32] hold sub-block 2p in their low nibbles and 2p+1 in their high nibbles.
// Q5_K (dot_q5_k_q8, lib.rs:886-938) is the same walk: 176-byte blocks whose two words behind the
// header hold the codes' fifth bits -- byte l of them serves weight l of every sub-block, sub-block
// j through bit j -- and whose nibbles start at word 3.
template <int LPR, bool Q5>
__device__ __forceinline__ void gemv_q45_k(const uint8_t *__restrict__ W, size_t row_stride, int rows, int nb,
                                           const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                           const int16_t *__restrict__ absums, float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    int8_t *sq = reinterpret_cast<int8_t *>(smem);      // nb*256 activation quants
    int *sbs = reinterpret_cast<int *>(sq + nb * 256);  // nb*8 sums over 32
    float *sd = reinterpret_cast<float *>(sbs + nb * 8);
    for (int i = threadIdx.x; i < nb * 16; i += 256) smem[i] = reinterpret_cast<const uint4 *>(aq)[i];
    for (int i = threadIdx.x; i < nb * 8; i += 256) sbs[i] = (int)absums[2 * i] + (int)absums[2 * i + 1];
    for (int i = threadIdx.x; i < nb; i += 256) sd[i] = ad[i];
    __syncthreads();

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 4;
    const long n_waves = (long)gridDim.x * 4;
    for (long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * PARTS; r0 < rows; r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * row_stride;
            for (int u = l; u < units; u += LPR) {
                const int b = u >> 2, p = u & 3;
                const uint4 *blk = reinterpret_cast<const uint4 *>(row + (size_t)b * (Q5 ? Q5_K_BYTES : Q4_K_BYTES));
                const uint4 h = blk[0];
                const uint4 qa = blk[(Q5 ? 3 : 1) + 2 * p], qb = blk[(Q5 ? 4 : 2) + 2 * p];
                // Q5_K: the words of fifth bits that belong to qa (weights 0..15 of a sub-block) and qb
                const uint4 fa = Q5 ? blk[1] : make_uint4(0u, 0u, 0u, 0u), fb = Q5 ? blk[2] : make_uint4(0u, 0u, 0u, 0u);
                auto lo_codes = [&](uint32_t q, uint32_t f) {  // sub-block 2p
                    uint32_t c = q & 0x0f0f0f0fu;
                    if (Q5) c |= ((f >> (2 * p)) & 0x01010101u) << 4;
                    return c;
                };
                auto hi_codes = [&](uint32_t q, uint32_t f) {  // sub-block 2p + 1
                    uint32_t c = (q >> 4) & 0x0f0f0f0fu;
                    if (Q5) c |= ((f >> (2 * p + 1)) & 0x01010101u) << 4;
                    return c;
                };
                const uint4 *a = reinterpret_cast<const uint4 *>(sq + b * 256 + p * 64);
                const uint4 a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
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
                int is1 = 0, is2 = 0;
                is1 = dot4(lo_codes(qa.x, fa.x), a0.x, is1);
                is1 = dot4(lo_codes(qa.y, fa.y), a0.y, is1);
                is1 = dot4(lo_codes(qa.z, fa.z), a0.z, is1);
                is1 = dot4(lo_codes(qa.w, fa.w), a0.w, is1);
                is1 = dot4(lo_codes(qb.x, fb.x), a1.x, is1);
                is1 = dot4(lo_codes(qb.y, fb.y), a1.y, is1);
                is1 = dot4(lo_codes(qb.z, fb.z), a1.z, is1);
                is1 = dot4(lo_codes(qb.w, fb.w), a1.w, is1);
                is2 = dot4(hi_codes(qa.x, fa.x), a2.x, is2);
                is2 = dot4(hi_codes(qa.y, fa.y), a2.y, is2);
                is2 = dot4(hi_codes(qa.z, fa.z), a2.z, is2);
                is2 = dot4(hi_codes(qa.w, fa.w), a2.w, is2);
                is2 = dot4(hi_codes(qb.x, fb.x), a3.x, is2);
                is2 = dot4(hi_codes(qb.y, fb.y), a3.y, is2);
                is2 = dot4(hi_codes(qb.z, fb.z), a3.z, is2);
                is2 = dot4(hi_codes(qb.w, fb.w), a3.w, is2);
                const int s1 = sc1 * is1 + sc2 * is2;
                const int s2 = m1 * sbs[b * 8 + 2 * p] + m2 * sbs[b * 8 + 2 * p + 1];
                const float da = sd[b];
                const float d = h2f(h.x & 0xffffu), dmin = h2f(h.x >> 16);
                acc += (d * da) * (float)s1 - (dmin * da) * (float)s2;
            }
        }
        acc = part_sum<LPR>(acc);
        if (l == 0 && r < rows) y[r] = acc;
    }
}

template <int LPR>
__global__ __launch_bounds__(256) void gemv_q4_k_kernel(const uint8_t *__restrict__ W, size_t row_stride, int rows,
                                                        int nb, const int8_t *__restrict__ aq,
                                                        const float *__restrict__ ad,
                                                        const int16_t *__restrict__ absums, float *__restrict__ y) {
    gemv_q45_k<LPR, false>(W, row_stride, rows, nb, aq, ad, absums, y);
}
template <int LPR>
__global__ __launch_bounds__(256) void gemv_q5_k_kernel(const uint8_t *__restrict__ W, size_t row_stride, int rows,
                                                        int nb, const int8_t *__restrict__ aq,
                                                        const float *__restrict__ ad,
                                                        const int16_t *__restrict__ absums, float *__restrict__ y) {
    gemv_q45_k<LPR, true>(W, row_stride, rows, nb, aq, ad, absums, y);
}

// ------------------------------------------------------------------ Q6_K x Q8_K
// dot_q6_k_q8 (crates/frink-quant/src/lib.rs:1069-1110) over the planar resident layout.
// Unit = (block b, half h, 16-lane column t): ql[64h+16t..], ql[64h+32+16t..], qh[32h+16t..]
// hold four 16-weight groups with scales sc[8h+t+{0,2,4,6}].  The -32 offset is folded as
// -32 * (sum of the 16 activation quants), which Q8_K's bsums already hold.
template <int LPR>
__global__ __launch_bounds__(256) void gemv_q6_k_kernel(const uint8_t *__restrict__ W, Layout lay, int rows, int nb,
                                                        const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                                        const int16_t *__restrict__ absums, float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    int8_t *sq = reinterpret_cast<int8_t *>(smem);
    int *sbs = reinterpret_cast<int *>(sq + nb * 256);  // nb*16 sums over 16
    float *sd = reinterpret_cast<float *>(sbs + nb * 16);
    for (int i = threadIdx.x; i < nb * 16; i += 256) smem[i] = reinterpret_cast<const uint4 *>(aq)[i];
    for (int i = threadIdx.x; i < nb * 16; i += 256) sbs[i] = (int)absums[i];
    for (int i = threadIdx.x; i < nb; i += 256) sd[i] = ad[i];
    __syncthreads();

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 4;
    const long n_waves = (long)gridDim.x * 4;
    for (long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * PARTS; r0 < rows; r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * lay.row_stride;
            for (int u = l; u < units; u += LPR) {
                const int b = u >> 2, h = (u >> 1) & 1, t = u & 1;
                const uint4 qla = *reinterpret_cast<const uint4 *>(row + (size_t)b * 128 + h * 64 + t * 16);
                const uint4 qlb = *reinterpret_cast<const uint4 *>(row + (size_t)b * 128 + h * 64 + 32 + t * 16);
                const uint4 qh = *reinterpret_cast<const uint4 *>(row + lay.off_a + (size_t)b * 64 + h * 32 + t * 16);
                const uint2 scv = *reinterpret_cast<const uint2 *>(row + lay.off_b + (size_t)b * 16 + h * 8);
                const uint32_t dbits = *reinterpret_cast<const uint16_t *>(row + lay.off_c + (size_t)b * 2);
                const int8_t *abase = sq + b * 256 + h * 128 + t * 16;
                const uint4 a0 = *reinterpret_cast<const uint4 *>(abase);
                const uint4 a1 = *reinterpret_cast<const uint4 *>(abase + 32);
                const uint4 a2 = *reinterpret_cast<const uint4 *>(abase + 64);
                const uint4 a3 = *reinterpret_cast<const uint4 *>(abase + 96);
                const int g = b * 16 + h * 8 + t;
                int d1 = 0, d2 = 0, d3 = 0, d4 = 0;
#define FRK_Q6_STEP(c)                                                                                \
    d1 = dot4((qla.c & 0x0f0f0f0fu) | ((qh.c << 4) & 0x30303030u), a0.c, d1);                         \
    d2 = dot4((qlb.c & 0x0f0f0f0fu) | ((qh.c << 2) & 0x30303030u), a1.c, d2);                         \
    d3 = dot4(((qla.c >> 4) & 0x0f0f0f0fu) | (qh.c & 0x30303030u), a2.c, d3);                         \
    d4 = dot4(((qlb.c >> 4) & 0x0f0f0f0fu) | ((qh.c >> 2) & 0x30303030u), a3.c, d4);
                FRK_Q6_STEP(x)
                FRK_Q6_STEP(y)
                FRK_Q6_STEP(z)
                FRK_Q6_STEP(w)
#undef FRK_Q6_STEP
                const uint32_t slo = t ? (scv.x >> 8) : scv.x, shi = t ? (scv.y >> 8) : scv.y;
                const int s1 = (int)(int8_t)(slo & 0xff), s2 = (int)(int8_t)((slo >> 16) & 0xff);
                const int s3 = (int)(int8_t)(shi & 0xff), s4 = (int)(int8_t)((shi >> 16) & 0xff);
                const int isum = s1 * (d1 - 32 * sbs[g]) + s2 * (d2 - 32 * sbs[g + 2]) + s3 * (d3 - 32 * sbs[g + 4]) +
                                 s4 * (d4 - 32 * sbs[g + 6]);
                acc += (h2f(dbits) * sd[b]) * (float)isum;
            }
        }
        acc = part_sum<LPR>(acc);
        if (l == 0 && r < rows) y[r] = acc;
    }
}

// ------------------------------------------------------------------ Q8_0 x f32
// dot_q8_0_f32 (crates/frink-quant/src/lib.rs:663-686) over the planar resident layout.
// Unit = 16 quants (half a block); the f32 activation is staged in LDS, a unit's 16 floats every 20:
// a lane owns a unit, so neighbouring lanes' 16-byte reads would otherwise be 64 bytes apart and
// share banks four ways.
constexpr int Q8_X_STRIDE = 20;
template <int LPR>
__global__ __launch_bounds__(256) void gemv_q8_0_f32_kernel(const uint8_t *__restrict__ W, Layout lay, int rows,
                                                            int nb, const float *__restrict__ x,
                                                            float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    float *sx = reinterpret_cast<float *>(smem);
    for (int i = threadIdx.x; i < nb * 8; i += 256)
        *reinterpret_cast<uint4 *>(sx + (i >> 2) * Q8_X_STRIDE + (i & 3) * 4) = reinterpret_cast<const uint4 *>(x)[i];
    __syncthreads();

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 2;
    const long n_waves = (long)gridDim.x * 4;
    for (long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * PARTS; r0 < rows; r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * lay.row_stride;
            for (int u = l; u < units; u += LPR) {
                const uint4 qv = *reinterpret_cast<const uint4 *>(row + (size_t)u * 16);
                const float scale = h2f(*reinterpret_cast<const uint16_t *>(row + lay.off_a + (size_t)(u >> 1) * 2));
                const float4 *xv = reinterpret_cast<const float4 *>(sx + u * Q8_X_STRIDE);
                float s = 0.0f;
#define FRK_Q8_STEP(c, k)                                                  \
    {                                                                      \
        const float4 xx = xv[k];                                           \
        s = fmaf((float)(int8_t)(qv.c & 0xff), xx.x, s);                   \
        s = fmaf((float)(int8_t)((qv.c >> 8) & 0xff), xx.y, s);            \
        s = fmaf((float)(int8_t)((qv.c >> 16) & 0xff), xx.z, s);           \
        s = fmaf((float)(int8_t)(qv.c >> 24), xx.w, s);                    \
    }
                FRK_Q8_STEP(x, 0)
                FRK_Q8_STEP(y, 1)
                FRK_Q8_STEP(z, 2)
                FRK_Q8_STEP(w, 3)
#undef FRK_Q8_STEP
                acc = fmaf(s, scale, acc);
            }
        }
        acc = part_sum<LPR>(acc);
        if (l == 0 && r < rows) y[r] = acc;
    }
}

// ------------------------------------------------------------------ Q8_0 x Q8_0
// dot_q8_0_q8 (crates/frink-quant/src/lib.rs:711-733).  Unit = 16 quants.
template <int LPR>
__global__ __launch_bounds__(256) void gemv_q8_0_q8_kernel(const uint8_t *__restrict__ W, Layout lay, int rows,
                                                           int nb, const int8_t *__restrict__ aq,
                                                           const float *__restrict__ ad, float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    float *sd = reinterpret_cast<float *>(smem + nb * 2);
    for (int i = threadIdx.x; i < nb * 2; i += 256) smem[i] = reinterpret_cast<const uint4 *>(aq)[i];
    for (int i = threadIdx.x; i < nb; i += 256) sd[i] = ad[i];
    __syncthreads();

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 2;
    const long n_waves = (long)gridDim.x * 4;
    for (long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * PARTS; r0 < rows; r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * lay.row_stride;
            for (int u = l; u < units; u += LPR) {
                const uint4 qv = *reinterpret_cast<const uint4 *>(row + (size_t)u * 16);
                const float dw = h2f(*reinterpret_cast<const uint16_t *>(row + lay.off_a + (size_t)(u >> 1) * 2));
                const uint4 a = smem[u];
                int isum = dot4(qv.x, a.x, 0);
                isum = dot4(qv.y, a.y, isum);
                isum = dot4(qv.z, a.z, isum);
                isum = dot4(qv.w, a.w, isum);
                acc += (dw * sd[u >> 1]) * (float)isum;
            }
        }
        acc = part_sum<LPR>(acc);
        if (l == 0 && r < rows) y[r] = acc;
    }
}

// ------------------------------------------------------------------ Q4_0
// Unit = one 32-weight block: 16 bytes of nibbles (byte i: element i low, element i + 16 high) from the
// quant plane and the block's f16 scale from the scale plane.
// dot_q4_0_f32 (crates/frink-quant/src/lib.rs:4253-4276): the block's sum of (nibble - 8) * x, then
// times the scale.  Here the sum is taken over the raw nibbles -- a byte of a masked word converts to
// float in one instruction -- and eight times the block's sum of x, formed once per workgroup while
// the activation is staged, comes off afterwards: two and a half vector instructions per weight
// instead of five.
template <int LPR>
// A lane owns a block, so neighbouring lanes read x a block apart: the blocks of x sit XS floats apart
// in LDS, 36 (where that fits) instead of 32, which puts eight lanes' 16-byte reads in different banks.
__global__ __launch_bounds__(256) void gemv_q4_0_f32_kernel(const uint8_t *__restrict__ W, Layout lay, int rows,
                                                            int nb, int XS, const float *__restrict__ x,
                                                            float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    float *sx = reinterpret_cast<float *>(smem);
    float *sxs = sx + nb * XS;  // the blocks' sums of x
    for (int i = threadIdx.x; i < nb * 8; i += 256)
        *reinterpret_cast<uint4 *>(sx + (i >> 3) * XS + (i & 7) * 4) = reinterpret_cast<const uint4 *>(x)[i];
    __syncthreads();
    for (int b = threadIdx.x; b < nb; b += 256) {
        float t = 0.0f;
        for (int i = 0; i < 32; i++) t += sx[b * XS + (i + threadIdx.x) % 32];  // (rotated: no bank conflicts)
        sxs[b] = t;
    }
    __syncthreads();

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const long n_waves = (long)gridDim.x * 4;
    for (long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * PARTS; r0 < rows; r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * lay.row_stride;
            for (int u = l; u < nb; u += LPR) {
                const uint4 qv = *reinterpret_cast<const uint4 *>(row + (size_t)u * 16);
                const float scale = h2f(*reinterpret_cast<const uint16_t *>(row + lay.off_a + (size_t)u * 2));
                const float4 *xv = reinterpret_cast<const float4 *>(sx + u * XS);
                float s = 0.0f;
#define FRK_Q4_STEP(c, k)                                                        \
    {                                                                            \
        const float4 lo = xv[k], hi = xv[4 + k];                                 \
        const uint32_t nl = qv.c & 0x0f0f0f0fu, nh = (qv.c >> 4) & 0x0f0f0f0fu;  \
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
                acc = fmaf(fmaf(-8.0f, sxs[u], s), scale, acc);
            }
        }
        acc = part_sum<LPR>(acc);
        if (l == 0 && r < rows) y[r] = acc;
    }
}

// dot_q4_0_q8 (crates/frink-quant/src/lib.rs:772-796) against Q8_0 activation blocks: the exact integer
// sum of (nibble - 8) * qa -- as the dots of the raw nibbles minus eight times the sum of the
// activation quants -- then acc += (dw * da) * isum.
template <int LPR>
__global__ __launch_bounds__(256) void gemv_q4_0_q8_kernel(const uint8_t *__restrict__ W, Layout lay, int rows,
                                                           int nb, const int8_t *__restrict__ aq,
                                                           const float *__restrict__ ad, float *__restrict__ y) {
    extern __shared__ uint4 smem[];
    float *sd = reinterpret_cast<float *>(smem + nb * 2);
    for (int i = threadIdx.x; i < nb * 2; i += 256) smem[i] = reinterpret_cast<const uint4 *>(aq)[i];
    for (int i = threadIdx.x; i < nb; i += 256) sd[i] = ad[i];
    __syncthreads();

    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int part = lane / LPR, l = lane % LPR;
    const long n_waves = (long)gridDim.x * 4;
    for (long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * PARTS; r0 < rows; r0 += n_waves * PARTS) {
        const long r = r0 + part;
        float acc = 0.0f;
        if (r < rows) {
            const uint8_t *row = W + (size_t)r * lay.row_stride;
            for (int u = l; u < nb; u += LPR) {
                const uint4 qv = *reinterpret_cast<const uint4 *>(row + (size_t)u * 16);
                const float dw = h2f(*reinterpret_cast<const uint16_t *>(row + lay.off_a + (size_t)u * 2));
                const uint4 lo = smem[2 * u], hi = smem[2 * u + 1];  // activation quants 0..15 and 16..31
                int isum = 0, asum = 0;
#define FRK_Q4_STEP(c)                                              \
    isum = dot4(qv.c & 0x0f0f0f0fu, lo.c, isum);                    \
    isum = dot4((qv.c >> 4) & 0x0f0f0f0fu, hi.c, isum);             \
    asum = dot4(0x01010101u, lo.c, asum);                           \
    asum = dot4(0x01010101u, hi.c, asum);
                FRK_Q4_STEP(x)
                FRK_Q4_STEP(y)
                FRK_Q4_STEP(z)
                FRK_Q4_STEP(w)
#undef FRK_Q4_STEP
                acc += (dw * sd[u]) * (float)(isum - 8 * asum);
            }
        }
        acc = part_sum<LPR>(acc);
        if (l == 0 && r < rows) y[r] = acc;
    }
}

// ------------------------------------------------------------------ launchers

static int lanes_per_row(int units) { return units > 32 ? 64 : units > 16 ? 32 : 16; }

static unsigned gemv_grid(size_t rows, int lpr) {
    // enough 4-wave workgroups that each wave owns two rows; never more than 16 per CU's worth
    const size_t rows_per_wg = 4 * (size_t)(64 / lpr) * 2;
    size_t g = (rows + rows_per_wg - 1) / rows_per_wg;
    if (g > 4096) g = 4096;
    if (g < 1) g = 1;
    return (unsigned)g;
}

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

#define FRK_DISPATCH_LPR(lpr, KERNEL, grid, shmem, s, ...)                                             \
    do {                                                                                                \
        if ((shmem) > 64 * 1024)                                                                        \
            return set_error(FRK_ERR_SHAPE, "activation of this width needs %zu bytes of LDS (limit 65536)", \
                             (size_t)(shmem));                                                          \
        if (lpr == 64) hipLaunchKernelGGL(KERNEL<64>, dim3(grid), dim3(256), shmem, s, __VA_ARGS__);    \
        else if (lpr == 32) hipLaunchKernelGGL(KERNEL<32>, dim3(grid), dim3(256), shmem, s, __VA_ARGS__); \
        else hipLaunchKernelGGL(KERNEL<16>, dim3(grid), dim3(256), shmem, s, __VA_ARGS__);              \
    } while (0)

// The same for kernels that may ask for more than 64 KB of LDS (long rows of f32 activation): the limit
// is raised once per instantiation.
constexpr size_t GEMV_LDS_LIMIT = 160 * 1024;
#define FRK_DISPATCH_LPR_BIG(lpr, KERNEL, grid, shmem, s, ...)                                          \
    do {                                                                                                \
        if ((shmem) > GEMV_LDS_LIMIT)                                                                   \
            return set_error(FRK_ERR_SHAPE, "activation of this width needs %zu bytes of LDS (limit %zu)", \
                             (size_t)(shmem), GEMV_LDS_LIMIT);                                          \
        static bool sized = false;                                                                      \
        if (!sized) {                                                                                   \
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&KERNEL<64>),                \
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMV_LDS_LIMIT)); \
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&KERNEL<32>),                \
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMV_LDS_LIMIT)); \
            FRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&KERNEL<16>),                \
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMV_LDS_LIMIT)); \
            sized = true;                                                                               \
        }                                                                                               \
        if (lpr == 64) hipLaunchKernelGGL(KERNEL<64>, dim3(grid), dim3(256), shmem, s, __VA_ARGS__);    \
        else if (lpr == 32) hipLaunchKernelGGL(KERNEL<32>, dim3(grid), dim3(256), shmem, s, __VA_ARGS__); \
        else hipLaunchKernelGGL(KERNEL<16>, dim3(grid), dim3(256), shmem, s, __VA_ARGS__);              \
    } while (0)

int launch_gemv_q4_k(const frk_weights *w, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    const int lpr = lanes_per_row(nb * 4);
    const size_t shmem = (size_t)nb * (256 + 8 * 4 + 4);
    FRK_DISPATCH_LPR(lpr, gemv_q4_k_kernel, gemv_grid(w->rows, lpr), shmem, s, w->dev, w->layout.row_stride,
                     (int)w->rows, nb, a.q, a.d, a.bsums, y);
    FRK_LAUNCH_CHECK("gemv_q4_k");
    return FRK_OK;
}

int launch_gemv_q5_k(const frk_weights *w, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    const int lpr = lanes_per_row(nb * 4);
    const size_t shmem = (size_t)nb * (256 + 8 * 4 + 4);
    FRK_DISPATCH_LPR(lpr, gemv_q5_k_kernel, gemv_grid(w->rows, lpr), shmem, s, w->dev, w->layout.row_stride,
                     (int)w->rows, nb, a.q, a.d, a.bsums, y);
    FRK_LAUNCH_CHECK("gemv_q5_k");
    return FRK_OK;
}

int launch_gemv_q6_k(const frk_weights *w, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    const int lpr = lanes_per_row(nb * 4);
    const size_t shmem = (size_t)nb * (256 + 16 * 4 + 4);
    FRK_DISPATCH_LPR(lpr, gemv_q6_k_kernel, gemv_grid(w->rows, lpr), shmem, s, w->dev, w->layout, (int)w->rows, nb,
                     a.q, a.d, a.bsums, y);
    FRK_LAUNCH_CHECK("gemv_q6_k");
    return FRK_OK;
}

int launch_gemv_q8_0_f32(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / Q8_0_ELEMS);
    const int lpr = lanes_per_row(nb * 2);
    const size_t shmem = (size_t)nb * 2 * Q8_X_STRIDE * 4;
    FRK_DISPATCH_LPR_BIG(lpr, gemv_q8_0_f32_kernel, gemv_grid(w->rows, lpr), shmem, s, w->dev, w->layout, (int)w->rows,
                     nb, x, y);
    FRK_LAUNCH_CHECK("gemv_q8_0_f32");
    return FRK_OK;
}

int launch_gemv_q8_0_q8(const frk_weights *w, const int8_t *q, const float *d, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / Q8_0_ELEMS);
    const int lpr = lanes_per_row(nb * 2);
    const size_t shmem = (size_t)nb * (32 + 4);
    FRK_DISPATCH_LPR(lpr, gemv_q8_0_q8_kernel, gemv_grid(w->rows, lpr), shmem, s, w->dev, w->layout, (int)w->rows,
                     nb, q, d, y);
    FRK_LAUNCH_CHECK("gemv_q8_0_q8");
    return FRK_OK;
}

int launch_gemv_q4_0_f32(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / Q8_0_ELEMS);
    const int lpr = lanes_per_row(nb);
    const int xs = (size_t)nb * (36 + 1) * 4 <= GEMV_LDS_LIMIT ? 36 : 32;
    const size_t shmem = (size_t)nb * (xs + 1) * 4;
    FRK_DISPATCH_LPR_BIG(lpr, gemv_q4_0_f32_kernel, gemv_grid(w->rows, lpr), shmem, s, w->dev, w->layout, (int)w->rows,
                     nb, xs, x, y);
    FRK_LAUNCH_CHECK("gemv_q4_0_f32");
    return FRK_OK;
}

int launch_gemv_q4_0_q8(const frk_weights *w, const int8_t *q, const float *d, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / Q8_0_ELEMS);
    const int lpr = lanes_per_row(nb);
    const size_t shmem = (size_t)nb * (32 + 4);
    FRK_DISPATCH_LPR(lpr, gemv_q4_0_q8_kernel, gemv_grid(w->rows, lpr), shmem, s, w->dev, w->layout, (int)w->rows,
                     nb, q, d, y);
    FRK_LAUNCH_CHECK("gemv_q4_0_q8");
    return FRK_OK;
}

}  // namespace frk
