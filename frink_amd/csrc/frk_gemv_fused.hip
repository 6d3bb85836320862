// Decode GEMV for Q4_K weights, one launch per matrix.
//
// FUSED mode: the workgroup quantizes the f32 activation to Q8_K itself (bit-exact with
// quantize_activations_q8_k) while its weight loads are already in flight, so a decode step is a
// single kernel.  PREQ modes take an activation quantized earlier (shared by gate/up or q/k/v).
//
// Shape of the kernel: every wavefront issues the 16-byte loads of all the rows it handles in a
// round before doing anything else; the activation's own loads go out first (a wavefront's loads
// return in order); the workgroup barrier in front of the arithmetic waits for LDS only, never
// for the weight loads.  A lane multiplies the same columns in every row, so its slice of the
// quantized activation is read once into registers.
#include "frk_device.hpp"

namespace frk {

enum { MODE_FUSED = 0, MODE_PREQ_LDS = 1, MODE_PREQ_DIRECT = 2 };

// Loads of the activation, issued before the weight loads, and their later deposit in LDS.
// LDS layout: sq[nb*256] i8 | sbs[nb*16] i16 | sd[nb] f32.  XB = ceil(nb / wavefronts).
template <int MODE, int XB>
struct ActStage {
    float4 xv[MODE == MODE_FUSED ? XB : 1];
    uint4 qv[MODE == MODE_PREQ_LDS ? XB : 1];
    uint32_t bv;  // two bsums
    float dv;

    __device__ __forceinline__ void load(int nb, const float *__restrict__ x, const int8_t *__restrict__ aq,
                                         const float *__restrict__ ad, const int16_t *__restrict__ absums) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
        if (MODE == MODE_PREQ_LDS) {
            // nb*16 words of quants over blockDim threads: XB >= nb*16 / blockDim
#pragma unroll
            for (int i = 0; i < XB; i++) {
                const int idx = min((int)threadIdx.x + i * (int)blockDim.x, nb * 16 - 1);
                qv[i] = reinterpret_cast<const uint4 *>(aq)[idx];
            }
            bv = reinterpret_cast<const uint32_t *>(absums)[min((int)threadIdx.x, nb * 8 - 1)];
            dv = ad[min((int)threadIdx.x, nb - 1)];
        } else if (MODE == MODE_FUSED) {
#pragma unroll
            for (int i = 0; i < XB; i++) {
                const int b = min(wave + i * nwaves, nb - 1);
                xv[i] = reinterpret_cast<const float4 *>(x + (size_t)b * QK_K)[lane];
            }
        }
    }

    __device__ __forceinline__ void store(int nb, int8_t *sq, int16_t *sbs, float *sd, const int16_t *__restrict__ absums) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
        if (MODE == MODE_PREQ_LDS) {
#pragma unroll
            for (int i = 0; i < XB; i++) {
                const int idx = (int)threadIdx.x + i * (int)blockDim.x;
                if (idx < nb * 16) reinterpret_cast<uint4 *>(sq)[idx] = qv[i];
            }
            if ((int)threadIdx.x < nb * 8) reinterpret_cast<uint32_t *>(sbs)[threadIdx.x] = bv;
            // (a workgroup of fewer threads than the row has pairs of sums -- few rows of many blocks -- fetches
            // the rest here)
            for (int i = (int)threadIdx.x + (int)blockDim.x; i < nb * 8; i += (int)blockDim.x)
                reinterpret_cast<uint32_t *>(sbs)[i] = reinterpret_cast<const uint32_t *>(absums)[i];
            if ((int)threadIdx.x < nb) sd[threadIdx.x] = dv;
        } else if (MODE == MODE_FUSED) {
#pragma unroll
            for (int i = 0; i < XB; i++) {
                const int b = wave + i * nwaves;
                float d;
                int bs;
                const uint32_t packed = quantize_q8_k_lane(xv[i], d, bs);
                if (b < nb) {  // uniform across the wavefront
                    reinterpret_cast<uint32_t *>(sq + b * QK_K)[lane] = packed;
                    if ((lane & 3) == 0) sbs[b * 16 + (lane >> 2)] = (int16_t)bs;
                    if (lane == 0) sd[b] = d;
                }
            }
        }
    }
};

// A lane owns "half blocks": unit u = 2*b + q covers pairs p = q and p = q + 2 of block b, that is
// qs[32q..32q+32] and qs[64+32q..64+32q+32] (sub-blocks 2q, 2q+1, 2q+4, 2q+5; 128 weights) plus the
// block's 16-byte header, all of which the two pairs need between them: p < 2 reads its 6-bit
// scales from the plain layout, p >= 2 from the split one (q4_k_scale_min,
// crates/frink-quant/src/lib.rs:321-330).
struct Q4Unit {
    uint4 a[8];  // 128 activation quants: pair q -> a[0..3], pair q+2 -> a[4..7]
    int bs[4];   // activation sums over sub-blocks 2q, 2q+1, 2q+4, 2q+5
    float da;    // Q8_K block scale (0 for a lane past the end of the row)
    int sh;      // 16*q: where this unit's two scale bytes sit in the decoded words
};

// dot_q4_k_q8 (crates/frink-quant/src/lib.rs:822-869) for one unit of one row.
__device__ __forceinline__ float q4_k_unit_dot(const uint4 h, const uint4 w0, const uint4 w1, const uint4 w2,
                                               const uint4 w3, const Q4Unit &U) {
    const uint32_t hy = h.y >> U.sh, hz = h.z >> U.sh, hw = h.w >> U.sh;  // bytes 0,1 are ours now
    const uint32_t sc_lo = hy & 0x3f3fu, m_lo = hz & 0x3f3fu;
    const uint32_t sc_hi = (hw & 0x0f0fu) | (((hy >> 6) & 0x0303u) << 4);
    const uint32_t m_hi = ((hw >> 4) & 0x0f0fu) | (((hz >> 6) & 0x0303u) << 4);
    int i0 = 0, i1 = 0, i2 = 0, i3 = 0;
#define FRK_LO(ACC, WW, AV)                      \
    ACC = dot4(WW.x & 0x0f0f0f0fu, AV.x, ACC);   \
    ACC = dot4(WW.y & 0x0f0f0f0fu, AV.y, ACC);   \
    ACC = dot4(WW.z & 0x0f0f0f0fu, AV.z, ACC);   \
    ACC = dot4(WW.w & 0x0f0f0f0fu, AV.w, ACC);
#define FRK_HI(ACC, WW, AV)                             \
    ACC = dot4((WW.x >> 4) & 0x0f0f0f0fu, AV.x, ACC);   \
    ACC = dot4((WW.y >> 4) & 0x0f0f0f0fu, AV.y, ACC);   \
    ACC = dot4((WW.z >> 4) & 0x0f0f0f0fu, AV.z, ACC);   \
    ACC = dot4((WW.w >> 4) & 0x0f0f0f0fu, AV.w, ACC);
    FRK_LO(i0, w0, U.a[0])
    FRK_LO(i0, w1, U.a[1])
    FRK_HI(i1, w0, U.a[2])
    FRK_HI(i1, w1, U.a[3])
    FRK_LO(i2, w2, U.a[4])
    FRK_LO(i2, w3, U.a[5])
    FRK_HI(i3, w2, U.a[6])
    FRK_HI(i3, w3, U.a[7])
#undef FRK_LO
#undef FRK_HI
    // every factor fits 24 bits: scales and mins < 64, |isum| <= 32*15*127, |bsum| <= 32*127
    int s1 = __mul24((int)(sc_lo & 0xff), i0);
    s1 += __mul24((int)(sc_lo >> 8), i1);
    s1 += __mul24((int)(sc_hi & 0xff), i2);
    s1 += __mul24((int)(sc_hi >> 8), i3);
    int s2 = __mul24((int)(m_lo & 0xff), U.bs[0]);
    s2 += __mul24((int)(m_lo >> 8), U.bs[1]);
    s2 += __mul24((int)(m_hi & 0xff), U.bs[2]);
    s2 += __mul24((int)(m_hi >> 8), U.bs[3]);
    const float d = h2f(h.x & 0xffffu), dmin = h2f(h.x >> 16);
    return (d * U.da) * (float)s1 - (dmin * U.da) * (float)s2;
}

// dot_q5_k_q8 (crates/frink-quant/src/lib.rs:886-938) for one unit of one row: the same with every weight's fifth
// bit put over its nibble (fa, fb: the block's 32 bytes of fifth bits, byte l holding weight l of every sub-block,
// sub-block j in bit j; the unit's sub-blocks are 2q, 2q+1, 2q+4 and 2q+5).
__device__ __forceinline__ float q5_k_unit_dot(const uint4 h, const uint4 fa, const uint4 fb, const uint4 w0, const uint4 w1,
                                               const uint4 w2, const uint4 w3, const Q4Unit &U, int q) {
    const uint32_t hy = h.y >> U.sh, hz = h.z >> U.sh, hw = h.w >> U.sh;  // bytes 0,1 are ours now
    const uint32_t sc_lo = hy & 0x3f3fu, m_lo = hz & 0x3f3fu;
    const uint32_t sc_hi = (hw & 0x0f0fu) | (((hy >> 6) & 0x0303u) << 4);
    const uint32_t m_hi = ((hw >> 4) & 0x0f0fu) | (((hz >> 6) & 0x0303u) << 4);
    auto code = [](uint32_t nib, uint32_t fifth, int j) { return (((fifth >> j) & 0x01010101u) << 4) | (nib & 0x0f0f0f0fu); };
    int i0 = 0, i1 = 0, i2 = 0, i3 = 0;
#define FRK_Q5(ACC, WW, FF, AV, SH, J)                       \
    ACC = dot4(code(WW.x >> SH, FF.x, J), AV.x, ACC);        \
    ACC = dot4(code(WW.y >> SH, FF.y, J), AV.y, ACC);        \
    ACC = dot4(code(WW.z >> SH, FF.z, J), AV.z, ACC);        \
    ACC = dot4(code(WW.w >> SH, FF.w, J), AV.w, ACC);
    const int j = 2 * q;
    FRK_Q5(i0, w0, fa, U.a[0], 0, j)
    FRK_Q5(i0, w1, fb, U.a[1], 0, j)
    FRK_Q5(i1, w0, fa, U.a[2], 4, j + 1)
    FRK_Q5(i1, w1, fb, U.a[3], 4, j + 1)
    FRK_Q5(i2, w2, fa, U.a[4], 0, j + 4)
    FRK_Q5(i2, w3, fb, U.a[5], 0, j + 4)
    FRK_Q5(i3, w2, fa, U.a[6], 4, j + 5)
    FRK_Q5(i3, w3, fb, U.a[7], 4, j + 5)
#undef FRK_Q5
    int s1 = __mul24((int)(sc_lo & 0xff), i0);
    s1 += __mul24((int)(sc_lo >> 8), i1);
    s1 += __mul24((int)(sc_hi & 0xff), i2);
    s1 += __mul24((int)(sc_hi >> 8), i3);
    int s2 = __mul24((int)(m_lo & 0xff), U.bs[0]);
    s2 += __mul24((int)(m_lo >> 8), U.bs[1]);
    s2 += __mul24((int)(m_hi & 0xff), U.bs[2]);
    s2 += __mul24((int)(m_hi >> 8), U.bs[3]);
    const float d = h2f(h.x & 0xffffu), dmin = h2f(h.x >> 16);
    return (d * U.da) * (float)s1 - (dmin * U.da) * (float)s2;
}

// LPR lanes share a row (a wavefront works on 64/LPR rows at once), a lane owns units
// l, l+LPR, ... (J of them) and keeps RPW rounds of rows in flight.
// GLU: two matrices of one shape (gate = W, up = W2) in one launch; row r of both is computed by the
// same lanes and y[r] = silu(W[r] . x) * (W2[r] . x) (frink_core::matmul::swiglu,
// crates/frink-core/src/matmul.rs:634-650), each dot the very sum the plain kernel forms.
// MULTI: up to four matrices of one row length that multiply the same activation (q/k/v, or any
// group launch_matvec_multi gets, crates/frink-cuda/src/matvec_launch.rs:485-534) in one launch: the
// kernel walks the matrices' rows as one list, `rows` long; row v of the list belongs to the last
// matrix m with first[m] <= v.
struct MultiArgs {
    const uint8_t *W[4];
    float *y[4];
    int first[4];  // unused entries hold the total
    // INDEXED (below)
    const int32_t *ids;
    int n_experts;
    int x_stride;
};
// INDEXED: the expert projections of the per-token MoE path (run_expert / gate_up_projections,
// crates/frink-moe/src/lib.rs:1068-1165): W (and W2) are stacks of n_experts matrices of `rows` rows
// each; workgroup (_, job, sub) multiplies activation row `job` with expert ids[job*gridDim.z + sub]
// and writes output row job*gridDim.z + sub.  Gate/up: job = token, sub = the token's slot, all slots
// share the token's activation.  Down: job = (token, slot), gridDim.z = 1, every job its own.
// (the plain kernel takes an empty struct in their place: a hundred bytes more of kernel arguments
// cost the 14336x4096 GEMV 0.06 us)
template <bool ANY>
struct MultiArgsFor {
    using type = MultiArgs;
};
template <>
struct MultiArgsFor<false> {
    struct type {};
};
template <int LPR, int J, int RPW, int XB, int MODE, int MAXT, bool GLU = false, bool MULTI = false, bool INDEXED = false>
__global__ __launch_bounds__(MAXT) void gemv_q4_k_fused_kernel(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ W2, size_t row_stride, int rows, int rows_per_wg, int nb,
    const float *__restrict__ x, const int8_t *__restrict__ aq, const float *__restrict__ ad,
    const int16_t *__restrict__ absums, float *__restrict__ y, typename MultiArgsFor<MULTI || INDEXED>::type ma_in) {
    // (only the variants that have one look into it)
    MultiArgs ma = {};
    if constexpr (MULTI || INDEXED) ma = ma_in;
    extern __shared__ uint4 smem[];
    int8_t *sq = reinterpret_cast<int8_t *>(smem);
    int16_t *sbs = reinterpret_cast<int16_t *>(sq + nb * QK_K);
    float *sd = reinterpret_cast<float *>(sbs + nb * 16);

    if (INDEXED) {
        const int out_row = blockIdx.y * gridDim.z + blockIdx.z;
        const int e = min(max(ma.ids[out_row], 0), ma.n_experts - 1);
        W += (size_t)e * rows * row_stride;
        if (GLU) W2 += (size_t)e * rows * row_stride;
        x += (size_t)blockIdx.y * ma.x_stride;
        y += (size_t)out_row * rows;
    }
    constexpr int PARTS = 64 / LPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int part = lane / LPR, l = lane % LPR;
    const int units = nb * 2;
    const int row_begin = blockIdx.x * rows_per_wg;
    const int row_end = min(rows, row_begin + rows_per_wg);
    const int slot = wave * PARTS + part, slots = nwaves * PARTS;

    int ub[J], uq[J];
    bool uok[J];
    size_t uoff[J];  // byte offset of the unit's block in a row
#pragma unroll
    for (int j = 0; j < J; j++) {
        const int u = l + j * LPR;
        uok[j] = u < units;
        const int uc = uok[j] ? u : units - 1;
        ub[j] = uc >> 1;
        uq[j] = uc & 1;
        uoff[j] = (size_t)ub[j] * Q4_K_BYTES;
    }

    // ---- the activation's loads go out first ----
    ActStage<MODE, XB> act;
    Q4Unit U[J];
    act.load(nb, x, aq, ad, absums);
    if (MODE == MODE_PREQ_DIRECT) {
#pragma unroll
        for (int j = 0; j < J; j++) {
            const uint4 *ap = reinterpret_cast<const uint4 *>(aq + ub[j] * QK_K + uq[j] * 64);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                U[j].a[i] = ap[i];
                U[j].a[4 + i] = ap[8 + i];
            }
            const uint2 b0 = *reinterpret_cast<const uint2 *>(absums + ub[j] * 16 + uq[j] * 4);
            const uint2 b1 = *reinterpret_cast<const uint2 *>(absums + ub[j] * 16 + 8 + uq[j] * 4);
            U[j].bs[0] = (int)(int16_t)(b0.x & 0xffff) + (int)(int16_t)(b0.x >> 16);
            U[j].bs[1] = (int)(int16_t)(b0.y & 0xffff) + (int)(int16_t)(b0.y >> 16);
            U[j].bs[2] = (int)(int16_t)(b1.x & 0xffff) + (int)(int16_t)(b1.x >> 16);
            U[j].bs[3] = (int)(int16_t)(b1.y & 0xffff) + (int)(int16_t)(b1.y >> 16);
            U[j].da = uok[j] ? ad[ub[j]] : 0.0f;
            U[j].sh = uq[j] * 16;
        }
    }

    // ---- then all the weight loads of the first round ----
    uint4 wh[RPW][J], w0[RPW][J], w1[RPW][J], w2[RPW][J], w3[RPW][J];
    constexpr int RPW2 = GLU ? RPW : 1, J2 = GLU ? J : 1;
    uint4 vh[RPW2][J2], v0[RPW2][J2], v1[RPW2][J2], v2[RPW2][J2], v3[RPW2][J2];  // the second matrix's rows
    auto issue = [&](int rbase) {
#pragma unroll
        for (int k = 0; k < RPW; k++) {
            const int r = min(rbase + slot + k * slots, rows - 1);
            const uint8_t *row = W + (size_t)r * row_stride;
            if (MULTI) {
                const uint8_t *base = ma.W[0];
                int first = 0;
                if (r >= ma.first[1]) base = ma.W[1], first = ma.first[1];
                if (r >= ma.first[2]) base = ma.W[2], first = ma.first[2];
                if (r >= ma.first[3]) base = ma.W[3], first = ma.first[3];
                row = base + (size_t)(r - first) * row_stride;
            }
#pragma unroll
            for (int j = 0; j < J; j++) {
                const uint4 *blk = reinterpret_cast<const uint4 *>(row + uoff[j]);
                const int q2 = 2 * uq[j];
                wh[k][j] = blk[0];
                w0[k][j] = blk[1 + q2];
                w1[k][j] = blk[2 + q2];
                w2[k][j] = blk[5 + q2];
                w3[k][j] = blk[6 + q2];
            }
            if (GLU) {
                const uint8_t *row2 = W2 + (size_t)r * row_stride;
#pragma unroll
                for (int j = 0; j < J2; j++) {
                    const uint4 *blk = reinterpret_cast<const uint4 *>(row2 + uoff[j]);
                    const int q2 = 2 * uq[j];
                    vh[k][j] = blk[0];
                    v0[k][j] = blk[1 + q2];
                    v1[k][j] = blk[2 + q2];
                    v2[k][j] = blk[5 + q2];
                    v3[k][j] = blk[6 + q2];
                }
            }
        }
    };
    issue(row_begin);

    if (MODE != MODE_PREQ_DIRECT) {
        act.store(nb, sq, sbs, sd, absums);
        lds_barrier();
#pragma unroll
        for (int j = 0; j < J; j++) {
            const uint4 *ap = reinterpret_cast<const uint4 *>(sq + ub[j] * QK_K + uq[j] * 64);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                U[j].a[i] = ap[i];
                U[j].a[4 + i] = ap[8 + i];
            }
            const int16_t *bp = sbs + ub[j] * 16 + uq[j] * 4;
            U[j].bs[0] = (int)bp[0] + (int)bp[1];
            U[j].bs[1] = (int)bp[2] + (int)bp[3];
            U[j].bs[2] = (int)bp[8] + (int)bp[9];
            U[j].bs[3] = (int)bp[10] + (int)bp[11];
            U[j].da = uok[j] ? sd[ub[j]] : 0.0f;  // a lane past the end of the row contributes nothing
            U[j].sh = uq[j] * 16;
        }
    }

    for (int rbase = row_begin; rbase < row_end; rbase += slots * RPW) {
        if (rbase != row_begin) issue(rbase);
#pragma unroll
        for (int k = 0; k < RPW; k++) {
            const int r = rbase + slot + k * slots;
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < J; j++) acc += q4_k_unit_dot(wh[k][j], w0[k][j], w1[k][j], w2[k][j], w3[k][j], U[j]);
            acc = part_sum<LPR>(acc);
            if (GLU) {
                float up = 0.0f;
#pragma unroll
                for (int j = 0; j < J2; j++) up += q4_k_unit_dot(vh[k][j], v0[k][j], v1[k][j], v2[k][j], v3[k][j], U[j]);
                up = part_sum<LPR>(up);
                acc = silu_as_host(acc) * up;  // (a host's bits: a quantizer downstream sees the reference's input)
            }
            if (MULTI) {
                float *out = ma.y[0];
                int first = 0;
                if (r >= ma.first[1]) out = ma.y[1], first = ma.first[1];
                if (r >= ma.first[2]) out = ma.y[2], first = ma.first[2];
                if (r >= ma.first[3]) out = ma.y[3], first = ma.first[3];
                if (l == 0 && r < row_end) out[r - first] = acc;
            } else if (l == 0 && r < row_end) {
                y[r] = acc;
            }
        }
    }
}

// ------------------------------------------------------------------ whole cache lines
// The same product for rows whose block count divides 64 (row lengths 2048 .. 16384 in powers of two),
// read the way a plain copy reads memory.  The kernel above gives every lane its own half block, so
// one load instruction touches some three dozen cache lines and the five loads of a block revisit
// them: its 33 MB cost the CU's L1 six times the line look-ups of a linear read.  Here a wavefront
// owns 64 consecutive blocks (9216 contiguous bytes = 64/NB whole rows, rows being stored back to
// back) and moves them into LDS with nine global_load_lds of 1 KB -- eight full lines per
// instruction, nothing staged in registers.  From there lane l reads block l of the span (nine
// 16-byte reads 144 bytes apart: conflict-free) and multiplies the whole block: dot_q4_k_q8's
// integers and its per-block float expression (crates/frink-quant/src/lib.rs:822-869), the blocks
// of a row then added by its NB lanes with DPP.  The activation's blocks sit 272 bytes apart in LDS,
// so that the lanes of a wavefront, which read NB different blocks at once, hit different banks.
// Q5: the same for Q5_K blocks (176 bytes: Q4_K's header, 32 bytes of fifth bits -- byte l holds weight l of
// every sub-block, sub-block j in bit j --, the nibbles; dot_q5_k_q8, crates/frink-quant/src/lib.rs:886-938):
// a span is 11 KB, and a weight's fifth bit is put over its nibble on the way into v_dot4.
constexpr int LINES_ACT_STRIDE = QK_K + 16;
// One block of a row against the matching block of the activation, both in LDS: dot_q4_k_q8's (Q5: dot_q5_k_q8's)
// integers and per-block float expression.  blk: the block's 16-byte words; ap: the activation block's quants;
// bs32: its eight 32-wide sums; da: its scale.
template <bool Q5>
__device__ __forceinline__ float lines_block_dot(const uint4 *blk, const uint4 *ap, const int *bs32, float da) {
    const uint4 hd = blk[0];
    const uint4 fa = Q5 ? blk[1] : make_uint4(0u, 0u, 0u, 0u), fb = Q5 ? blk[2] : make_uint4(0u, 0u, 0u, 0u);  // fifth bits
    constexpr int QS = Q5 ? 3 : 1;  // where the nibbles start, in 16-byte words
    // a word of nibbles (shifted down by 4 for the high ones) under the fifth bits of sub-block j
    auto code = [&](uint32_t nib, uint32_t fifth, int j) {
        const uint32_t q4 = nib & 0x0f0f0f0fu;
        return Q5 ? (((fifth >> j) & 0x01010101u) << 4) | q4 : q4;
    };
    const uint32_t sc_lo = hd.y & 0x3f3f3f3fu, m_lo = hd.z & 0x3f3f3f3fu;
    const uint32_t sc_hi = (hd.w & 0x0f0f0f0fu) | (((hd.y >> 6) & 0x03030303u) << 4);
    const uint32_t m_hi = ((hd.w >> 4) & 0x0f0f0f0fu) | (((hd.z >> 6) & 0x03030303u) << 4);
    int s1 = 0;
#pragma unroll
    for (int p = 0; p < 4; p++) {  // the 32 bytes qs[32p..]: sub-block 2p in their low nibbles, 2p+1 in their high ones
        const uint4 qa = blk[QS + 2 * p], qb = blk[QS + 1 + 2 * p];
        const uint4 a0 = ap[4 * p], a1 = ap[4 * p + 1], a2 = ap[4 * p + 2], a3 = ap[4 * p + 3];
        int lo = 0, hi = 0;
        lo = dot4(code(qa.x, fa.x, 2 * p), a0.x, lo);
        lo = dot4(code(qa.y, fa.y, 2 * p), a0.y, lo);
        lo = dot4(code(qa.z, fa.z, 2 * p), a0.z, lo);
        lo = dot4(code(qa.w, fa.w, 2 * p), a0.w, lo);
        lo = dot4(code(qb.x, fb.x, 2 * p), a1.x, lo);
        lo = dot4(code(qb.y, fb.y, 2 * p), a1.y, lo);
        lo = dot4(code(qb.z, fb.z, 2 * p), a1.z, lo);
        lo = dot4(code(qb.w, fb.w, 2 * p), a1.w, lo);
        hi = dot4(code(qa.x >> 4, fa.x, 2 * p + 1), a2.x, hi);
        hi = dot4(code(qa.y >> 4, fa.y, 2 * p + 1), a2.y, hi);
        hi = dot4(code(qa.z >> 4, fa.z, 2 * p + 1), a2.z, hi);
        hi = dot4(code(qa.w >> 4, fa.w, 2 * p + 1), a2.w, hi);
        hi = dot4(code(qb.x >> 4, fb.x, 2 * p + 1), a3.x, hi);
        hi = dot4(code(qb.y >> 4, fb.y, 2 * p + 1), a3.y, hi);
        hi = dot4(code(qb.z >> 4, fb.z, 2 * p + 1), a3.z, hi);
        hi = dot4(code(qb.w >> 4, fb.w, 2 * p + 1), a3.w, hi);
        const uint32_t scw = (p < 2 ? sc_lo : sc_hi) >> ((p & 1) * 16);
        s1 += __mul24((int)(scw & 0xff), lo) + __mul24((int)((scw >> 8) & 0xff), hi);
    }
    const int4 bsa = *reinterpret_cast<const int4 *>(bs32), bsb = *reinterpret_cast<const int4 *>(bs32 + 4);
    int s2 = __mul24((int)(m_lo & 0xff), bsa.x) + __mul24((int)((m_lo >> 8) & 0xff), bsa.y) +
             __mul24((int)((m_lo >> 16) & 0xff), bsa.z) + __mul24((int)(m_lo >> 24), bsa.w);
    s2 += __mul24((int)(m_hi & 0xff), bsb.x) + __mul24((int)((m_hi >> 8) & 0xff), bsb.y) +
          __mul24((int)((m_hi >> 16) & 0xff), bsb.z) + __mul24((int)(m_hi >> 24), bsb.w);
    const float d = h2f(hd.x & 0xffffu), dmin = h2f(hd.x >> 16);
    return (d * da) * (float)s1 - (dmin * da) * (float)s2;
}

// MULTI: up to four matrices of this row length, each a whole number of spans, that multiply the same activation
// (q/k/v: launch_matvec_multi, crates/frink-cuda/src/matvec_launch.rs:485-534) as one list of rows, `rows` long;
// row v of the list belongs to the last matrix m with first[m] <= v.
template <int NB, int MODE, int WAVES, bool Q5 = false, int AHEAD = 0, bool MULTI = false>
__global__ __launch_bounds__(64 * WAVES) void gemv_q4_k_lines_kernel(const uint8_t *__restrict__ W, int rows,
                                                                    const float *__restrict__ x,
                                                                    const int8_t *__restrict__ aq,
                                                                    const float *__restrict__ ad,
                                                                    const int16_t *__restrict__ absums,
                                                                    float *__restrict__ y,
                                                                    typename MultiArgsFor<MULTI>::type ma) {
    constexpr int RPS = 64 / NB;  // rows of a wavefront's span
    constexpr int BB = Q5 ? Q5_K_BYTES : Q4_K_BYTES, SPAN = 64 * BB, PIECES = SPAN / 1024;  // 9 or 11 KB
    // AHEAD > 0: only that many kilobytes of the span are requested before the activation is quantized, the
    // rest behind the barrier.  For a launch whose workgroups all start at once (one round, the CUs full) the
    // memory pipeline is then not yet full of weight requests when the activation's loads and the barrier
    // want through: 8.0 against 8.55 us at 14336 x 4096 with four ahead (three 8.15, five 8.65).  A launch of
    // several rounds, or of few workgroups, loses by it (4096 x 4096 5.05 against 4.7 us): AHEAD = 0 there.
    constexpr int FIRST = AHEAD > 0 && MODE == MODE_FUSED ? AHEAD : PIECES;
    static_assert(64 % NB == 0 && NB >= 8, "a span of 64 blocks is a whole number of rows of at least 8 blocks");
    static_assert(NB * 16 <= 3 * 64 * WAVES, "three 16-byte words of quantized activation a thread at most");
    extern __shared__ uint4 smem[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
    int8_t *sq = reinterpret_cast<int8_t *>(lds);                          // NB blocks of quants, 272 bytes apart
    int *sbs = reinterpret_cast<int *>(lds + NB * LINES_ACT_STRIDE);       // NB x 8 sums over 32
    float *sd = reinterpret_cast<float *>(lds + NB * LINES_ACT_STRIDE + NB * 32);
    uint8_t *sw = lds + NB * LINES_ACT_STRIDE + NB * 32 + NB * 4;          // WAVES spans (16-byte aligned)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t span = (size_t)blockIdx.x * WAVES + wave;
    const size_t bytes = (size_t)rows * NB * BB;
    const bool has_rows = span * SPAN < bytes;  // (a wavefront past the matrix still quantizes its share)

    // ---- the activation's loads first (a wavefront's loads return in order), then the span ----
    typedef float xv_t __attribute__((ext_vector_type(4)));
    typedef uint32_t uq_t __attribute__((ext_vector_type(4)));
    xv_t xv[(NB + WAVES - 1) / WAVES];
    uq_t qv = {0u, 0u, 0u, 0u}, qv2 = {0u, 0u, 0u, 0u}, qv3 = {0u, 0u, 0u, 0u};
    uint32_t bv = 0;
    float dv = 0.0f;
    // (All of this kernel's global loads are issued from assembly and waited for by hand: the compiler
    // waits for every load in flight, the span's included, before it touches a register an older load
    // fills when loads that write LDS are among the younger ones.)
    if (MODE == MODE_FUSED) {
#pragma unroll
        for (int i = 0; i < (NB + WAVES - 1) / WAVES; i++) {
            const int b = min(wave + i * WAVES, NB - 1);
            const float4 *src = reinterpret_cast<const float4 *>(x + (size_t)b * QK_K) + lane;
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xv[i]) : "v"(src) : "memory");
        }
    } else {
        // quants: NB*16 words over 64*WAVES threads (at most three each); sums and scales.
        // Every lane loads (a clamped index where it has no word of its own) and the stores are masked.
        const int t = threadIdx.x;
        const uq_t *q_src = reinterpret_cast<const uq_t *>(aq);
        const uq_t *s0 = q_src + min(t, NB * 16 - 1), *s1 = q_src + min(t + 64 * WAVES, NB * 16 - 1);
        const uq_t *s1b = q_src + min(t + 128 * WAVES, NB * 16 - 1);
        const uint32_t *s2 = reinterpret_cast<const uint32_t *>(absums) + min(t, NB * 8 - 1);
        const float *s3 = ad + min(t, NB - 1);
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qv) : "v"(s0) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qv2) : "v"(s1) : "memory");
        if (NB * 16 > 128 * WAVES) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qv3) : "v"(s1b) : "memory");
        asm volatile("global_load_dword %0, %1, off" : "=v"(bv) : "v"(s2) : "memory");
        asm volatile("global_load_dword %0, %1, off" : "=v"(dv) : "v"(s3) : "memory");
    }
    // (a wavefront past the matrix fetches the last span and stores nothing)
    const size_t span_c = min(span, (bytes - 1) / SPAN);
    const uint8_t *span_src = W + span_c * SPAN;
    int list_first = 0;  // MULTI: the list's row at which this span's matrix begins
    if constexpr (MULTI) {
        const int row0 = (int)(span_c * RPS);
        const uint8_t *base = ma.W[0];
        y = ma.y[0];
        if (row0 >= ma.first[1]) base = ma.W[1], y = ma.y[1], list_first = ma.first[1];
        if (row0 >= ma.first[2]) base = ma.W[2], y = ma.y[2], list_first = ma.first[2];
        if (row0 >= ma.first[3]) base = ma.W[3], y = ma.y[3], list_first = ma.first[3];
        span_src = base + (size_t)(row0 - list_first) * NB * BB;
    }
    const uint32_t left = (uint32_t)min((size_t)SPAN, bytes - span_c * SPAN);  // (the last span may be short)
    const uint32_t slot = lds_address(sw) + (uint32_t)wave * SPAN;
#pragma unroll
    for (int c = 0; c < FIRST; c++) dma16_nt(slot + c * 1024, span_src, min((uint32_t)(c * 1024 + lane * 16), left - 16));

    // ---- the activation into LDS ----
    if (MODE == MODE_FUSED) {
        // the activation's loads are older than the span's nine (Q5_K: eleven; AHEAD: those requested so far)
        // (one wait that names them all, so that the blocks' quantizations can be interleaved)
        constexpr int XB = (NB + WAVES - 1) / WAVES;
        // (exactly the registers there are: an operand named twice would be copied in front of the wait)
        static_assert(XB >= 1 && XB <= 8, "up to eight blocks of the activation a wavefront");
        if constexpr (XB == 1) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(xv[0]) : "n"(FIRST));
        if constexpr (XB == 2) asm volatile("s_waitcnt vmcnt(%2)" : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]) : "n"(FIRST));
        if constexpr (XB == 3)
            asm volatile("s_waitcnt vmcnt(%3)" : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]) : "n"(FIRST));
        if constexpr (XB == 4)
            asm volatile("s_waitcnt vmcnt(%4)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0])
                         : "n"(FIRST));
        if constexpr (XB == 5)
            asm volatile("s_waitcnt vmcnt(%5)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0])
                         : "n"(FIRST));
        if constexpr (XB == 6)
            asm volatile("s_waitcnt vmcnt(%6)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0]), "+v"(xv[XB > 5 ? 5 : 0])
                         : "n"(FIRST));
        if constexpr (XB == 7)
            asm volatile("s_waitcnt vmcnt(%7)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0]), "+v"(xv[XB > 5 ? 5 : 0]), "+v"(xv[XB > 6 ? 6 : 0])
                         : "n"(FIRST));
        if constexpr (XB == 8)
            asm volatile("s_waitcnt vmcnt(%8)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0]), "+v"(xv[XB > 5 ? 5 : 0]), "+v"(xv[XB > 6 ? 6 : 0]), "+v"(xv[XB > 7 ? 7 : 0])
                         : "n"(FIRST));
#pragma unroll
        for (int i = 0; i < XB; i++) {
            const int b = wave + i * WAVES;
            float d;
            int bs;
            const uint32_t packed = quantize_q8_k_lane(make_float4(xv[i].x, xv[i].y, xv[i].z, xv[i].w), d, bs);
            // a lane's 16-wide sum is in all four lanes of its quad: pairs of them make the 32-wide sums
            const int bs32 = bs + __shfl_xor(bs, 4);
            if (b < NB) {  // uniform across the wavefront
                // (stored from assembly: a store the compiler sees makes it wait for the span's loads
                // first, which write LDS too -- and the quantization would no longer run in their shadow)
                lds_store32(lds_address(sq + b * LINES_ACT_STRIDE) + lane * 4, packed);
                if ((lane & 7) == 0) lds_store32(lds_address(sbs + b * 8) + (lane >> 3) * 4, (uint32_t)bs32);
                if (lane == 0) lds_store32(lds_address(sd + b), __float_as_uint(d));
            }
        }
    } else {
        asm volatile("s_waitcnt vmcnt(%5)" : "+v"(qv), "+v"(qv2), "+v"(qv3), "+v"(bv), "+v"(dv) : "n"(PIECES));  // (older than the span's)
        auto put = [&](int t, uq_t v) {  // word t of the quants: block t / 16, word t % 16 of it
            if (t < NB * 16) lds_store128(lds_address(sq + (t >> 4) * LINES_ACT_STRIDE + (t & 15) * 16), v);
        };
        put(threadIdx.x, qv);
        if (NB * 16 > 64 * WAVES) put(threadIdx.x + 64 * WAVES, qv2);
        if (NB * 16 > 128 * WAVES) put(threadIdx.x + 128 * WAVES, qv3);
        if ((int)threadIdx.x < NB * 8)
            lds_store32(lds_address(sbs + threadIdx.x), (uint32_t)((int)(int16_t)(bv & 0xffff) + (int)(int16_t)(bv >> 16)));
        if ((int)threadIdx.x < NB) lds_store32(lds_address(sd + threadIdx.x), __float_as_uint(dv));
    }
    // Only the activation is shared: the barrier comes before the wait for the span, so that a wavefront
    // starts multiplying when ITS blocks have landed, whatever the others' have done.
    lds_barrier();
#pragma unroll
    for (int c = FIRST; c < PIECES; c++) dma16_nt(slot + c * 1024, span_src, min((uint32_t)(c * 1024 + lane * 16), left - 16));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the span has landed (in this wavefront's own slot)
    if (!has_rows) return;

    // ---- lane l multiplies block l of the span ----
    const int b = lane % NB;
    float v = lines_block_dot<Q5>(reinterpret_cast<const uint4 *>(sw + wave * SPAN + lane * BB),
                                  reinterpret_cast<const uint4 *>(sq + b * LINES_ACT_STRIDE), sbs + b * 8, sd[b]);
    const size_t row = span * RPS + lane / NB;
    if (row >= (size_t)rows) v = 0.0f;  // (a short last span: this lane's block is not there)
    v = part_sum<NB>(v);
    if (lane % NB == 0 && row < (size_t)rows) y[row - list_first] = v;
}

// The same for rows of ANY block count up to 64 (11008, 14336, 5120 ... columns): a wavefront's span is the
// 64 / nb whole rows that fit 64 lanes -- contiguous bytes still, rows being stored back to back, though no
// longer a whole number of kilobytes: the last of the nine (eleven) requests is clamped to the span's end
// -- lanes past the span's blocks idle, and a row's blocks are added by a segmented shuffle in place of
// the DPP butterfly (lane b of a row takes lane b + step's sum while that lane is in the row).  The
// activation comes quantized (MODE_PREQ_LDS) or is quantized here, eight blocks a wavefront at most.
template <int MODE, int WAVES, bool Q5 = false>
__global__ __launch_bounds__(64 * WAVES) void gemv_q4_k_rows_kernel(const uint8_t *__restrict__ W, int rows, int nb,
                                                                   const float *__restrict__ x,
                                                                   const int8_t *__restrict__ aq,
                                                                   const float *__restrict__ ad,
                                                                   const int16_t *__restrict__ absums,
                                                                   float *__restrict__ y) {
    constexpr int BB = Q5 ? Q5_K_BYTES : Q4_K_BYTES, SLOT = 64 * BB, PIECES = SLOT / 1024;
    static_assert(WAVES >= 6 && (MODE != MODE_FUSED || WAVES >= 8), "64 blocks of activation: eight a wavefront, three words of quants a thread");
    extern __shared__ uint4 smem[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
    int8_t *sq = reinterpret_cast<int8_t *>(lds);                       // nb blocks of quants, 272 bytes apart
    int *sbs = reinterpret_cast<int *>(lds + nb * LINES_ACT_STRIDE);    // nb x 8 sums over 32
    float *sd = reinterpret_cast<float *>(lds + nb * LINES_ACT_STRIDE + nb * 32);
    uint8_t *sw = lds + ((nb * (LINES_ACT_STRIDE + 32 + 4) + 15) & ~15);  // WAVES slots of 64 blocks
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rps = 64 / nb;  // rows of a span
    const uint32_t span_bytes = (uint32_t)(rps * nb) * BB;
    const size_t span = (size_t)blockIdx.x * WAVES + wave;
    const size_t bytes = (size_t)rows * nb * BB;
    const bool has_rows = span * span_bytes < bytes;

    typedef float xv_t __attribute__((ext_vector_type(4)));
    typedef uint32_t uq_t __attribute__((ext_vector_type(4)));
    xv_t xv[8];
    uq_t qv = {0u, 0u, 0u, 0u}, qv2 = {0u, 0u, 0u, 0u}, qv3 = {0u, 0u, 0u, 0u};
    uint32_t bv = 0, bv2 = 0;
    float dv = 0.0f;
    if (MODE == MODE_FUSED) {
#pragma unroll
        for (int i = 0; i < 8; i++) {  // (a block past the row's end: the last one again, not used)
            const int b = min(wave + i * WAVES, nb - 1);
            const float4 *src = reinterpret_cast<const float4 *>(x + (size_t)b * QK_K) + lane;
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xv[i]) : "v"(src) : "memory");
        }
    } else {
        const int t = threadIdx.x;
        const uq_t *q_src = reinterpret_cast<const uq_t *>(aq);
        const uq_t *s0 = q_src + min(t, nb * 16 - 1), *s1 = q_src + min(t + 64 * WAVES, nb * 16 - 1);
        const uq_t *s1b = q_src + min(t + 128 * WAVES, nb * 16 - 1);
        // (nb * 8 <= 512 pairs of 16-wide sums over 64 * WAVES >= 384 threads: two a thread)
        const uint32_t *s2 = reinterpret_cast<const uint32_t *>(absums) + min(t, nb * 8 - 1);
        const uint32_t *s2b = reinterpret_cast<const uint32_t *>(absums) + min(t + 64 * WAVES, nb * 8 - 1);
        const float *s3 = ad + min(t, nb - 1);
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qv) : "v"(s0) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qv2) : "v"(s1) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qv3) : "v"(s1b) : "memory");
        asm volatile("global_load_dword %0, %1, off" : "=v"(bv) : "v"(s2) : "memory");
        asm volatile("global_load_dword %0, %1, off" : "=v"(bv2) : "v"(s2b) : "memory");
        asm volatile("global_load_dword %0, %1, off" : "=v"(dv) : "v"(s3) : "memory");
    }
    {
        const size_t span_c = min(span, (bytes - 1) / span_bytes);
        const uint8_t *src = W + span_c * span_bytes;
        const uint32_t left = (uint32_t)min((size_t)span_bytes, bytes - span_c * span_bytes);
        const uint32_t slot = lds_address(sw) + (uint32_t)wave * SLOT;
#pragma unroll
        for (int c = 0; c < PIECES; c++) dma16_nt(slot + c * 1024, src, min((uint32_t)(c * 1024 + lane * 16), left - 16));
    }
    if (MODE == MODE_FUSED) {
        asm volatile("s_waitcnt vmcnt(%8)"
                     : "+v"(xv[0]), "+v"(xv[1]), "+v"(xv[2]), "+v"(xv[3]), "+v"(xv[4]), "+v"(xv[5]), "+v"(xv[6]), "+v"(xv[7])
                     : "n"(PIECES));
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int b = wave + i * WAVES;
            if (b < nb) {  // uniform across the wavefront
                float d;
                int bs;
                const uint32_t packed = quantize_q8_k_lane(make_float4(xv[i].x, xv[i].y, xv[i].z, xv[i].w), d, bs);
                const int bs32 = bs + __shfl_xor(bs, 4);
                lds_store32(lds_address(sq + b * LINES_ACT_STRIDE) + lane * 4, packed);
                if ((lane & 7) == 0) lds_store32(lds_address(sbs + b * 8) + (lane >> 3) * 4, (uint32_t)bs32);
                if (lane == 0) lds_store32(lds_address(sd + b), __float_as_uint(d));
            }
        }
    } else {
        asm volatile("s_waitcnt vmcnt(%6)" : "+v"(qv), "+v"(qv2), "+v"(qv3), "+v"(bv), "+v"(bv2), "+v"(dv) : "n"(PIECES));
        auto put = [&](int t, uq_t v) {
            if (t < nb * 16) lds_store128(lds_address(sq + (t >> 4) * LINES_ACT_STRIDE + (t & 15) * 16), v);
        };
        put(threadIdx.x, qv);
        put(threadIdx.x + 64 * WAVES, qv2);
        put(threadIdx.x + 128 * WAVES, qv3);
        auto put_sum = [&](int t, uint32_t pair) {  // two 16-wide sums make a 32-wide one
            if (t < nb * 8) lds_store32(lds_address(sbs + t), (uint32_t)((int)(int16_t)(pair & 0xffff) + (int)(int16_t)(pair >> 16)));
        };
        put_sum(threadIdx.x, bv);
        put_sum(threadIdx.x + 64 * WAVES, bv2);
        if ((int)threadIdx.x < nb) lds_store32(lds_address(sd + threadIdx.x), __float_as_uint(dv));
    }
    lds_barrier();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (!has_rows) return;

    const int r_in = lane / nb, b_in = lane - r_in * nb;  // this lane's row of the span and block of the row
    const bool live = r_in < rps;
    const int b = live ? b_in : 0;
    float v = lines_block_dot<Q5>(reinterpret_cast<const uint4 *>(sw + wave * SLOT + (live ? lane : 0) * BB),
                                  reinterpret_cast<const uint4 *>(sq + b * LINES_ACT_STRIDE), sbs + b * 8, sd[b]);
    const size_t row = span * rps + r_in;
    if (!live || row >= (size_t)rows) v = 0.0f;
    for (int step = 1; step < nb; step <<= 1) {  // (uniform bound)
        const float o = __shfl_down(v, step);
        if (b_in + step < nb) v += o;
    }
    if (live && b_in == 0 && row < (size_t)rows) y[row] = v;
}

// One launch for long rows of any block count, with the columns split between the wavefronts of a workgroup:
// wavefront w takes blocks 4w .. 4w+3 of the workgroup's 8 * U rows, quantizes exactly those four blocks of the
// activation (through a corner of LDS that only it touches) and keeps its lanes' slices of them in registers for
// every row.  Nothing is shared before the sums, so no barrier stands between the requests and the arithmetic
// (a barrier there is reached only once the memory pipeline has taken every wavefront's requests); the
// wavefronts' partial sums of a row meet in LDS at the very end, added in the order of the columns.
// Round j of a wavefront covers rows 8j .. 8j+7 of the workgroup: lane = 8 * (row of the round) + unit, a unit
// being a half block as in gemv_q4_k_fused_kernel (the block's header and four of its eight 16-byte words).
constexpr int COLS_WAVE_LDS = 4 * (QK_K + 32 + 4);  // four blocks: quants, 16-wide sums, scale
template <int U, bool Q5 = false>
__global__ __launch_bounds__(1024) void gemv_q4_k_cols_kernel(const uint8_t *__restrict__ W, size_t row_stride, int rows, int nb,
                                                             const float *__restrict__ x, float *__restrict__ y) {
    typedef float xv_t __attribute__((ext_vector_type(4)));
    typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
    extern __shared__ uint4 smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), waves = blockDim.x >> 6;
    uint8_t *mine = reinterpret_cast<uint8_t *>(smem) + wave * COLS_WAVE_LDS;
    float *parts = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(smem) + waves * COLS_WAVE_LDS);
    const int b0 = wave * 4, r0 = (int)blockIdx.x * 8 * U;

    // the activation's loads first: a wavefront's loads return in issue order
    xv_t xv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {  // (a block past the row's end: the last one again, not used)
        const float *src = x + (size_t)min(b0 + i, nb - 1) * QK_K + lane * 4;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xv[i]) : "v"(src) : "memory");
    }
    const int ul = lane & 7, bl = ul >> 1, q = ul & 1;
    const bool live = b0 + bl < nb;
    const int b = min(b0 + bl, nb - 1);
    // (Q5: Q5_K blocks, Q4_K's with 32 bytes of fifth bits between the header and the nibbles -- seven loads a round)
    constexpr int BB = Q5 ? Q5_K_BYTES : Q4_K_BYTES, LOADS = Q5 ? 7 : 5;
    u4_t wh[U], w0[U], w1[U], w2[U], w3[U], fa[Q5 ? U : 1], fb[Q5 ? U : 1];
    auto request = [&](int j) {
        const int r = min(r0 + 8 * j + (lane >> 3), rows - 1);  // a row past the end: the last one again, not stored
        const uint8_t *blk = W + (size_t)r * row_stride + (size_t)b * BB;
        const uint8_t *qs = blk + (BB - 128) + 32 * q;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(wh[j]) : "v"(blk) : "memory");
        if constexpr (Q5) {
            asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(fa[j]) : "v"(blk) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off offset:32" : "=v"(fb[j]) : "v"(blk) : "memory");
        }
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(w0[j]) : "v"(qs) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(w1[j]) : "v"(qs) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off offset:64" : "=v"(w2[j]) : "v"(qs) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off offset:80" : "=v"(w3[j]) : "v"(qs) : "memory");
    };
    request(0);
    // (the other rounds are requested once the activation is here: behind every wavefront's later rounds a late
    // wavefront's activation came late)
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(xv[0]), "+v"(xv[1]), "+v"(xv[2]), "+v"(xv[3]) : "n"(LOADS));
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
    Q4Unit unit;
    {
        const uint4 *ap = reinterpret_cast<const uint4 *>(mine + bl * QK_K + q * 64);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            unit.a[i] = ap[i];
            unit.a[4 + i] = ap[8 + i];
        }
        const int16_t *bp = sbs + bl * 16 + q * 4;
        unit.bs[0] = (int)bp[0] + (int)bp[1];
        unit.bs[1] = (int)bp[2] + (int)bp[3];
        unit.bs[2] = (int)bp[8] + (int)bp[9];
        unit.bs[3] = (int)bp[10] + (int)bp[11];
        unit.da = live ? sd[bl] : 0.0f;  // a lane past the end of the row contributes nothing
        unit.sh = q * 16;
    }
    auto as4 = [](u4_t v) { return make_uint4(v.x, v.y, v.z, v.w); };
    float sums[U];
#define FRK_COLS_ROUND(j)                                                                                         \
    if constexpr (U > j) {                                                                                        \
        float term;                                                                                               \
        if constexpr (Q5) {                                                                                       \
            asm volatile("s_waitcnt vmcnt(%7)"                                                                    \
                         : "+v"(wh[j]), "+v"(fa[j]), "+v"(fb[j]), "+v"(w0[j]), "+v"(w1[j]), "+v"(w2[j]), "+v"(w3[j]) \
                         : "n"(LOADS * (U - 1 - j)));                                                             \
            term = q5_k_unit_dot(as4(wh[j]), as4(fa[j]), as4(fb[j]), as4(w0[j]), as4(w1[j]), as4(w2[j]), as4(w3[j]), unit, q); \
        } else {                                                                                                  \
            asm volatile("s_waitcnt vmcnt(%5)"                                                                    \
                         : "+v"(wh[j]), "+v"(w0[j]), "+v"(w1[j]), "+v"(w2[j]), "+v"(w3[j])                        \
                         : "n"(LOADS * (U - 1 - j)));                                                             \
            term = q4_k_unit_dot(as4(wh[j]), as4(w0[j]), as4(w1[j]), as4(w2[j]), as4(w3[j]), unit);               \
        }                                                                                                         \
        sums[j] = part_sum<8>(live ? term : 0.0f);                                                                \
    }
    FRK_COLS_ROUND(0)
    FRK_COLS_ROUND(1)
    FRK_COLS_ROUND(2)
#undef FRK_COLS_ROUND
    static_assert(U <= (Q5 ? 2 : 3), "three rounds at most (Q5_K: two): more do not fit the registers of sixteen wavefronts");
#pragma unroll
    for (int j = 0; j < U; j++)
        if (ul == 0) parts[wave * (8 * U) + 8 * j + (lane >> 3)] = sums[j];
    lds_barrier();
    // a row's partial sums, in the order of the columns
    if ((int)threadIdx.x < 8 * U && r0 + (int)threadIdx.x < rows) {
        float v = 0.0f;
        for (int w = 0; w < waves; w++) v += parts[w * (8 * U) + threadIdx.x];
        y[r0 + threadIdx.x] = v;
    }
}

// ------------------------------------------------------------------ launchers

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

static int g_cus = 0;
static int compute_units() {
    if (!g_cus) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            g_cus = n;
        else
            g_cus = 256;
    }
    return g_cus;
}

struct FusedGeom {
    int lpr, j, rpw, threads, grid, rows_per_wg;
};

// units = half blocks per row.  J units per lane: 1 up to 64 units (cols <= 8192), then 2, then 4.
// Measured on the 14336x4096 gate/up shape: FUSED runs best with two 512-thread workgroups per
// compute unit, each quantizing the activation once and walking its rows in rounds of one row per
// wavefront part; PREQ runs best with 256-thread workgroups that each take a single round.
static FusedGeom fused_geom(size_t rows, int units, bool fused) {
    FusedGeom g;
    g.lpr = units > 32 ? 64 : units > 16 ? 32 : 16;
    const int per_lane = (units + g.lpr - 1) / g.lpr;
    g.j = per_lane <= 1 ? 1 : per_lane <= 2 ? 2 : 4;
    g.rpw = 1;
    const int parts = 64 / g.lpr;
    g.threads = fused ? 512 : 256;
    const size_t slots = (size_t)(g.threads / 64) * parts;
    size_t grid = (rows + slots - 1) / slots;  // a single round of rows per workgroup ...
    if (fused) {
        const size_t two_per_cu = (size_t)compute_units() * 2;
        if (grid > two_per_cu) grid = two_per_cu;  // ... or several, so x is quantized 512 times at most
    }
    g.grid = (int)grid;
    g.rows_per_wg = (int)((rows + grid - 1) / grid);
    return g;
}

template <int MODE, bool GLU = false, bool MULTI = false, bool INDEXED = false>
static int launch_q4_k_fused(const frk_weights *w, const frk_weights *w2, const float *x, Q8KActs a, float *y,
                             hipStream_t s, size_t rows_total = 0, const MultiArgs *multi = nullptr, unsigned jobs = 1,
                             unsigned per_job = 1) {
    const int nb = (int)(w->cols / QK_K);
    const size_t rows = (MULTI || INDEXED) ? rows_total : w->rows;
    typename MultiArgsFor<MULTI || INDEXED>::type ma;
    if constexpr (MULTI || INDEXED) ma = *multi;
    FusedGeom g = fused_geom(rows, nb * 2, MODE == MODE_FUSED);
    const size_t shmem = MODE == MODE_PREQ_DIRECT ? 0 : (size_t)nb * (256 + 32 + 4);
    const int nwaves = g.threads / 64;
    const int xb = (nb + nwaves - 1) / nwaves;
#define FRK_GO2(LPR, J, RPW, XB, MAXT)                                                                            \
    hipLaunchKernelGGL((gemv_q4_k_fused_kernel<LPR, J, RPW, XB, MODE, MAXT, GLU, MULTI, INDEXED>),                \
                       dim3(g.grid, jobs, per_job), dim3(g.threads), shmem, s, w->dev, GLU ? w2->dev : nullptr,      \
                       w->layout.row_stride, (int)rows, g.rows_per_wg, nb, x, a.q, a.d, a.bsums, y, ma)
#define FRK_GO(LPR, J, RPW, MAXT)                                               \
    do {                                                                        \
        if (MODE == MODE_PREQ_DIRECT || xb <= 1) FRK_GO2(LPR, J, RPW, 1, MAXT); \
        else if (xb <= 2) FRK_GO2(LPR, J, RPW, 2, MAXT);                        \
        else if (xb <= 4) FRK_GO2(LPR, J, RPW, 4, MAXT);                        \
        else FRK_GO2(LPR, J, RPW, 8, MAXT);                                     \
    } while (0)
    if (g.lpr == 16) FRK_GO(16, 1, 1, 512);
    else if (g.lpr == 32) FRK_GO(32, 1, 1, 512);
    else if (g.j == 1) FRK_GO(64, 1, 1, 512);
    else if (g.j == 2) FRK_GO(64, 2, 1, 512);
    else FRK_GO(64, 4, 1, 512);
#undef FRK_GO
#undef FRK_GO2
    FRK_LAUNCH_CHECK("gemv_q4_k_fused");
    return FRK_OK;
}

bool fused_gemv_fits(const frk_weights *w) {
    // up to 4 half blocks per lane and 8 activation blocks per wavefront: rows of at most 64
    // blocks; wider rows take the generic kernels
    return w->cols <= FUSED_GEMV_MAX_COLS;
}

// rows stored back to back whose block count divides 64
static bool lines_kernel_fits(const frk_weights *w) {
    const size_t nb = w->cols / QK_K;
    const size_t bb = w->kind == FRK_KIND_Q5_K ? Q5_K_BYTES : Q4_K_BYTES;
    return (nb == 8 || nb == 16 || nb == 32 || nb == 64) && w->layout.row_stride == nb * bb;
}
template <int NB, int MODE, int WAVES, bool Q5 = false, int AHEAD = 0, bool MULTI = false>
static int launch_q4_k_lines_as(const frk_weights *w, const float *x, Q8KActs a, float *y, hipStream_t s, size_t rows_total = 0,
                                const MultiArgs *multi = nullptr) {
    constexpr size_t shmem = (size_t)NB * (LINES_ACT_STRIDE + 32 + 4) + (size_t)WAVES * 64 * (Q5 ? Q5_K_BYTES : Q4_K_BYTES);
    static_assert(shmem <= 160 * 1024, "LDS of a CU");
    const size_t rows = MULTI ? rows_total : w->rows;
    typename MultiArgsFor<MULTI>::type ma;
    if constexpr (MULTI) ma = *multi;
    const size_t spans = (rows * (size_t)NB + 63) / 64;
    const unsigned grid = (unsigned)((spans + WAVES - 1) / WAVES);
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4_k_lines_kernel<NB, MODE, WAVES, Q5, AHEAD, MULTI>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(gemv lines, LDS %zu): %s", shmem, hipGetErrorString(e));
        sized = true;
    }
    hipLaunchKernelGGL((gemv_q4_k_lines_kernel<NB, MODE, WAVES, Q5, AHEAD, MULTI>), dim3(grid), dim3(64 * WAVES), shmem, s, w->dev,
                       (int)rows, x, a.q, a.d, a.bsums, y, ma);
    FRK_LAUNCH_CHECK("gemv_q4_k_lines");
    return FRK_OK;
}
// (Eight wavefronts to a workgroup, two workgroups to a CU.  Measured at 14336x4096, one-launch form /
// pre-quantized form in us: 8 wavefronts 8.1 / 7.5; 7 (which spreads the 3584 spans evenly, 14 per CU)
// 8.7 / 7.7; 14 in one workgroup per CU 9.2 / 8.7; 4 9.0 / 8.3; 2 12.1 / 8.3.)
template <int MODE>
static int launch_q4_k_lines(const frk_weights *w, const float *x, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    constexpr int WIDE = 8;
    // (few workgroups -- fewer of eight wavefronts than half the CUs: four wavefronts each, twice as many CUs take part)
    const size_t few = (size_t)compute_units() / 2;
    if (nb == 8) {  // 4096x2048 3.5 against 4.0 us, 8192x2048 4.0 / 4.35
        const size_t wgs8 = (w->rows * (size_t)8 / 64 + WIDE - 1) / WIDE;
        if (wgs8 <= few) return launch_q4_k_lines_as<8, MODE, 4>(w, x, a, y, s);
        return launch_q4_k_lines_as<8, MODE, WIDE>(w, x, a, y, s);
    }
    if (nb == 16) {
        // one round of workgroups that fills the CUs (two workgroups each): part of the span behind the barrier
        const size_t wgs = (w->rows * (size_t)16 / 64 + WIDE - 1) / WIDE, room = 2 * (size_t)compute_units();
        // between one and one and a half workgroups of eight a CU (10240, 11008 rows): six wavefronts to a workgroup
        // spread the spans more evenly (11008x4096 7.5 against 7.8 us, from quantized activations 6.8 / 7.2; five
        // and seven are behind six, and 12288 rows and more are best with eight)
        if (2 * wgs > room && 4 * wgs < 3 * room)
            return MODE == MODE_FUSED ? launch_q4_k_lines_as<16, MODE, 6, false, 4>(w, x, a, y, s) : launch_q4_k_lines_as<16, MODE, 6>(w, x, a, y, s);
        if (MODE == MODE_FUSED && wgs <= room && 4 * wgs >= 3 * room) return launch_q4_k_lines_as<16, MODE, WIDE, false, 4>(w, x, a, y, s);
        // few workgroups: four wavefronts each, so that twice as many CUs take part (4096x4096 4.4 against 4.7 us,
        // 1024x4096 from quantized activations 3.1 / 3.6; two wavefronts quantize eight blocks each: 5.6 at 1024x4096)
        if (wgs <= few) return launch_q4_k_lines_as<16, MODE, 4>(w, x, a, y, s);
        return launch_q4_k_lines_as<16, MODE, WIDE>(w, x, a, y, s);
    }
    if (nb == 32) {  // (from quantized activations: 2048x8192 4.0 against 4.25 us, 1024x8192 3.4 / 3.85)
        const size_t wgs32 = (w->rows * (size_t)32 / 64 + WIDE - 1) / WIDE;
        if (wgs32 <= few) return launch_q4_k_lines_as<32, MODE, 4>(w, x, a, y, s);
        return launch_q4_k_lines_as<32, MODE, WIDE>(w, x, a, y, s);
    }
    return launch_q4_k_lines_as<64, MODE, 8>(w, x, a, y, s);
}

int launch_gemv_q4_k_fused(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    if (lines_kernel_fits(w)) return launch_q4_k_lines<MODE_FUSED>(w, x, Q8KActs{nullptr, nullptr, nullptr}, y, s);
    return launch_q4_k_fused<MODE_FUSED>(w, nullptr, x, Q8KActs{nullptr, nullptr, nullptr}, y, s);
}
int launch_gemv_q4_k_preq(const frk_weights *w, Q8KActs a, float *y, hipStream_t s) {
    if (lines_kernel_fits(w)) return launch_q4_k_lines<MODE_PREQ_LDS>(w, nullptr, a, y, s);
    if (w->cols <= 8192) return launch_q4_k_fused<MODE_PREQ_DIRECT>(w, nullptr, nullptr, a, y, s);
    return launch_q4_k_fused<MODE_PREQ_LDS>(w, nullptr, nullptr, a, y, s);
}
// rows of any block count up to 64, stored back to back: whole rows to a wavefront (gemv_q4_k_rows_kernel)
bool rows_gemv_fits(const frk_weights *w) {
    const size_t nb = w->cols / QK_K;
    const size_t bb = w->kind == FRK_KIND_Q5_K ? Q5_K_BYTES : Q4_K_BYTES;
    return (w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K) && nb >= 1 && nb <= 64 && w->layout.row_stride == nb * bb;
}
template <int MODE, bool Q5, int WAVES = 8>
static int launch_rows_as(const frk_weights *w, const float *x, Q8KActs a, float *y, hipStream_t s) {
    constexpr size_t slot = 64 * (Q5 ? Q5_K_BYTES : Q4_K_BYTES);
    const int nb = (int)(w->cols / QK_K);
    const size_t shmem = (((size_t)nb * (LINES_ACT_STRIDE + 32 + 4) + 15) & ~(size_t)15) + WAVES * slot;
    const size_t spans = (w->rows + (size_t)(64 / nb) - 1) / (size_t)(64 / nb);
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        constexpr size_t most = ((64 * (LINES_ACT_STRIDE + 32 + 4) + 15) & ~15) + WAVES * slot;
        static_assert(most <= 160 * 1024, "LDS of a CU");
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4_k_rows_kernel<MODE, WAVES, Q5>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)most);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(gemv rows): %s", hipGetErrorString(e));
        sized = true;
    }
    hipLaunchKernelGGL((gemv_q4_k_rows_kernel<MODE, WAVES, Q5>), dim3((unsigned)((spans + WAVES - 1) / WAVES)), dim3(64 * WAVES),
                       shmem, s, w->dev, (int)w->rows, nb, x, a.q, a.d, a.bsums, y);
    FRK_LAUNCH_CHECK("gemv_q4_k_rows");
    return FRK_OK;
}
int launch_gemv_rows_fused(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const Q8KActs none{nullptr, nullptr, nullptr};
    return w->kind == FRK_KIND_Q5_K ? launch_rows_as<MODE_FUSED, true>(w, x, none, y, s) : launch_rows_as<MODE_FUSED, false>(w, x, none, y, s);
}
// (six wavefronts to a workgroup: two workgroups' slots and activations fit a CU's LDS up to 64 blocks a row;
// measured at 4096x14336 from quantized activations, kernel + the quantization launch: 6: 11.8 us, 7: 12.1,
// 8: 12.6, 10: 13.9, 14: 15.4)
int launch_gemv_rows_preq(const frk_weights *w, Q8KActs a, float *y, hipStream_t s) {
    // (Q5_K's slots are 11 KB: six wavefronts would be alone on a CU, eight are more)
    return w->kind == FRK_KIND_Q5_K ? launch_rows_as<MODE_PREQ_LDS, true, 8>(w, nullptr, a, y, s)
                                    : launch_rows_as<MODE_PREQ_LDS, false, 6>(w, nullptr, a, y, s);
}
// Which form a decode GEMV of this matrix takes, by measurement (Q4_K, us; one launch with the quantization
// inside on the per-lane kernel / on the whole-rows kernel / a quantization launch and the whole-rows kernel):
//   4096x14336 15.3 / 15.3 / 11.8    4096x11008 13.6 / 13.2 / 11.0    5120x13824 19.0 / 21.2 / 13.6
//   4096x16384 15.2 (whole lines) / 16.2 / 12.3 -- a workgroup quantizing 56 KB of activation for 74 KB of
//   weights is what a long row costs in one launch;
//   5120x5120 7.8 / 5.9 / 6.9    6144x6144 8.7 / 8.8 / 9.0    8192x3072 5.5 / 5.2 / 6.7    3072x3072 3.7 / 4.6 / 5.9
//   2560x2560 3.4 / 4.5 / 5.8
// Rows of 8, 16 and 32 blocks have the whole-cache-line kernel (14336x4096: 8.2 / 8.9 / 10.3).
int launch_gemv_q4_k_cols(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K), waves = (nb + 3) / 4;
    const int cus = compute_units();
    int best_u = 1;
    size_t best = SIZE_MAX;
    // rows to a workgroup, 8 * U: the U with the least (workgroups of the busiest CU) x (8 * U rows + the quantization
    // of the activation, about seven rows' worth), the larger of equals
    const bool q5 = w->kind == FRK_KIND_Q5_K;
    for (int u = 1; u <= (q5 ? 2 : 3); u++) {
        const size_t wgs = (w->rows + 8 * u - 1) / (8 * u);
        const size_t cost = (wgs + cus - 1) / cus * (8 * u + 7);
        if (cost <= best) best = cost, best_u = u;
    }
    const size_t lds = (size_t)waves * (COLS_WAVE_LDS + 8 * best_u * 4);
    const dim3 grid((unsigned)((w->rows + 8 * best_u - 1) / (8 * best_u))), block(64 * waves);
#define FRK_GO_COLS(UU) \
    hipLaunchKernelGGL((gemv_q4_k_cols_kernel<UU>), grid, block, lds, s, w->dev, w->layout.row_stride, (int)w->rows, nb, x, y)
#define FRK_GO_COLS5(UU) \
    hipLaunchKernelGGL((gemv_q4_k_cols_kernel<UU, true>), grid, block, lds, s, w->dev, w->layout.row_stride, (int)w->rows, nb, x, y)
    if (q5 && best_u == 1) FRK_GO_COLS5(1);
    else if (q5) FRK_GO_COLS5(2);
    else if (best_u == 1) FRK_GO_COLS(1);
    else if (best_u == 2) FRK_GO_COLS(2);
    else FRK_GO_COLS(3);  // (four rounds do not fit the registers of sixteen wavefronts)
#undef FRK_GO_COLS5
#undef FRK_GO_COLS
    FRK_LAUNCH_CHECK("gemv_q4_k_cols");
    return FRK_OK;
}

// Which kernel a one-launch GEMV of Q4_K / Q5_K rows of other lengths than 8 and 16 blocks takes.
int rows_gemv_form(const frk_weights *w) {
    if (!rows_gemv_fits(w)) return ROWS_FORM_NONE;
    const size_t nb = w->cols / QK_K;
    if (w->kind == FRK_KIND_Q4_K) {
        // The column form, measured against what was there (us): 4096x14336 10.5 / 12.5, 4096x11008 9.2 / 11.5,
        // 5120x13824 12.6 / 14.2, 8192x10240 14.1 / 17.3, 4096x6144 6.0 / 6.4, 2048x14336 7.0 / 8.8; against the
        // whole-cache-line kernel at 64 blocks 4096x16384 11.2 / 12.9, 2048x16384 7.4 / 9.3, at 32 blocks
        // 28672x8192 28.9 / 36.0, 14336x8192 17.1 / 21.0, 8192x8192 11.1 / 12.1, 1024x8192 4.8 / 5.3, but
        // 4096x8192 7.2 / 6.8; rows of 20 blocks 5120x5120 6.3 / 6.0, of 16 blocks 14336x4096 10.5 / 8.1.
        if (nb > 20 && nb != 32) return ROWS_FORM_COLUMNS;
        if (nb == 32 && (w->rows <= 2048 || w->rows >= 6144)) return ROWS_FORM_COLUMNS;
    }
    // Q5_K on the same kernel (two rounds at most): 4096x14336 12.8 / 14.8, 4096x11008 10.4 / 13.7, 8192x10240 17.5 / 22.5,
    // 4096x16384 13.3 / 16.8, 2048x16384 8.3 / 9.1; up to 32 blocks it is behind (5120x5120 7.6 / 6.8, 4096x8192 8.3 / 7.3)
    if (w->kind == FRK_KIND_Q5_K && nb > 32) return ROWS_FORM_COLUMNS;
    if (nb > 16 && nb < 32) return ROWS_FORM_ONE_LAUNCH;
    if (rows_gemv_takes_quantized(w)) return ROWS_FORM_QUANTIZED;
    return ROWS_FORM_NONE;
}
// Rows of more than 32 blocks from activations quantized beforehand: whole rows to a wavefront.
// (Q5_K rows of 64 blocks: the whole-cache-line kernel is ahead, 9.2 us against 12.2 at 2048x16384.)
bool rows_gemv_takes_quantized(const frk_weights *w) {
    const size_t nb = w->cols / QK_K;
    return rows_gemv_fits(w) && nb > 32 && !(nb == 64 && w->kind == FRK_KIND_Q5_K);
}

// Q5_K rows of 8, 16, 32 or 64 blocks on the same kernel.  Wavefronts to a workgroup, measured (one-launch form,
// us): 14336x4096 -- 4: 10.4, 5: 11.7, 6: 11.6, 7: 12.0, 8: 10.9; 4096x8192 -- 4: 9.0, 6: 10.9, 8: 7.3;
// 8192x2048 -- 4: 4.1, 8: 4.6.  (An 11 KB span a wavefront: four wavefronts make three workgroups a CU.)
bool q5_k_lines_gemv_fits(const frk_weights *w) { return w->kind == FRK_KIND_Q5_K && lines_kernel_fits(w); }
template <int MODE>
static int launch_q5_k_lines(const frk_weights *w, const float *x, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    if (nb == 8) return launch_q4_k_lines_as<8, MODE, 4, true>(w, x, a, y, s);
    if (nb == 16) return launch_q4_k_lines_as<16, MODE, 4, true>(w, x, a, y, s);
    if (nb == 32) return launch_q4_k_lines_as<32, MODE, 8, true>(w, x, a, y, s);
    return launch_q4_k_lines_as<64, MODE, 8, true>(w, x, a, y, s);
}
int launch_gemv_q5_k_fused(const frk_weights *w, const float *x, float *y, hipStream_t s) {
    return launch_q5_k_lines<MODE_FUSED>(w, x, Q8KActs{nullptr, nullptr, nullptr}, y, s);
}
int launch_gemv_q5_k_preq(const frk_weights *w, Q8KActs a, float *y, hipStream_t s) {
    return launch_q5_k_lines<MODE_PREQ_LDS>(w, nullptr, a, y, s);
}
// ys[i] = ws[i] . x for 2..4 Q4_K matrices of one row length (fused_gemv_fits), one launch
int launch_gemv_q4_k_group(const frk_weights *const *ws, size_t n, const float *x, float *const *ys, hipStream_t s) {
    MultiArgs ma;
    size_t total = 0;
    for (size_t i = 0; i < 4; i++) {
        const size_t j = i < n ? i : n - 1;
        ma.W[i] = ws[j]->dev;
        ma.y[i] = ys[j];
        ma.first[i] = (int)total;
        if (i < n) total += ws[i]->rows;
    }
    for (size_t i = n; i < 4; i++) ma.first[i] = (int)total;
    // rows of 8 or 16 blocks, every matrix a whole number of spans: the whole-cache-line kernel over the list
    // (q/k/v of 4096 + 1024 + 1024 rows x 4096: 5.3 us against 6.3 on the per-lane kernel)
    const size_t nb = ws[0]->cols / QK_K;
    bool lines = nb == 8 || nb == 16;
    for (size_t i = 0; i < n; i++) lines = lines && lines_kernel_fits(ws[i]) && ws[i]->cols == ws[0]->cols && ws[i]->rows % (64 / nb) == 0;
    if (lines) {
        const Q8KActs none{nullptr, nullptr, nullptr};
        if (nb == 8) return launch_q4_k_lines_as<8, MODE_FUSED, 8, false, 0, true>(ws[0], x, none, ys[0], s, total, &ma);
        return launch_q4_k_lines_as<16, MODE_FUSED, 8, false, 0, true>(ws[0], x, none, ys[0], s, total, &ma);
    }
    return launch_q4_k_fused<MODE_FUSED, false, true>(ws[0], nullptr, x, Q8KActs{nullptr, nullptr, nullptr}, ys[0], s, total, &ma);
}
// One launch for `jobs` activation rows against `per_job` experts each, out of a stack of n_experts
// Q4_K matrices of rows_e rows (fused_gemv_fits): y[(job*per_job + sub)][rows_e]; with w2, silu(w.x)*(w2.x).
int launch_gemv_q4_k_experts(const frk_weights *w, const frk_weights *w2, int n_experts, size_t rows_e, const float *x,
                             size_t x_stride, const int32_t *ids, size_t jobs, size_t per_job, float *y, hipStream_t s) {
    if (jobs > 65535 || per_job > 65535) return set_error(FRK_ERR_SHAPE, "%zu x %zu expert launches exceed the grid", jobs, per_job);
    MultiArgs ma = {};
    ma.ids = ids;
    ma.n_experts = n_experts;
    ma.x_stride = (int)x_stride;
    const Q8KActs none = {nullptr, nullptr, nullptr};
    if (w2) return launch_q4_k_fused<MODE_FUSED, true, false, true>(w, w2, x, none, y, s, rows_e, &ma, (unsigned)jobs, (unsigned)per_job);
    return launch_q4_k_fused<MODE_FUSED, false, false, true>(w, nullptr, x, none, y, s, rows_e, &ma, (unsigned)jobs, (unsigned)per_job);
}
// act[r] = silu(gate[r] . x) * (up[r] . x): both matrices Q4_K of one shape, fused_gemv_fits
int launch_gemv_q4_k_glu(const frk_weights *gate, const frk_weights *up, const float *x, float *act, hipStream_t s) {
    return launch_q4_k_fused<MODE_FUSED, true>(gate, up, x, Q8KActs{nullptr, nullptr, nullptr}, act, s);
}

}  // namespace frk
