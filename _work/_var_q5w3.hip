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
template <int NB, int MODE, int WAVES, bool Q5 = false>
__global__ __launch_bounds__(64 * WAVES) void gemv_q4_k_lines_kernel(const uint8_t *__restrict__ W, int rows,
                                                                    const float *__restrict__ x,
                                                                    const int8_t *__restrict__ aq,
                                                                    const float *__restrict__ ad,
                                                                    const int16_t *__restrict__ absums,
                                                                    float *__restrict__ y) {
    constexpr int RPS = 64 / NB;  // rows of a wavefront's span
    constexpr int BB = Q5 ? Q5_K_BYTES : Q4_K_BYTES, SPAN = 64 * BB, PIECES = SPAN / 1024;  // 9 or 11 KB
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
    {
        const size_t span_c = min(span, (bytes - 1) / SPAN);
        const uint8_t *src = W + span_c * SPAN;
        const uint32_t left = (uint32_t)min((size_t)SPAN, bytes - span_c * SPAN);  // (the last span may be short)
        const uint32_t slot = lds_address(sw) + (uint32_t)wave * SPAN;
#pragma unroll
        for (int c = 0; c < PIECES; c++) dma16(slot + c * 1024, src, min((uint32_t)(c * 1024 + lane * 16), left - 16));
    }

    // ---- the activation into LDS ----
    if (MODE == MODE_FUSED) {
        // the activation's loads are older than the span's nine (Q5_K: eleven)
        // (one wait that names them all, so that the blocks' quantizations can be interleaved)
        constexpr int XB = (NB + WAVES - 1) / WAVES;
        // (exactly the registers there are: an operand named twice would be copied in front of the wait)
        static_assert(XB >= 1 && XB <= 8, "up to eight blocks of the activation a wavefront");
        if constexpr (XB == 1) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(xv[0]) : "n"(PIECES));
        if constexpr (XB == 2) asm volatile("s_waitcnt vmcnt(%2)" : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]) : "n"(PIECES));
        if constexpr (XB == 3)
            asm volatile("s_waitcnt vmcnt(%3)" : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]) : "n"(PIECES));
        if constexpr (XB == 4)
            asm volatile("s_waitcnt vmcnt(%4)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0])
                         : "n"(PIECES));
        if constexpr (XB == 5)
            asm volatile("s_waitcnt vmcnt(%5)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0])
                         : "n"(PIECES));
        if constexpr (XB == 6)
            asm volatile("s_waitcnt vmcnt(%6)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0]), "+v"(xv[XB > 5 ? 5 : 0])
                         : "n"(PIECES));
        if constexpr (XB == 7)
            asm volatile("s_waitcnt vmcnt(%7)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0]), "+v"(xv[XB > 5 ? 5 : 0]), "+v"(xv[XB > 6 ? 6 : 0])
                         : "n"(PIECES));
        if constexpr (XB == 8)
            asm volatile("s_waitcnt vmcnt(%8)"
                         : "+v"(xv[0]), "+v"(xv[XB > 1 ? 1 : 0]), "+v"(xv[XB > 2 ? 2 : 0]), "+v"(xv[XB > 3 ? 3 : 0]),
                           "+v"(xv[XB > 4 ? 4 : 0]), "+v"(xv[XB > 5 ? 5 : 0]), "+v"(xv[XB > 6 ? 6 : 0]), "+v"(xv[XB > 7 ? 7 : 0])
                         : "n"(PIECES));
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
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the span has landed (in this wavefront's own slot)
    if (!has_rows) return;

    // ---- lane l multiplies block l of the span ----
    const int b = lane % NB;
    const uint4 *blk = reinterpret_cast<const uint4 *>(sw + wave * SPAN + lane * BB);
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
    const uint4 *ap = reinterpret_cast<const uint4 *>(sq + b * LINES_ACT_STRIDE);
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
    const int4 bsa = *reinterpret_cast<const int4 *>(sbs + b * 8), bsb = *reinterpret_cast<const int4 *>(sbs + b * 8 + 4);
    int s2 = __mul24((int)(m_lo & 0xff), bsa.x) + __mul24((int)((m_lo >> 8) & 0xff), bsa.y) +
             __mul24((int)((m_lo >> 16) & 0xff), bsa.z) + __mul24((int)(m_lo >> 24), bsa.w);
    s2 += __mul24((int)(m_hi & 0xff), bsb.x) + __mul24((int)((m_hi >> 8) & 0xff), bsb.y) +
          __mul24((int)((m_hi >> 16) & 0xff), bsb.z) + __mul24((int)(m_hi >> 24), bsb.w);
    const float da = sd[b];
    const float d = h2f(hd.x & 0xffffu), dmin = h2f(hd.x >> 16);
    float v = (d * da) * (float)s1 - (dmin * da) * (float)s2;
    const size_t row = span * RPS + lane / NB;
    if (row >= (size_t)rows) v = 0.0f;  // (a short last span: this lane's block is not there)
    v = part_sum<NB>(v);
    if (lane % NB == 0 && row < (size_t)rows) y[row] = v;
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
template <int NB, int MODE, int WAVES, bool Q5 = false>
static int launch_q4_k_lines_as(const frk_weights *w, const float *x, Q8KActs a, float *y, hipStream_t s) {
    constexpr size_t shmem = (size_t)NB * (LINES_ACT_STRIDE + 32 + 4) + (size_t)WAVES * 64 * (Q5 ? Q5_K_BYTES : Q4_K_BYTES);
    static_assert(shmem <= 160 * 1024, "LDS of a CU");
    const size_t spans = (w->rows * (size_t)NB + 63) / 64;
    const unsigned grid = (unsigned)((spans + WAVES - 1) / WAVES);
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4_k_lines_kernel<NB, MODE, WAVES, Q5>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(gemv lines, LDS %zu): %s", shmem, hipGetErrorString(e));
        sized = true;
    }
    hipLaunchKernelGGL((gemv_q4_k_lines_kernel<NB, MODE, WAVES, Q5>), dim3(grid), dim3(64 * WAVES), shmem, s, w->dev, (int)w->rows, x,
                       a.q, a.d, a.bsums, y);
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
    if (nb == 8) return launch_q4_k_lines_as<8, MODE, WIDE>(w, x, a, y, s);
    if (nb == 16) return launch_q4_k_lines_as<16, MODE, WIDE>(w, x, a, y, s);
    if (nb == 32) return launch_q4_k_lines_as<32, MODE, WIDE>(w, x, a, y, s);
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
// Q5_K rows of 8, 16, 32 or 64 blocks on the same kernel (six wavefronts to a workgroup: two workgroups'
// 11 KB spans fit a CU's LDS beside the activation; rows of 64 blocks eight)
bool q5_k_lines_gemv_fits(const frk_weights *w) { return w->kind == FRK_KIND_Q5_K && lines_kernel_fits(w); }
template <int MODE>
static int launch_q5_k_lines(const frk_weights *w, const float *x, Q8KActs a, float *y, hipStream_t s) {
    const int nb = (int)(w->cols / QK_K);
    constexpr int WAVES = 3;
    if (nb == 8) return launch_q4_k_lines_as<8, MODE, WAVES, true>(w, x, a, y, s);
    if (nb == 16) return launch_q4_k_lines_as<16, MODE, WAVES, true>(w, x, a, y, s);
    if (nb == 32) return launch_q4_k_lines_as<32, MODE, WAVES, true>(w, x, a, y, s);
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
