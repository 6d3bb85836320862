// Prefill / batched GEMM over Q4_K weights on the matrix cores:
//   y[tok][row] = sum_k W[row][k] * x[tok][k],  x quantized per token to Q8_K first.
//
// Arithmetic is dot_q4_k_q8's (crates/frink-quant/src/lib.rs:822-869), regrouped so that a whole
// 256-weight block accumulates inside the MFMA:
//   S1 = sum_j sc_j * isum_j   with sc_j = 8*sh_j + sl_j (sh, sl < 8): a weight row's block becomes two
//                              int8 operand planes  H = sh_j * q  and  L = sl_j * q  (each < 106), so
//                              S1 = 8 * (acts . H) + (acts . L), exact, no per-sub-block rescale;
//   S2 = sum_j m_j * bsum_j    the activation's 16-wide sums (|bsum| <= 2032) and the 6-bit mins are both
//                              exact in f16, their products and the 16-term sum exact in f32, so one
//                              v_mfma_f32_32x32x16_f16 gives S2 already as a float.
// Per block and output the epilogue is then  acc += da * (d * S1 - dmin * S2)  in f32.
// (Scaling each sub-block's product after a K=32 MFMA instead -- one v_mad_i32_i24 per result and
// sub-block -- was measured slower here: it is bound by the vector ALU and needs more registers.)
//
// MFMA operand roles: A = activations (tile row = token), B = weights (tile column = weight row), so
// a lane's 16 results share one weight row (its d, dmin are per-lane values) and span 16 tokens.
// Operand layout of v_mfma_i32_32x32x32_i8 (checked on the device): lane l holds, for row/column
// l % 32, the 16 k-values 16*(l/32) .. +15 (8*(l/32) .. +7 for the K=16 f16 form); result register
// r of lane l is D[8*(r/4) + 4*(l/32) + r%4][l % 32].
//
// Data movement: everything a block needs -- the workgroup's 128 weight rows (raw 144-byte blocks)
// and its activation tile -- goes from global memory straight into LDS with global_load_lds_dwordx4
// (the 64 lanes' 16-byte pieces land in 1 KB of consecutive LDS; each lane chooses which piece it
// fetches, so the LDS image is whatever order the consumer wants), several blocks ahead, in rings of
// stages.  No prefetch lives in registers, and the only waits on memory are "the stage issued P
// iterations ago has landed".
#include "frk_device.hpp"

#include <type_traits>

namespace frk {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short us2 __attribute__((ext_vector_type(2)));

// Activation side: Q8_K quantization (quantize_activations_q8_k, crates/frink-quant/src/act_quant.rs:69-104)
// into the tiled form, one workgroup per record (32 rows x one block).
// Without `gather`, out row r = x[r] (rows from `rows` to the end of the last tile become zeros); with
// it, out row r = x[gather[r]] (zeros where the entry is negative) for the records whose first entry
// is not negative.
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void quantize_q8_k_tiled_kernel(const float *__restrict__ x, int rows, int nb,
                                                                  const int *__restrict__ gather, Q8KTiled out) {
    __shared__ Q8KRecordLds L;
    const int t32 = blockIdx.x / nb, kb = blockIdx.x % nb, lane = threadIdx.x & 63;
    if (gather && gather[t32 * 32] < 0) return;
    quantize_q8k_record<WAVES>(out, (size_t)t32 * nb + kb, L, [&](int r) {
        const int row = t32 * 32 + r;
        const int src = gather ? gather[row] : (row < rows ? row : -1);
        if (src < 0) return make_float4(0.f, 0.f, 0.f, 0.f);
        return reinterpret_cast<const float4 *>(x + ((size_t)src * nb + kb) * QK_K)[lane];
    });
}

struct GemmArgs {
    const uint8_t *W;
    size_t row_stride;
    int rows, nb, M;
    Q8KTiled a;  // ceil(M / 32) tiles
    float *y;    // [M][rows]
    int row_tiles, tok_tiles;
    int k_split;     // 1, or 2/4: blockIdx.y takes that share of a row's blocks and writes its sums to `partial`
    float *partial;  // [k_split][M][rows], added up in order afterwards (launch_sum_parts)
};

// The grouped form: work items (tile, matrix, row group of 256 rows) streamed by persistent workgroups.
struct StreamArgs {
    const uint8_t *W[2];
    float *y[2];  // [32 * tiles][rows]
    int n_mat;
    size_t row_stride;
    int rows, nb;  // of one expert
    Q8KTiled a;
    const int4 *tiles;  // {expert, 32 * t, rows in use, 0}
    const int *n_tiles;
    int row_tiles;  // ceil(rows / 256)
};

// One block of a lane's weight row as MFMA B operands: the two pre-scaled planes of the 8 sub-blocks,
// the mins as f16 and the block's two f32 scales.  (Named members, not arrays: they must stay in
// registers.)
struct BPlanes {
    v4i H0, H1, H2, H3, H4, H5, H6, H7;
    v4i L0, L1, L2, L3, L4, L5, L6, L7;
    v8h m;
    float d, ndmin;
};
struct RawBlock {  // header + the lane's 16-byte half of each 32-byte nibble pair, as read from LDS
    v4i wh, q0, q1, q2, q3;
};
struct TileOperands {  // one 32-token tile of a block: 8 k-slices of quants and the bsums
    v4i a0, a1, a2, a3, a4, a5, a6, a7;
    v8h bs;
};
struct TileScales {  // the tile's 16 block scales this lane's results need
    v4f da0, da1, da2, da3;
};
struct TileAcc {
    v16i s1;  // sum_j sc_j * isum_j
    v16f s2;  // sum_j m_j * bsum_j
};

// LDS reads are issued from inline assembly so that the compiler's wait-count insertion does not see
// them: it cannot tell that an LDS read does not alias a stage a global_load_lds is still filling
// and would wait for vmcnt(0), i.e. for the whole prefetch, in front of every read.  The price is
// that the waits are placed by hand.  LDS operations of a wavefront complete in order, so
// "at most N outstanding" means everything but the N youngest reads has arrived; each wait names the
// registers it releases so that their uses cannot be scheduled above it.
#define FRK_DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:" #off : "=v"(dst) : "v"(addr))

__device__ __forceinline__ void read_raw(RawBlock &R, uint32_t header, uint32_t quants) {
    FRK_DS_READ(R.wh, header, 0);
    FRK_DS_READ(R.q0, quants, 16);
    FRK_DS_READ(R.q1, quants, 48);
    FRK_DS_READ(R.q2, quants, 80);
    FRK_DS_READ(R.q3, quants, 112);
}
__device__ __forceinline__ void read_ops(TileOperands &T, uint32_t quants, uint32_t bsums) {
    FRK_DS_READ(T.a0, quants, 0);
    FRK_DS_READ(T.a1, quants, 1024);
    FRK_DS_READ(T.a2, quants, 2048);
    FRK_DS_READ(T.a3, quants, 3072);
    FRK_DS_READ(T.a4, quants, 4096);
    FRK_DS_READ(T.a5, quants, 5120);
    FRK_DS_READ(T.a6, quants, 6144);
    FRK_DS_READ(T.a7, quants, 7168);
    FRK_DS_READ(T.bs, bsums, 0);
}
// result register r belongs to token 8*(r/4) + 4*(lane/32) + r%4 of the tile
__device__ __forceinline__ void read_scales(TileScales &S, uint32_t scales) {
    FRK_DS_READ(S.da0, scales, 0);
    FRK_DS_READ(S.da1, scales, 32);
    FRK_DS_READ(S.da2, scales, 64);
    FRK_DS_READ(S.da3, scales, 96);
}
template <int N>
__device__ __forceinline__ void wait_scales(TileScales &S) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(S.da0), "+v"(S.da1), "+v"(S.da2), "+v"(S.da3) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_raw(RawBlock &R) {
    asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(R.wh), "+v"(R.q0), "+v"(R.q1), "+v"(R.q2), "+v"(R.q3) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// raw block -> operand planes, in pieces (so that a caller can spread them between other work):
// the 6-bit scales and mins, one nibble pair at a time, the rest.  lg = lane / 32 selects which half
// of every sub-block this lane holds.
struct BlockScales {
    uint32_t sc_lo, sc_hi, m_lo, m_hi;  // a byte per sub-block: 0..3 and 4..7
};
__device__ __forceinline__ BlockScales block_scales(const RawBlock &R) {
    const uint32_t hy = (uint32_t)R.wh.y, hz = (uint32_t)R.wh.z, hw = (uint32_t)R.wh.w;
    BlockScales s;
    s.sc_lo = hy & 0x3f3f3f3fu;
    s.m_lo = hz & 0x3f3f3f3fu;
    s.sc_hi = (hw & 0x0f0f0f0fu) | (((hy >> 6) & 0x03030303u) << 4);
    s.m_hi = ((hw >> 4) & 0x0f0f0f0fu) | (((hz >> 6) & 0x03030303u) << 4);
    return s;
}
// one nibble pair: 16 bytes -> the lane's H and L operands of sub-blocks 2p (low nibbles) and 2p+1
// (high nibbles); scw holds their two scales in its low bytes
__device__ __forceinline__ void unpack_pair(const v4i q, const uint32_t scw, v4i &H0, v4i &L0, v4i &H1, v4i &L1) {
    const uint32_t s0 = scw & 0xff, s1 = (scw >> 8) & 0xff;
    const us2 h0 = {(unsigned short)(s0 >> 3), (unsigned short)(s0 >> 3)};
    const us2 l0 = {(unsigned short)(s0 & 7), (unsigned short)(s0 & 7)};
    const us2 h1 = {(unsigned short)(s1 >> 3), (unsigned short)(s1 >> 3)};
    const us2 l1 = {(unsigned short)(s1 & 7), (unsigned short)(s1 & 7)};
    auto one = [&](const int wi, int &o0, int &o1, int &o2, int &o3) {
        const uint32_t w = (uint32_t)wi;
        const uint32_t nl = w & 0x0f0f0f0fu, nh = (w >> 4) & 0x0f0f0f0fu;
        us2 a, b;
        __builtin_memcpy(&a, &nl, 4);
        __builtin_memcpy(&b, &nh, 4);
        const us2 r0 = a * h0, r1 = a * l0, r2 = b * h1, r3 = b * l1;  // bytes stay below 106
        __builtin_memcpy(&o0, &r0, 4);
        __builtin_memcpy(&o1, &r1, 4);
        __builtin_memcpy(&o2, &r2, 4);
        __builtin_memcpy(&o3, &r3, 4);
    };
    int a0, a1, a2, a3, b0, b1, b2, b3, c0, c1, c2, c3, d0, d1, d2, d3;
    one(q.x, a0, a1, a2, a3);
    one(q.y, b0, b1, b2, b3);
    one(q.z, c0, c1, c2, c3);
    one(q.w, d0, d1, d2, d3);
    H0 = v4i{a0, b0, c0, d0};
    L0 = v4i{a1, b1, c1, d1};
    H1 = v4i{a2, b2, c2, d2};
    L1 = v4i{a3, b3, c3, d3};
}
__device__ __forceinline__ void unpack_rest(const RawBlock &R, const BlockScales &s, int lg, BPlanes &B) {
    // mins of the four sub-blocks whose 16-wide groups are 8*lg .. 8*lg+7, each twice
    const uint32_t hx = (uint32_t)R.wh.x;
    const uint32_t mw = lg ? s.m_hi : s.m_lo;
    const _Float16 m0 = (_Float16)(int)(mw & 0xff), m1 = (_Float16)(int)((mw >> 8) & 0xff);
    const _Float16 m2 = (_Float16)(int)((mw >> 16) & 0xff), m3 = (_Float16)(int)(mw >> 24);
    B.m = v8h{m0, m0, m1, m1, m2, m2, m3, m3};
    B.d = h2f(hx & 0xffffu);
    B.ndmin = -h2f(hx >> 16);
}
__device__ __forceinline__ void unpack_block(const RawBlock &R, int lg, BPlanes &B) {
    const BlockScales s = block_scales(R);
    unpack_pair(R.q0, s.sc_lo, B.H0, B.L0, B.H1, B.L1);
    unpack_pair(R.q1, s.sc_lo >> 16, B.H2, B.L2, B.H3, B.L3);
    unpack_pair(R.q2, s.sc_hi, B.H4, B.L4, B.H5, B.L5);
    unpack_pair(R.q3, s.sc_hi >> 16, B.H6, B.L6, B.H7, B.L7);
    unpack_rest(R, s, lg, B);
}

__device__ __forceinline__ void tile_epilogue(const TileAcc &X, const TileScales &S, const BPlanes &B, v16f &acc) {
    const v4f dav[4] = {S.da0, S.da1, S.da2, S.da3};
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int r = c * 4 + e;
            const float v = fmaf(B.ndmin, X.s2[r], B.d * (float)X.s1[r]);
            acc[r] = fmaf(dav[c][e], v, acc[r]);
        }
}

// The 16 + 1 MFMAs of a tile, each waiting only for the operand it needs: the tile's nine LDS reads
// (a0..a7, bs, in that order) must be the wavefront's youngest LDS operations.
// (Each wait also names the running sum as modified, which pins it between its two MFMAs: without
// that the MFMAs are free to sink below all the waits, and the chain starts only when the last
// operand is there.)
#define FRK_WAIT_LGKM(n, reg, acc) asm volatile("s_waitcnt lgkmcnt(" #n ")" : "+v"(reg), "+v"(acc))
// between(i, acc) is called after MFMA i of the integer chain has been issued, i = 0..14: what it does
// shares the gaps of the chain, every MFMA of which waits for the one before it.
struct NothingBetween {
    __device__ __forceinline__ void operator()(int, v16i &) const {}
};
template <class Between = NothingBetween>
__device__ __forceinline__ void tile_mfmas_as_they_land(TileOperands &T, const BPlanes &B, TileAcc &X,
                                                        Between between = Between()) {
    const v16i zi = {0};
    const v16f zf = {0.0f};
    asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(T.a0));
    v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.H0, zi, 0, 0, 0);
    between(0, acc);
    FRK_WAIT_LGKM(7, T.a1, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.H1, acc, 0, 0, 0);
    between(1, acc);
    FRK_WAIT_LGKM(6, T.a2, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.H2, acc, 0, 0, 0);
    between(2, acc);
    FRK_WAIT_LGKM(5, T.a3, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.H3, acc, 0, 0, 0);
    between(3, acc);
    FRK_WAIT_LGKM(4, T.a4, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.H4, acc, 0, 0, 0);
    between(4, acc);
    FRK_WAIT_LGKM(3, T.a5, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.H5, acc, 0, 0, 0);
    between(5, acc);
    FRK_WAIT_LGKM(2, T.a6, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.H6, acc, 0, 0, 0);
    between(6, acc);
    FRK_WAIT_LGKM(1, T.a7, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.H7, acc, 0, 0, 0);
    between(7, acc);
    FRK_WAIT_LGKM(0, T.bs, acc);
    X.s2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(T.bs, B.m, zf, 0, 0, 0);
    acc = acc << 3;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.L0, acc, 0, 0, 0);
    between(8, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.L1, acc, 0, 0, 0);
    between(9, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.L2, acc, 0, 0, 0);
    between(10, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.L3, acc, 0, 0, 0);
    between(11, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.L4, acc, 0, 0, 0);
    between(12, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.L5, acc, 0, 0, 0);
    between(13, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.L6, acc, 0, 0, 0);
    between(14, acc);
    X.s1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.L7, acc, 0, 0, 0);
}

// The dense kernel's form of a tile, one accumulator less: the mins' MFMA adds onto the converted
// integer sums instead of into registers of its own.  With d' = d / (-dmin):
//     d * S1 - dmin * S2 = (-dmin) * (d' * S1 + S2),
// so the f16 MFMA takes d' * S1 as its C operand and the epilogue multiplies by -dmin (and the token's
// scale).  A row whose dmin is zero keeps d and a factor of one, and zero mins.  (Not the same
// rounding as the two-term form: both are within a few ulp of the exact sum.)
__device__ __forceinline__ void fold_mins(BPlanes &B) {
    const bool z = B.ndmin == 0.0f;
    B.d = z ? B.d : B.d * __builtin_amdgcn_rcpf(B.ndmin);
    B.ndmin = z ? 1.0f : B.ndmin;
    if (z) B.m = v8h{0, 0, 0, 0, 0, 0, 0, 0};
}
template <class Between = NothingBetween>
__device__ __forceinline__ v16f tile_mfmas_folded(TileOperands &T, const BPlanes &B, Between between = Between()) {
    const v16i zi = {0};
    asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(T.a0));
    v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.H0, zi, 0, 0, 0);
    between(0, acc);
    FRK_WAIT_LGKM(7, T.a1, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.H1, acc, 0, 0, 0);
    between(1, acc);
    FRK_WAIT_LGKM(6, T.a2, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.H2, acc, 0, 0, 0);
    between(2, acc);
    FRK_WAIT_LGKM(5, T.a3, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.H3, acc, 0, 0, 0);
    between(3, acc);
    FRK_WAIT_LGKM(4, T.a4, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.H4, acc, 0, 0, 0);
    between(4, acc);
    FRK_WAIT_LGKM(3, T.a5, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.H5, acc, 0, 0, 0);
    between(5, acc);
    FRK_WAIT_LGKM(2, T.a6, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.H6, acc, 0, 0, 0);
    between(6, acc);
    FRK_WAIT_LGKM(1, T.a7, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.H7, acc, 0, 0, 0);
    between(7, acc);
    acc = acc << 3;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.L0, acc, 0, 0, 0);
    between(8, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.L1, acc, 0, 0, 0);
    between(9, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.L2, acc, 0, 0, 0);
    between(10, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.L3, acc, 0, 0, 0);
    between(11, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.L4, acc, 0, 0, 0);
    between(12, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.L5, acc, 0, 0, 0);
    between(13, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.L6, acc, 0, 0, 0);
    between(14, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.L7, acc, 0, 0, 0);
    FRK_WAIT_LGKM(0, T.bs, acc);
    v16f c;
#pragma unroll
    for (int r = 0; r < 16; r++) c[r] = B.d * (float)acc[r];
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(T.bs, B.m, c, 0, 0, 0);
}
__device__ __forceinline__ void tile_epilogue_folded(const v16f &c, const TileScales &S, const BPlanes &B, v16f &acc) {
    const v4f dav[4] = {S.da0, S.da1, S.da2, S.da3};
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int r = q * 4 + e;
            acc[r] = fmaf(dav[q][e] * B.ndmin, c[r], acc[r]);
        }
}

// A workgroup = RG*WT wavefronts = RG row groups of 32 weight rows x WT token groups of MT 32-token
// tiles.  A wavefront keeps the current block of its 32 rows in registers as MFMA B operands and
// runs its MT tiles against them, so a block of a row is unpacked once per MT tiles.  A SIMD holds
// two wavefronts: while one issues a tile's MFMAs the other does its vector work (unpack,
// epilogue), which is how the matrix cores and the vector ALU overlap here.
//
// What bounds the tile shape: every block moves (32*RG*144 + 32*NT*292) bytes from L2 into LDS for
// 2*32*RG*32*NT*256 operations, and a CU's address unit takes roughly 40 cycles per kilobyte of such
// loads (whether they write LDS directly or go through registers), so more rows and tokens per
// workgroup is better -- until the registers run out: 256 rows x 128 tokens (8 wavefronts, four
// tiles each) fits two wavefronts per SIMD (256 registers per lane) without spills, and a spill is
// fatal here because scratch reloads wait on the same counter as the prefetch.  What keeps the
// registers down: the prefetch writes LDS directly, its addresses are recomputed from the lane
// number at every use (made opaque, or the compiler keeps them all), the mins' term shares the
// integer sums' accumulator (tile_mfmas_folded) and every tile's epilogue is pinned to its tile.
//
// LDS rings.  Activations, 2 stages:
//     quants [NT][8 k-slices][1 KB] | bsums f16 [NT][1 KB] | scales f32 [NT*32],  NT = MT*WT tiles
// weights, WS stages of [RG][32 rows][144 B] raw blocks; block kb+1 is unpacked at the end of
// iteration kb, so with WS = 2 a stage is refilled two blocks ahead, with WS = 4 three.
template <int RG, int WT, int MT, int WS>
struct GemmLds {
    static constexpr int NT = WT * MT;
    static constexpr int OFF_BS = NT * 8192;
    static constexpr int OFF_DA = NT * 9216;
    static constexpr int A_STAGE = OFF_DA + ((NT + 1) / 2) * 256;
    static constexpr int W_GROUP = 32 * Q4_K_BYTES;  // 4608
    static constexpr int W_STAGE = RG * W_GROUP;
    static constexpr size_t BYTES = (size_t)2 * A_STAGE + (size_t)WS * W_STAGE;
};

template <int RG, int WT, int MT, int WS>
__global__ __launch_bounds__(64 * RG * WT) void gemm_q4_k_mfma_kernel(GemmArgs g) {
    using L = GemmLds<RG, WT, MT, WS>;
    constexpr int NW = RG * WT, NT = L::NT, TM = 32 * NT, ROWS = 32 * RG;
    constexpr int N_DA = (NT + 1) / 2;
    static_assert(NW == 4 || NW == 8, "the k-slice to wavefront map assumes 4 or 8 wavefronts");
    static_assert(WS == 2 || WS == 4, "weight ring of 2 or 4 stages");
    static_assert(WT == 1 || WT == 2, "one or two token groups");
    constexpr int WD = WS == 4 ? 3 : 2;  // weights are requested WD blocks ahead
    // global_load_lds instructions per wavefront for one block of weights
    constexpr int C_W = WT == 1 ? 5 : 3;
    extern __shared__ uint4 smem_gemm[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem_gemm);
    uint8_t *lds_w = lds + 2 * L::A_STAGE;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lg = lane >> 5;
    const int rgrp = wave % RG, tgrp = wave / RG;

    // workgroups that share weight rows (different token tiles) sit on one XCD (block id mod 8)
    const int bid = blockIdx.x;
    const int per_group = 8 * g.tok_tiles;
    const int grp = bid / per_group, in_grp = bid % per_group;
    const int row_tile = grp * 8 + (in_grp & 7);
    if (row_tile >= g.row_tiles) return;  // uniform per workgroup
    const int tok0 = (in_grp >> 3) * TM;
    const int row0 = row_tile * ROWS + rgrp * 32;  // this wavefront's first weight row
    const int row = row0 + li;
    const int nb = g.nb;  // blocks of a row (strides); this workgroup multiplies blocks kb0 .. kb1 - 1
    const int kb0 = nb * (int)blockIdx.y / g.k_split, kb1 = nb * ((int)blockIdx.y + 1) / g.k_split;
    const int tile0 = tok0 / 32, last_tile = (g.M - 1) / 32;

    // ---- what this lane fetches ----
    // Only 32-bit offsets of the first piece are kept in registers; everything else is uniform or is
    // recomputed from them where it is used.
    // activations: the tiled form is the LDS image, so chunk (tile t, slice ks) is 1 KB of consecutive
    // memory and lane j brings its bytes 16*j..; same for the sums.  Tiles past the last one repeat it.
    // (offsets from the quants: the three arrays of the tiled form are carved from one allocation,
    // quants first)
    const uint8_t *Qb = reinterpret_cast<const uint8_t *>(g.a.q);
    const uint32_t bs_base = (uint32_t)(reinterpret_cast<const uint8_t *>(g.a.bs) - Qb);
    const uint32_t d_base = (uint32_t)(reinterpret_cast<const uint8_t *>(g.a.d) - Qb);
    auto tile_rec = [&](int t) { return (uint32_t)min(tile0 + t, last_tile) * (uint32_t)nb; };  // uniform
    // with fewer chunks than wavefronts some fetch a chunk twice, into the same place
    const int bs_tile = wave % NT, da_chunk = wave % N_DA;
    // weights: a row group's 32 rows x 9 sixteen-byte pieces, piece p = 64*c + lane of chunk c, so that
    // LDS holds the rows back to back (144 bytes each) and consecutive lanes read consecutive memory:
    // chunk c is 7c rows further down and c pieces to the right of chunk 0, modulo the nine of a row.
    // Offsets past the matrix are pulled back to its last 16 bytes (such rows are never stored).
    // With WT = 2 the two wavefronts of a row group split the five chunks (3 + 2, one fetched twice).
    const uint8_t *Wb = g.W;
    const uint32_t stride = (uint32_t)g.row_stride;
    const uint32_t w_last = (uint32_t)g.rows * stride - 16;
    const int wc0 = (WT == 1) ? 0 : (tgrp == 0 ? 0 : 3);
    auto chunk_of = [&](int i) { return min(wc0 + i, 4) - ((WT == 2 && tgrp == 1 && i == 2) ? 1 : 0); };  // tgrp 1: 3, 4, 3
    auto opaque_lane = [&]() {  // the lane number as a value the compiler cannot hoist expressions of
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };

    // the prefetch of one block, as N_A + 2 + C_W separate loads so that they can be issued one by one
    constexpr int N_A = NT * (8 / NW), N_DMA = N_A + 2 + C_W;
    auto act_part = [&](int j, int kb) {  // j = 0 .. N_A + 1
        asm volatile("" : "+s"(kb));  // (seen as the loop counter, every address becomes a pointer of its own)
        uint8_t *st = lds + (kb & 1) * L::A_STAGE;
        const uint32_t l = (uint32_t)opaque_lane();
        if (j < N_A) {
            const int t = j / (8 / NW), i = j % (8 / NW);
            const int ks = ((wave + t) % NW) + NW * i;
            load_to_lds16(Qb + ((tile_rec(t) + kb) * 8192 + ks * 1024 + l * 16), st + (t * 8 + ks) * 1024);
        } else if (j == N_A) {
            load_to_lds16(Qb + (bs_base + (tile_rec(bs_tile) + kb) * 1024 + l * 16), st + L::OFF_BS + bs_tile * 1024);
        } else {
            load_to_lds4(Qb + (d_base + (tile_rec(2 * da_chunk + (l >> 5)) + kb) * 128 + (l & 31) * 4),
                         st + L::OFF_DA + da_chunk * 256);
        }
    };
    auto weight_part = [&](int i, int kb) {  // i = 0 .. C_W - 1
        asm volatile("" : "+s"(kb));
        uint8_t *st = lds_w + (kb % WS) * L::W_STAGE + rgrp * L::W_GROUP;
        const uint32_t l = (uint32_t)opaque_lane();
        const uint32_t pc0 = l % 9;
        const uint32_t off0 = ((uint32_t)(row_tile * ROWS + rgrp * 32) + l / 9) * stride + pc0 * 16 + (uint32_t)kb * Q4_K_BYTES;
        const int c = chunk_of(i);
        const uint32_t v = pc0 + c, wrap = v >= 9 ? 1u : 0u;  // c <= 4: at most one wrap
        const uint32_t off = off0 + (uint32_t)(7 * c) * stride + wrap * (stride - 144) + c * 16;
        // chunk 4 is half a chunk: 32 pieces
        if (c < 4 || l < 32) load_to_lds16(Wb + min(off, w_last), st + c * 1024);
    };
    auto issue_acts = [&](int kb) {
#pragma unroll
        for (int j = 0; j < N_A + 2; j++) act_part(j, kb);
    };
    auto issue_weights = [&](int kb) {
#pragma unroll
        for (int i = 0; i < C_W; i++) weight_part(i, kb);
    };

    const uint32_t lds_a = lds_address(lds);
    const uint32_t lds_wv = lds_address(lds_w) + rgrp * L::W_GROUP + li * Q4_K_BYTES;

    v16f accF[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) accF[mt] = v16f{0.0f};

    BPlanes B;
    RawBlock R;
    v16i accI0 = {0};  // (an argument the prefetch does not use)
    const int pf_tile = __builtin_amdgcn_readfirstlane(wave >= NW / 2 ? MT / 2 : 0);

    // prologue: weights of blocks 0..WD-1, activations of block 0; the last weights may stay in flight
    issue_weights(kb0);
    issue_acts(kb0);
#pragma unroll
    for (int i = 1; i < WD; i++)
        if (kb0 + i < kb1) issue_weights(kb0 + i);
    if (WS == 4 && kb1 - kb0 > 2) wait_vm<C_W>();
    else wait_vm<0>();
    lds_barrier();
    {
        const uint32_t first = lds_wv + (kb0 % WS) * L::W_STAGE;
        read_raw(R, first, first + 16 * lg);
    }
    wait_raw<0>(R);
    unpack_block(R, lg, B);
    fold_mins(B);

    for (int kb = kb0; kb < kb1; kb++) {
        // The first tile's operands are requested before anything else: they travel from LDS while
        // the prefetch below is issued.  In the same way every later tile's operands are requested
        // before the epilogue of the tile before it.
        const uint32_t st = lds_a + (kb & 1) * L::A_STAGE;
        const uint32_t qa = st + lane * 16, ba = st + L::OFF_BS + lane * 16, sa = st + L::OFF_DA + lg * 16;
        const uint32_t wa = lds_wv + ((kb + 1) % WS) * L::W_STAGE;
        TileOperands T;
        read_ops(T, qa + (tgrp * MT) * 8192, ba + (tgrp * MT) * 1024);
        // The prefetch (the stages refilled were last read in iteration kb-1, which every wavefront
        // has left).  A wavefront is stalled while its loads wait for the CU's one address unit, and
        // a block's loads keep that unit busy for about as long as half the block's MFMAs take: so the
        // two wavefronts of a SIMD (w and w + NW/2) issue theirs at different times, from inside the
        // chain of MFMAs of their first and of their middle tile, one load per gap; while one is
        // stalled the other has the matrix core.  With one tile per wavefront there is no such choice.
        auto prefetch_part = [&](int j, v16i &) {
            if (j < N_A + 2) {
                if (kb + 1 < kb1) act_part(j, kb + 1);
            } else if (j < N_DMA) {
                if (kb + WD < kb1) weight_part(j - (N_A + 2), kb + WD);
            }
        };
        if (MT == 1) {
#pragma unroll
            for (int j = 0; j < N_DMA; j++) prefetch_part(j, accI0);
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const int t = tgrp * MT + mt;
            TileScales S;
            v16f c;
            if (MT > 1 && (mt == 0 || mt == MT / 2)) {
                // (one chain for both cases, the choice made per load: two copies of the chain behind
                // a branch would meet in register copies of the operands, which the compiler, blind
                // to the hand-placed waits, is free to put in front of them)
                c = tile_mfmas_folded(T, B, [&](int j, v16i &a) {
                    if (mt == pf_tile) prefetch_part(j, a);
                });
            } else {
                c = tile_mfmas_folded(T, B);
            }
            read_scales(S, sa + t * 128);
            if (mt + 1 < MT) {
                read_ops(T, qa + (t + 1) * 8192, ba + (t + 1) * 1024);
                wait_scales<9>(S);
            } else {
                wait_scales<0>(S);
            }
            tile_epilogue_folded(c, S, B, accF[mt]);
            // (the sums are next used in the following iteration, which lets the compiler sink the
            // epilogues of all tiles to the end of this one, every tile's MFMA result alive until then)
            asm volatile("" : "+v"(accF[mt]));
        }
        if (kb + 1 < kb1) {
            // the next block's raw weights landed during iteration kb-1
            read_raw(R, wa, wa + 16 * lg);
            wait_raw<0>(R);
            unpack_block(R, lg, B);
            fold_mins(B);
            // activations of block kb+1 and weights of block kb+2 must have landed; with four weight
            // stages the weights requested above (younger than both) may stay in flight
            if (WS == 4 && kb + WD < kb1) wait_vm<C_W>();
            else wait_vm<0>();
        }
        lds_barrier();
    }

    // store: a lane holds one weight row and 16 tokens per tile
    float *const dst = g.k_split > 1 ? g.partial + (size_t)blockIdx.y * g.M * g.rows : g.y;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int tok = tok0 + (tgrp * MT + mt) * 32 + (r >> 2) * 8 + lg * 4 + (r & 3);
            if (row < g.rows && tok < g.M) dst[(size_t)tok * g.rows + row] = accF[mt][r];
        }
}

// The grouped (per-expert) GEMM: with a few dozen activation rows per expert the work is a stream
// over the experts' weights.  Persistent workgroups (one per CU, 8 wavefronts, 256 weight rows) walk
// a list of work items (tile, matrix, row group); one step = one 256-wide block of one item.  A
// step's data travels into LDS three steps ahead, across item boundaries: the weights (a wavefront
// fetches and reads only its own 32 rows, so that ring needs no barrier: two stages, each refilled as
// soon as its block has left it for the registers) and the tile's activation record (shared, four
// stages, one barrier per step).  A tile is up to 64 activation rows, two 32-row halves that share
// the unpacked weights; the second half is neither fetched nor multiplied when not in use.
// The unpacked weights are double-buffered in registers: step s+1 is unpacked from inside the chain
// of MFMAs of step s.  The two wavefronts of a SIMD (w and w+4) issue their loads at different
// times, one before its MFMAs and one after: a wavefront is stalled while its loads wait for the
// CU's address unit, and this way the other one has the matrix core meanwhile.
// Items of a tile sit on one XCD (block id mod 8), whose L2 then serves the tile's activations.
struct StreamLds {
    static constexpr int RG = 8;
    static constexpr int W_WAVE = 32 * Q4_K_BYTES;  // a wavefront's 32 rows of one block
    static constexpr int W_STAGE = RG * W_WAVE;     // 36864
    static constexpr int W_STAGES = 2;
    static constexpr int A_BS = 8192, A_DA = 9216;  // record of 32 rows: quants | sums | scales
    static constexpr int A_HALF = 9472;
    static constexpr int A_STAGE = 2 * A_HALF;       // a tile is two records
    static constexpr int A_STAGES = 4;
    static constexpr int OFF_A = W_STAGES * W_STAGE;
    // {expert, rows in use} of each of the workgroup's items, filled once: looked up from LDS, an
    // item change costs no global load (whose completion would count in vmcnt, in the middle of the
    // prefetch bookkeeping)
    static constexpr int OFF_ITEMS = OFF_A + A_STAGES * A_STAGE;
    static constexpr int MAX_ITEMS = 128;
    static constexpr size_t BYTES = (size_t)OFF_ITEMS + MAX_ITEMS * 8;
};

__global__ __launch_bounds__(64 * StreamLds::RG) void gemm_q4_k_stream_kernel(StreamArgs g) {
    using L = StreamLds;
    extern __shared__ uint4 smem_gemm[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem_gemm);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lg = lane >> 5;
    const int nb = g.nb;

    // this workgroup's items: the list of its XCD holds the tiles t = xcd (mod 8), every (matrix, row
    // group) of a tile in a row; the XCD's workgroups take list entries slot, slot + per_xcd, ...
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
    const int n_tiles = *g.n_tiles;
    const int per_tile = g.n_mat * g.row_tiles;
    const int list_len = (n_tiles > xcd ? (n_tiles - xcd + 7) / 8 : 0) * per_tile;
    const int my_items = list_len > slot ? (list_len - slot + per_xcd - 1) / per_xcd : 0;
    const int total_steps = my_items * nb;
    if (total_steps == 0) return;
    // (the quotients are wavefront-uniform but come out of the vector ALU; back in scalar registers
    // they keep the address arithmetic that follows scalar)
    auto item_of = [&](int ord, int &t, int &m, int &rg) {
        const int j = slot + ord * per_xcd;
        const int jt = __builtin_amdgcn_readfirstlane(j / per_tile);
        const int w = j - jt * per_tile;
        t = xcd + 8 * jt;
        m = __builtin_amdgcn_readfirstlane(w / g.row_tiles);
        rg = w - m * g.row_tiles;
    };
    {
        int2 *table = reinterpret_cast<int2 *>(lds + L::OFF_ITEMS);
        for (int i = tid; i < my_items; i += 64 * L::RG) {
            const int4 ti = g.tiles[xcd + 8 * ((slot + i * per_xcd) / per_tile)];
            table[i] = make_int2(ti.x, ti.z);
        }
        __syncthreads();
    }
    const uint32_t lds_items = lds_address(lds + L::OFF_ITEMS);
    auto item_info = [&](int ord, int &expert, int &count) {
        v2i v;
        asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_items + ord * 8));
        expert = __builtin_amdgcn_readfirstlane(v.x);
        count = __builtin_amdgcn_readfirstlane(v.y);
    };

    // ---- the fetch side: a cursor (item, block) three steps ahead of the arithmetic ----
    // weights of a step: this wavefront's 32 rows x 9 sixteen-byte pieces, piece p = 64*c + lane of
    // chunk c (4.5 chunks, 5 loads); activations: quant slice `wave`, plus the sums (wavefront 0) or
    // the scales (wavefront 1).  Addresses are a uniform base that moves with the cursor plus a lane
    // offset that is fixed per item.  Registers are short here, so of the five weight offsets only
    // the first is kept: piece p + 64 = 7 rows + 1 piece further on, one more row where the piece
    // index wraps past 8.  (Everything else the fetch needs is recomputed from the lane number.)
    uint32_t w_off0 = 0;
    // activations: quant slice `wave` of each half in use, plus one of the four small pieces: sums
    // (wavefronts 0, 2) and scales (1, 3) of the first (0, 1) and second half (2, 3)
    const bool x_sums = (wave & 1) == 0;
    auto opaque_lane = [&]() {  // the lane number as a value the compiler cannot hoist expressions of
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    const uint8_t *f_w, *f_x;
    const int8_t *f_q;
    int f_ord = 0, f_kb = 0, f_step = 0;
    bool f_two = false;  // the cursor's tile has rows in its second half
    int issued = 0;      // loads of the fetch most recently issued by this wavefront
    auto point_at = [&](int ord) {  // uniform
        int t, m, rg, expert, count;
        item_of(ord, t, m, rg);
        item_info(ord, expert, count);
        f_w = (m ? g.W[1] : g.W[0]) + (size_t)expert * g.rows * g.row_stride;
        const int l = opaque_lane();
        w_off0 = (uint32_t)(rg * (32 * L::RG) + wave * 32 + l / 9) * (uint32_t)g.row_stride + (uint32_t)(l % 9) * 16;
        f_two = count > 32;
        const size_t rec = (size_t)(2 * t + (wave >> 1 & 1)) * nb;  // the small piece's half
        f_q = g.a.q + (size_t)2 * t * nb * 8192;
        f_x = x_sums ? reinterpret_cast<const uint8_t *>(g.a.bs + rec * 512)
                     : reinterpret_cast<const uint8_t *>(g.a.d + rec * 32);
    };
    auto fetch_acts = [&]() {  // of the cursor's step
        uint8_t *st = lds + L::OFF_A + (f_step & 3) * L::A_STAGE;
        const int l = opaque_lane();
        const uint32_t q_off = (uint32_t)(wave * 1024 + l * 16);
        const uint32_t x_off = x_sums ? (uint32_t)l * 16 : (uint32_t)(l & 31) * 4;
        load_to_lds16(f_q + q_off, st + wave * 1024);
        issued = 1;
        if (f_two) {
            load_to_lds16(f_q + (size_t)nb * 8192 + q_off, st + L::A_HALF + wave * 1024);
            issued = 2;
        }
        if (wave < 2 || (wave < 4 && f_two)) {
            uint8_t *half = st + (wave >> 1) * L::A_HALF;
            if (x_sums) load_to_lds16(f_x + x_off, half + L::A_BS);
            else load_to_lds4(f_x + x_off, half + L::A_DA);  // both lane halves fetch the same 32 scales
            issued++;
        }
    };
    auto fetch_weights = [&]() {  // of the cursor's step; moves the cursor on
        uint8_t *st = lds + (f_step & 1) * L::W_STAGE + wave * L::W_WAVE;
        const int l = opaque_lane();
        const uint32_t r0 = (uint32_t)l % 9, stride = (uint32_t)g.row_stride;
        // rows past the matrix (a last, partial row group) fetch its last piece instead
        const uint32_t last = (uint32_t)(g.rows - 1) * stride + 128;
#pragma unroll
        for (int c = 0; c < 5; c++) {
            const uint32_t off = w_off0 + c * (7 * stride + 16) + (r0 + c >= 9 ? stride - Q4_K_BYTES : 0u);
            if (c < 4 || l < 32) load_to_lds16(f_w + min(off, last), st + c * 1024);
        }
        issued += 5;
        f_step++;
        f_w += Q4_K_BYTES;
        f_q += 8192;
        f_x += x_sums ? 1024 : 128;
        if (++f_kb == nb) {
            f_kb = 0;
            if (++f_ord < my_items) point_at(f_ord);
        }
    };
    // prologue: the data of steps 0 and 1
    point_at(0);
    fetch_acts();
    fetch_weights();
    if (total_steps > 1) {
        fetch_acts();
        fetch_weights();
    }
    wait_vm<0>();
    lds_barrier();

    // ---- the arithmetic.  The unpacked weights are double-buffered in registers: while step s is
    // multiplied out of one set, step s+1 is unpacked into the other, the unpacking's vector
    // instructions filling the gaps between the MFMAs, each of which waits for the one before it.
    // (Every wavefront overlaps its own two kinds of work, so the wavefronts of a SIMD need not
    // be kept in different phases.)  The loop body exists twice, one copy per set. ----
    const uint32_t lds0 = lds_address(lds);
    BPlanes B0, B1;
    v16f accF0 = v16f{0.0f}, accF1 = v16f{0.0f};  // the tile's two halves
    const bool fetch_late = wave >= L::RG / 2;
    int c_ord = 0, c_kb = 0, c_count = 0;
    int pending = -1, pending_count = 0;  // item whose results wait to be stored
    auto raw_of_step = [&](int s) {  // this lane's part of its row's block, read and arrived
        const int l = opaque_lane(), li = l & 31, lg = l >> 5;
        const uint32_t wa = lds0 + (s & 1) * L::W_STAGE + (wave * 32 + li) * Q4_K_BYTES;
        RawBlock R;
        read_raw(R, wa, wa + 16 * lg);
        wait_raw<0>(R);
        return R;
    };
    auto multiply_half = [&](uint32_t st, v16f &accF, const BPlanes &B, auto between) {
        const int lane = opaque_lane(), lg = lane >> 5;
        TileOperands T;
        TileScales S;
        TileAcc X;
        read_ops(T, st + lane * 16, st + L::A_BS + lane * 16);
        tile_mfmas_as_they_land(T, B, X, between);
        read_scales(S, st + L::A_DA + lg * 16);
        wait_scales<0>(S);
        tile_epilogue(X, S, B, accF);
        // the epilogue must not sink below the next half's operand reads (its inputs would stay
        // live through that half's MFMAs): an empty volatile statement that "modifies" the sums
        // keeps its place among the volatile LDS reads
        asm volatile("" : "+v"(accF));
    };
    // (the next step's block R is unpacked into Bnext from inside the first half's chain of MFMAs)
    auto multiply_step = [&](int s, const BPlanes &B, const RawBlock &R, BPlanes &Bnext) {
        const uint32_t st = lds0 + L::OFF_A + (s & 3) * L::A_STAGE;
        if (c_kb == 0) {
            int expert;
            item_info(c_ord, expert, c_count);
        }
        const BlockScales sc = block_scales(R);
        const int lg_next = opaque_lane() >> 5;
        multiply_half(st, accF0, B, [&](int i, v16i &) {
            if (i == 0) unpack_pair(R.q0, sc.sc_lo, Bnext.H0, Bnext.L0, Bnext.H1, Bnext.L1);
            if (i == 2) unpack_pair(R.q1, sc.sc_lo >> 16, Bnext.H2, Bnext.L2, Bnext.H3, Bnext.L3);
            if (i == 4) unpack_pair(R.q2, sc.sc_hi, Bnext.H4, Bnext.L4, Bnext.H5, Bnext.L5);
            if (i == 6) unpack_pair(R.q3, sc.sc_hi >> 16, Bnext.H6, Bnext.L6, Bnext.H7, Bnext.L7);
            if (i == 8) unpack_rest(R, sc, lg_next, Bnext);
        });
        if (c_count > 32) multiply_half(st + L::A_HALF, accF1, B, NothingBetween());
        if (++c_kb == nb) {
            pending = c_ord++;
            pending_count = c_count;
            c_kb = 0;
        }
    };
    // a finished item's results are stored at the top of the next step: a store counts in vmcnt like
    // a load, and there it has the whole step before the wait at the step's end
    auto store_item = [&](int ord) {  // a lane holds one weight row and 16 rows of the tile
        int t, m, rg;
        item_of(ord, t, m, rg);
        const int count = pending_count;
        const int l = opaque_lane(), li = l & 31, lg = l >> 5;
        const int row = rg * (32 * L::RG) + wave * 32 + li;
        int rows = g.rows;
        asm volatile("" : "+s"(rows));  // opaque: keeps the 16 row offsets from being hoisted out of the loop and held
        float *y = (m ? g.y[1] : g.y[0]) + (size_t)t * MOE_TILE * rows;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int tok = (r >> 2) * 8 + lg * 4 + (r & 3);
            if (row < rows && tok < count) y[(uint32_t)(tok * rows + row)] = accF0[r];
        }
        accF0 = v16f{0.0f};
        if (count > 32) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int tok = 32 + (r >> 2) * 8 + lg * 4 + (r & 3);
                if (row < rows && tok < count) y[(uint32_t)(tok * rows + row)] = accF1[r];
            }
            accF1 = v16f{0.0f};
        }
    };

    {  // step 0's weights into the first set; its stage is refilled at once
        const RawBlock R = raw_of_step(0);
        unpack_block(R, lg, B0);
        if (total_steps > 2) {
            fetch_acts();
            fetch_weights();
        }
    }
    auto step = [&](int s, const BPlanes &Bcur, BPlanes &Bnext) {
        if (pending >= 0) {
            store_item(pending);
            pending = -1;
        }
        // step s+1's raw weights leave LDS, which frees their stage for step s+3 (past the last step:
        // whatever the stage holds, unpacked into a set nobody will use)
        const RawBlock R = raw_of_step(s + 1);
        // A wavefront is stalled while its loads wait for the CU's one address unit (600 clocks for
        // the first four wavefronts that ask, 1700 for the other four): so half of the wavefronts,
        // one of every SIMD's two, fetch before they multiply and half after, and the unit serves
        // the one half while the other half has the matrix cores.
        const bool more = s + 3 < total_steps;
        if (more && !fetch_late) {
            fetch_acts();  // (into the stage last read in step s-1)
            fetch_weights();
        }
        multiply_step(s, Bcur, R, Bnext);
        if (more && fetch_late) {
            fetch_acts();
            fetch_weights();
        }
        // steps s+1 and s+2 must have landed; the request just made (step s+3, the `issued` youngest
        // loads; a finished item's stores are older) may stay in flight
        if (!more) wait_vm<0>();
        else if (issued == 6) wait_vm<6>();
        else if (issued == 7) wait_vm<7>();
        else wait_vm<8>();
        lds_barrier();
    };
    for (int s = 0; s < total_steps; s += 2) {
        step(s, B0, B1);
        if (s + 1 < total_steps) step(s + 1, B1, B0);
    }
    if (pending >= 0) store_item(pending);
}

// ------------------------------------------------------------------ launchers

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

template <int RG, int WT, int MT, int WS>
static int launch_variant(const GemmArgs &g, unsigned grid, hipStream_t s) {
    constexpr size_t shmem = GemmLds<RG, WT, MT, WS>::BYTES;
    static_assert(shmem <= 160 * 1024, "LDS of a CU");
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (shmem > 65536 && !sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4_k_mfma_kernel<RG, WT, MT, WS>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(LDS %zu): %s", shmem, hipGetErrorString(e));
        sized = true;
    }
    hipLaunchKernelGGL((gemm_q4_k_mfma_kernel<RG, WT, MT, WS>), dim3(grid, (unsigned)g.k_split), dim3(64 * RG * WT), shmem, s, g);
    FRK_LAUNCH_CHECK("gemm_q4_k_mfma");
    if (g.k_split > 1) return launch_sum_parts(g.partial, g.k_split, (size_t)g.M * g.rows, g.y, s);
    return FRK_OK;
}

// ---- the tiled activations ----
static size_t tiled_records(size_t rows, size_t cols) { return (rows + 31) / 32 * (cols / QK_K); }
size_t q8k_tiled_bytes(size_t rows, size_t cols) {
    // the scales end with slack: a wavefront fetches 64 of them where 32 are used
    return tiled_records(rows, cols) * (8192 + 1024 + 128) + 256;
}
Q8KTiled q8k_tiled_carve(void *base, size_t rows, size_t cols) {
    const size_t rec = tiled_records(rows, cols);
    Q8KTiled a;
    a.q = (int8_t *)base;
    a.bs = (_Float16 *)((char *)base + rec * 8192);
    a.d = (float *)((char *)base + rec * (8192 + 1024));
    return a;
}
template <int WAVES>
static int launch_quantize_records(const float *x, size_t rows, size_t nb, const int *gather, size_t n_rec, Q8KTiled out,
                                   hipStream_t s) {
    hipLaunchKernelGGL((quantize_q8_k_tiled_kernel<WAVES>), dim3((unsigned)n_rec), dim3(64 * WAVES), 0, s, x, (int)rows,
                       (int)nb, gather, out);
    FRK_LAUNCH_CHECK("quantize_q8_k_tiled");
    return FRK_OK;
}
int launch_quantize_q8_k_tiled(const float *x, size_t rows, size_t cols, Q8KTiled out, hipStream_t s) {
    const size_t nb = cols / QK_K, n_rec = (rows + 31) / 32 * nb;
    if (n_rec == 0) return FRK_OK;
    return n_rec <= 1024 ? launch_quantize_records<16>(x, rows, nb, nullptr, n_rec, out, s)
                         : launch_quantize_records<4>(x, rows, nb, nullptr, n_rec, out, s);
}
int launch_quantize_q8_k_gather(const float *x, size_t cols, const int *gather, size_t max_rows, Q8KTiled out,
                                hipStream_t s) {
    const size_t nb = cols / QK_K, n_rec = max_rows / 32 * nb;
    if (n_rec == 0) return FRK_OK;
    return n_rec <= 1024 ? launch_quantize_records<16>(x, 0, nb, gather, n_rec, out, s)
                         : launch_quantize_records<4>(x, 0, nb, gather, n_rec, out, s);
}

constexpr int Q4K_MAX_SPLIT = 4;
// The workgroup tile of a batch: 256 rows x 128 or 64 tokens when that still gives (about) every CU a
// workgroup, else 128 rows x 64 or 32 tokens -- and with those small tiles, when the grid fills few of
// the CUs, a row's blocks split between 2 or 4 workgroups (no finer than four blocks each) whose sums
// are added in order afterwards.
struct Q4KPlan {
    int rows_wg, tok_wg, k_split;
};
static Q4KPlan q4_k_plan(size_t rows, size_t M, size_t nb) {
    if (M > 64 && ((rows + 255) / 256) * ((M + 127) / 128) >= 200) return {256, 128, 1};
    if (M > 64 && ((rows + 255) / 256) * ((M + 63) / 64) >= 256) return {256, 64, 1};
    const int tm = M > 32 ? 64 : 32;
    const size_t grid = (((rows + 127) / 128 + 7) / 8 * 8) * ((M + (size_t)tm - 1) / (size_t)tm);
    int ks = 1;
    while (ks < Q4K_MAX_SPLIT && grid * (size_t)ks * 2 <= 256 && nb / (size_t)(ks * 2) >= 4) ks *= 2;
    return {128, tm, ks};
}
// the tiled activations, then room for the parts' sums where the blocks are split
size_t gemm_q4_k_workspace_bytes(size_t M, size_t cols, size_t rows) {
    const Q4KPlan p = q4_k_plan(rows, M, cols / QK_K);
    return round_up(q8k_tiled_bytes(M, cols), 256) + (p.k_split > 1 ? (size_t)p.k_split * M * rows * sizeof(float) : 0);
}

int launch_gemm_q4_k(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s) {
    // the kernel addresses the weights and the tiled activations with 32-bit byte offsets
    if ((uint64_t)w->rows * w->layout.row_stride >= (1ull << 32) || (uint64_t)q8k_tiled_bytes(M, w->cols) >= (1ull << 32))
        return set_error(FRK_ERR_SHAPE, "gemm_q4_k: %zu x %zu weights with %zu activation rows exceed 4 GiB per operand", w->rows,
                         w->cols, M);
    GemmArgs g;
    g.a = q8k_tiled_carve(ws, M, w->cols);
    int rc = launch_quantize_q8_k_tiled(x, M, w->cols, g.a, s);
    if (rc) return rc;
    g.W = w->dev;
    g.row_stride = w->layout.row_stride;
    g.rows = (int)w->rows;
    g.nb = (int)(w->cols / QK_K);
    g.M = (int)M;
    g.y = y;
    g.k_split = 1;
    g.partial = reinterpret_cast<float *>((char *)ws + round_up(q8k_tiled_bytes(M, w->cols), 256));
    const Q4KPlan p = q4_k_plan(w->rows, M, (size_t)g.nb);
    g.row_tiles = (int)((w->rows + p.rows_wg - 1) / p.rows_wg);
    g.tok_tiles = (int)((M + p.tok_wg - 1) / p.tok_wg);
    g.k_split = p.k_split;
    const unsigned grid = (unsigned)((g.row_tiles + 7) / 8 * 8 * g.tok_tiles);
    if (p.rows_wg == 256) return p.tok_wg == 128 ? launch_variant<8, 1, 4, 2>(g, grid, s) : launch_variant<8, 1, 2, 2>(g, grid, s);
    if (p.tok_wg == 64) return launch_variant<4, 2, 1, 4>(g, grid, s);
    return launch_variant<4, 1, 1, 2>(g, grid, s);
}

int launch_gemm_q4_k_stream(const frk_weights *w0, const frk_weights *w1, size_t rows_e, Q8KTiled a,
                            const int4 *tiles, const int *n_tiles, int max_tiles, float *y0, float *y1,
                            hipStream_t s) {
    StreamArgs g;
    g.W[0] = w0->dev;
    g.W[1] = w1 ? w1->dev : w0->dev;
    g.y[0] = y0;
    g.y[1] = y1;
    g.n_mat = w1 ? 2 : 1;
    g.row_stride = w0->layout.row_stride;
    g.rows = (int)rows_e;
    g.nb = (int)(w0->cols / QK_K);
    g.a = a;
    g.tiles = tiles;
    g.n_tiles = n_tiles;
    g.row_tiles = (int)((rows_e + 255) / 256);
    static int grid = 0;
    if (grid == 0) {
        int dev = 0, cus = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4_k_stream_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)StreamLds::BYTES);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "gemm_q4_k_stream setup: %s", hipGetErrorString(e));
        grid = cus < 8 ? 8 : cus / 8 * 8;  // one workgroup per CU, a multiple of the 8 XCDs
    }
    // more workgroups than CUs when a workgroup's share of the largest possible list would not fit
    // its item table
    const size_t most_items = ((size_t)max_tiles + 7) / 8 * g.n_mat * g.row_tiles;
    const unsigned rounds = (unsigned)((most_items + (size_t)(grid / 8) * StreamLds::MAX_ITEMS - 1) /
                                       ((size_t)(grid / 8) * StreamLds::MAX_ITEMS));
    hipLaunchKernelGGL(gemm_q4_k_stream_kernel, dim3((unsigned)grid * (rounds ? rounds : 1)), dim3(64 * StreamLds::RG),
                       StreamLds::BYTES, s, g);
    FRK_LAUNCH_CHECK("gemm_q4_k_stream");
    return FRK_OK;
}

}  // namespace frk
