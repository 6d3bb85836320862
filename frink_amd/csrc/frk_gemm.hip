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
    float *y[2];  // row (tile's first row of y + r) x [rows]: tile row r
    int n_mat;
    size_t row_stride;
    int rows, nb;  // of one expert
    Q8KTiled a;
    const int4 *tiles;  // {expert, first row of the grouped order, rows in use, first row of y}
    const int *n_tiles;
    int row_tiles;  // ceil(rows / 256)
    // the gathering form: the activations are the source rows' Q8_K, quantized once each, and row r of the
    // grouped order is source row gather[r] (negative: a row not in use)
    Q8KRows src;
    const int *gather;
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
// Q5_K: the same block with a fifth bit per weight -- byte l of the 32 bytes behind the header holds weight l of
// every sub-block, sub-block j in bit j (dot_q5_k_q8, crates/frink-quant/src/lib.rs:886-938); fh is the lane's
// 16-byte half of them.  With q5 = q4 + 16 * bit the scaled weight is sc * q5 = 8 * H + L + 16 * P for a third
// int8 plane P = sc * bit (0 .. 63): three chains of MFMAs, S1 = 8 * (2 * acc_P + acc_H) + acc_L.
struct FifthBits {
    v4i fh;
};
struct PPlanes {
    v4i P0, P1, P2, P3, P4, P5, P6, P7;
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
__device__ __forceinline__ void read_fifth(FifthBits &F, uint32_t addr) { FRK_DS_READ(F.fh, addr, 0); }
template <int N>
__device__ __forceinline__ void wait_raw5(RawBlock &R, FifthBits &F) {
    asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(R.wh), "+v"(R.q0), "+v"(R.q1), "+v"(R.q2), "+v"(R.q3), "+v"(F.fh) : "n"(N));
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

// the third plane of Q5_K: sub-block j's scale where the weight's fifth bit is set (bytes 0 or sc <= 63)
__device__ __forceinline__ void unpack_fifth(const RawBlock &R, const FifthBits &F, PPlanes &P) {
    const BlockScales s = block_scales(R);
    auto plane = [&](int j) {
        const unsigned short sc = (unsigned short)(((j < 4 ? s.sc_lo : s.sc_hi) >> (8 * (j & 3))) & 0xff);
        const us2 scs = {sc, sc};
        v4i o;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t bits = ((uint32_t)F.fh[c] >> j) & 0x01010101u;
            us2 b;
            __builtin_memcpy(&b, &bits, 4);
            const us2 r = b * scs;  // 0x0101 * sc: both bytes sc, no carry between them
            int ri;
            __builtin_memcpy(&ri, &r, 4);
            o[c] = ri;
        }
        return o;
    };
    P.P0 = plane(0), P.P1 = plane(1), P.P2 = plane(2), P.P3 = plane(3);
    P.P4 = plane(4), P.P5 = plane(5), P.P6 = plane(6), P.P7 = plane(7);
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
// shares the gaps of the chain, every MFMA of which waits for the one before it.  It must not branch:
// hipcc counts the wait states between an MFMA and a vector instruction that reads its result within
// one basic block only, and a branch between MFMA 7 and the shift of its sums left the shift three
// instructions behind the MFMA (the last two registers of the sums were read before they were written).
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

// The dense kernel's form of a tile's float step, one accumulator less: the mins' MFMA adds onto the
// converted integer sums instead of into registers of its own.  With d' = d / (-dmin):
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
// ---------------------------------------------------------------------------------------------
// The dense kernel in its pipelined form.
//
// What bounds a SIMD here is its one issue port, not the matrix core alone: measured on this part, a
// v_mfma_i32_32x32x32_i8 keeps the matrix core 32 clocks but costs the SIMD about 20 clocks in which no
// vector instruction issues, and every vector instruction another 2.6 -- whichever wavefront they come
// from.  About five vector instructions fit between two MFMAs for free; a tile (16 + 1 MFMAs) has ~80
// of epilogue.  So the epilogue of tile t-1 is cut into sixteen pieces that ride in the gaps of tile
// t's chain of MFMAs, the address arithmetic of the prefetch is scalar (global_load_lds with a scalar
// base and lane offsets that are computed once), and what stays exposed is the unpacking of the
// next block and the last tile's epilogue.
//
// A workgroup = 8 wavefronts = RG row groups of 32 weight rows x KS shares of the blocks; a wavefront
// runs MT 32-token tiles against its rows' current block.  KS = 2 (small matrices: 128 rows x 64 tokens
// per workgroup fill the chip where 256 x 128 would not) halves the blocks between two wavefronts whose
// sums are added through LDS at the end, always the first half's plus the second half's.
//
// LDS: activations in a ring of 3 stages (requested two steps ahead), their scales in a ring of 4
// (they are read by an epilogue that may run a step later), the raw weights in ONE slot per
// wavefront: a block leaves its slot for registers at the end of the step before it is multiplied,
// and the slot is refilled at once.  One barrier per step.
template <int RG, int KS, int MT, bool Q5 = false>
struct PipeLds {
    static constexpr int BB = Q5 ? Q5_K_BYTES : Q4_K_BYTES;  // bytes of a weight block
    static constexpr int NW = RG * KS;
    static constexpr int NT = KS * MT;  // tile slots of a stage
    static constexpr int OFF_BS = NT * 8192;
    static constexpr int A_STAGE = NT * 9216;  // quants [NT][8 slices][1 KB] | sums f16 [NT][1 KB]
    static constexpr int A_STAGES = 3;
    static constexpr int OFF_DA = A_STAGES * A_STAGE;
    static constexpr int DA_STAGE = NT * 128, DA_STAGES = 4;
    static constexpr int OFF_W = OFF_DA + DA_STAGES * DA_STAGE;
    static constexpr int W_SLOT = 32 * BB;
    static constexpr size_t BYTES = (size_t)OFF_W + (size_t)NW * W_SLOT;
};

template <int OFF>
__device__ __forceinline__ void ds_read16(v4i &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void ds_read16(v8h &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void ds_read16(v4f &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
// tile slot SLOT of a stage: its eight k-slices and its sums (nine reads, in this order)
template <int SLOT>
__device__ __forceinline__ void read_tile(TileOperands &T, uint32_t qa, uint32_t ba) {
    ds_read16<SLOT * 8192 + 0>(T.a0, qa);
    ds_read16<SLOT * 8192 + 1024>(T.a1, qa);
    ds_read16<SLOT * 8192 + 2048>(T.a2, qa);
    ds_read16<SLOT * 8192 + 3072>(T.a3, qa);
    ds_read16<SLOT * 8192 + 4096>(T.a4, qa);
    ds_read16<SLOT * 8192 + 5120>(T.a5, qa);
    ds_read16<SLOT * 8192 + 6144>(T.a6, qa);
    ds_read16<SLOT * 8192 + 7168>(T.a7, qa);
    ds_read16<SLOT * 1024>(T.bs, ba);
}
// operand J (0..7) of tile slot SLOT
template <int SLOT, int J>
__device__ __forceinline__ void read_tile_operand(TileOperands &T, uint32_t qa) {
    v4i &dst = J == 0 ? T.a0 : J == 1 ? T.a1 : J == 2 ? T.a2 : J == 3 ? T.a3 : J == 4 ? T.a4 : J == 5 ? T.a5 : J == 6 ? T.a6 : T.a7;
    ds_read16<SLOT * 8192 + J * 1024>(dst, qa);
}
template <int SLOT>
__device__ __forceinline__ void read_tile_sums(TileOperands &T, uint32_t ba) {
    ds_read16<SLOT * 1024>(T.bs, ba);
}
template <int SLOT>
__device__ __forceinline__ void read_tile_scales(TileScales &S, uint32_t sa) {
    ds_read16<SLOT * 128 + 0>(S.da0, sa);
    ds_read16<SLOT * 128 + 32>(S.da1, sa);
    ds_read16<SLOT * 128 + 64>(S.da2, sa);
    ds_read16<SLOT * 128 + 96>(S.da3, sa);
}

// The sixteen integer MFMAs of a tile.  Its operands were requested in the order a0..a7, sums, and then
// EXTRA more LDS reads; each MFMA waits only for its own operand.  between(i) runs after MFMA i has been
// issued; from MFMA 8 on operand a(i-8) has been read for the last time, and next(i-8) may request the
// next tile's into its place.
template <int N, class V>
__device__ __forceinline__ void wait_lgkm(V &reg, v16i &acc) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(reg), "+v"(acc) : "n"(N));
}
// (Q5_K: the chain of the fifth bits' plane runs first, each of its MFMAs waiting for its operand; the sum is
// doubled and the two chains below follow with every operand there.)
template <int EXTRA>
__device__ __forceinline__ v16i fifth_chain(TileOperands &T, const PPlanes &P) {
    const v16i zi = {0};
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(T.a0) : "n"(8 + EXTRA));
    v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, P.P0, zi, 0, 0, 0);
    wait_lgkm<7 + EXTRA>(T.a1, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, P.P1, acc, 0, 0, 0);
    wait_lgkm<6 + EXTRA>(T.a2, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, P.P2, acc, 0, 0, 0);
    wait_lgkm<5 + EXTRA>(T.a3, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, P.P3, acc, 0, 0, 0);
    wait_lgkm<4 + EXTRA>(T.a4, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, P.P4, acc, 0, 0, 0);
    wait_lgkm<3 + EXTRA>(T.a5, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, P.P5, acc, 0, 0, 0);
    wait_lgkm<2 + EXTRA>(T.a6, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, P.P6, acc, 0, 0, 0);
    wait_lgkm<1 + EXTRA>(T.a7, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, P.P7, acc, 0, 0, 0);
    return acc << 1;
}
// SEEDED: the running sum starts from `seed` (the doubled sum of the fifth bits' chain) and every operand has
// landed already.
template <int EXTRA, bool SEEDED = false, class Between, class Next>
__device__ __forceinline__ v16i tile_chain(TileOperands &T, const BPlanes &B, Between between, Next next, v16i seed = v16i{0}) {
    const v16i zi = seed;
    if (!SEEDED) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(T.a0) : "n"(8 + EXTRA));
    v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.H0, zi, 0, 0, 0);
    between(0);
    wait_lgkm<7 + EXTRA>(T.a1, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.H1, acc, 0, 0, 0);
    between(1);
    wait_lgkm<6 + EXTRA>(T.a2, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.H2, acc, 0, 0, 0);
    between(2);
    wait_lgkm<5 + EXTRA>(T.a3, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.H3, acc, 0, 0, 0);
    between(3);
    wait_lgkm<4 + EXTRA>(T.a4, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.H4, acc, 0, 0, 0);
    between(4);
    wait_lgkm<3 + EXTRA>(T.a5, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.H5, acc, 0, 0, 0);
    between(5);
    wait_lgkm<2 + EXTRA>(T.a6, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.H6, acc, 0, 0, 0);
    between(6);
    wait_lgkm<1 + EXTRA>(T.a7, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.H7, acc, 0, 0, 0);
    between(7);
    wait_lgkm<0>(T.bs, acc);  // (and the EXTRA reads behind the sums)
    acc = acc << 3;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.L0, acc, 0, 0, 0);
    next(0);
    between(8);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.L1, acc, 0, 0, 0);
    next(1);
    between(9);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.L2, acc, 0, 0, 0);
    next(2);
    between(10);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.L3, acc, 0, 0, 0);
    next(3);
    between(11);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.L4, acc, 0, 0, 0);
    next(4);
    between(12);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.L5, acc, 0, 0, 0);
    next(5);
    between(13);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.L6, acc, 0, 0, 0);
    next(6);
    between(14);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.L7, acc, 0, 0, 0);
    next(7);
    between(15);
    return acc;
}

// A finished tile's way into the float sums (the arithmetic fold_mins prepares), in sixteen pieces:
//   pieces 0..7   c[r] = d' * float(S1[r]) for two results each,
//   piece  7      then the mins' MFMA adds S2 onto c,
//   pieces 8..15  sum[r] += (da[r] * -dmin) * c[r] for two results each.
struct TileTail {
    v16i s1;      // the integer sums
    v16f c;       // d' * S1, then + S2
    v8h bs;       // the tile's 16-wide activation sums
    TileScales S; // the tile's activation scales
};
__device__ __forceinline__ void tail_piece(int i, TileTail &E, const BPlanes &B, v16f &sum) {
    if (i < 8) {
        E.c[2 * i] = B.d * (float)E.s1[2 * i];
        E.c[2 * i + 1] = B.d * (float)E.s1[2 * i + 1];
        if (i == 7) E.c = __builtin_amdgcn_mfma_f32_32x32x16_f16(E.bs, B.m, E.c, 0, 0, 0);
    } else {
        const v4f dav[4] = {E.S.da0, E.S.da1, E.S.da2, E.S.da3};
#pragma unroll
        for (int r = 2 * (i - 8); r < 2 * (i - 8) + 2; r++) sum[r] = fmaf(dav[r >> 2][r & 3] * B.ndmin, E.c[r], sum[r]);
    }
}

// Up to four pieces of 1 KB that lie 1 KB apart in LDS and whose lane offsets already carry the matching
// distance in global memory: a request's instruction offset moves BOTH of its addresses (checked on the
// device), so one write of M0 serves the four.  `lds_uniform` and `base_uniform` must be scalar values.
template <int N>
__device__ __forceinline__ void dma16_run(uint32_t lds_uniform, const void *base_uniform, uint32_t o0, uint32_t o1, uint32_t o2,
                                          uint32_t o3) {
    static_assert(N >= 1 && N <= 4, "the instruction offset reaches 3072");
    if (N == 4)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %5\n\tglobal_load_lds_dwordx4 %2, %5 offset:1024\n\t"
                     "global_load_lds_dwordx4 %3, %5 offset:2048\n\tglobal_load_lds_dwordx4 %4, %5 offset:3072"
                     :
                     : "s"(lds_uniform), "v"(o0), "v"(o1), "v"(o2), "v"(o3), "s"(base_uniform)
                     : "memory");
    else if (N == 2)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %3\n\tglobal_load_lds_dwordx4 %2, %3 offset:1024"
                     :
                     : "s"(lds_uniform), "v"(o0), "v"(o1), "s"(base_uniform)
                     : "memory");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_uniform), "v"(o0), "s"(base_uniform) : "memory");
}

// The block's scales as the packed multiply wants them: for sub-block j one register with sh_j = sc_j >> 3 in
// its low half and sl_j = sc_j & 7 in its high half.  The multiply picks a half for both of its 16-bit lanes
// through op_sel, so nothing has to be replicated.
struct ScalePairs {
    uint32_t p0, p1, p2, p3, p4, p5, p6, p7;
};
__device__ __forceinline__ ScalePairs scale_pairs(const BlockScales &s) {
    const uint32_t sh_lo = (s.sc_lo >> 3) & 0x07070707u, sl_lo = s.sc_lo & 0x07070707u;
    const uint32_t sh_hi = (s.sc_hi >> 3) & 0x07070707u, sl_hi = s.sc_hi & 0x07070707u;
    // v_perm_b32: selector bytes 0..3 take the second operand's bytes, 4..7 the first's, 0x0c gives zero
    ScalePairs r;
    r.p0 = __builtin_amdgcn_perm(sl_lo, sh_lo, 0x0c040c00u);
    r.p1 = __builtin_amdgcn_perm(sl_lo, sh_lo, 0x0c050c01u);
    r.p2 = __builtin_amdgcn_perm(sl_lo, sh_lo, 0x0c060c02u);
    r.p3 = __builtin_amdgcn_perm(sl_lo, sh_lo, 0x0c070c03u);
    r.p4 = __builtin_amdgcn_perm(sl_hi, sh_hi, 0x0c040c00u);
    r.p5 = __builtin_amdgcn_perm(sl_hi, sh_hi, 0x0c050c01u);
    r.p6 = __builtin_amdgcn_perm(sl_hi, sh_hi, 0x0c060c02u);
    r.p7 = __builtin_amdgcn_perm(sl_hi, sh_hi, 0x0c070c03u);
    return r;
}
// bytes of `nib` (each below 16) times the low (H) and the high (L) half of `pair`: bytes stay below 106
__device__ __forceinline__ void scaled_planes(uint32_t nib, uint32_t pair, int &h, int &l) {
    asm("v_pk_mul_lo_u16 %0, %1, %2 op_sel_hi:[1,0]" : "=v"(h) : "v"(nib), "v"(pair));
    asm("v_pk_mul_lo_u16 %0, %1, %2 op_sel:[0,1] op_sel_hi:[1,1]" : "=v"(l) : "v"(nib), "v"(pair));
}
__device__ __forceinline__ void unpack_pair_sel(const v4i q, uint32_t pair0, uint32_t pair1, v4i &H0, v4i &L0, v4i &H1, v4i &L1) {
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const uint32_t w = (uint32_t)q[c];
        int h0, l0, h1, l1;
        scaled_planes(w & 0x0f0f0f0fu, pair0, h0, l0);
        scaled_planes((w >> 4) & 0x0f0f0f0fu, pair1, h1, l1);
        H0[c] = h0, L0[c] = l0, H1[c] = h1, L1[c] = l1;
    }
}
// The same in plain vector arithmetic (the compiler finds the op_sel forms itself), for a kernel that leaves
// the place of the unpacking to the compiler: statements of inline assembly stay where they are written.
__device__ __forceinline__ void unpack_pair_free(const v4i q, uint32_t pair0, uint32_t pair1, v4i &H0, v4i &L0, v4i &H1, v4i &L1) {
    us2 p0, p1;
    __builtin_memcpy(&p0, &pair0, 4);
    __builtin_memcpy(&p1, &pair1, 4);
    const us2 h0 = {p0.x, p0.x}, l0 = {p0.y, p0.y}, h1 = {p1.x, p1.x}, l1 = {p1.y, p1.y};
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const uint32_t w = (uint32_t)q[c];
        const uint32_t nl = w & 0x0f0f0f0fu, nh = (w >> 4) & 0x0f0f0f0fu;
        us2 a, b;
        __builtin_memcpy(&a, &nl, 4);
        __builtin_memcpy(&b, &nh, 4);
        const us2 r0 = a * h0, r1 = a * l0, r2 = b * h1, r3 = b * l1;  // bytes stay below 106
        int o0, o1, o2, o3;
        __builtin_memcpy(&o0, &r0, 4);
        __builtin_memcpy(&o1, &r1, 4);
        __builtin_memcpy(&o2, &r2, 4);
        __builtin_memcpy(&o3, &r3, 4);
        H0[c] = o0, L0[c] = o1, H1[c] = o2, L1[c] = o3;
    }
}
__device__ __forceinline__ void unpack_block_sel(const RawBlock &R, int lg, BPlanes &B) {
    const BlockScales s = block_scales(R);
    const ScalePairs p = scale_pairs(s);
    unpack_pair_sel(R.q0, p.p0, p.p1, B.H0, B.L0, B.H1, B.L1);
    unpack_pair_sel(R.q1, p.p2, p.p3, B.H2, B.L2, B.H3, B.L3);
    unpack_pair_sel(R.q2, p.p4, p.p5, B.H4, B.L4, B.H5, B.L5);
    unpack_pair_sel(R.q3, p.p6, p.p7, B.H6, B.L6, B.H7, B.L7);
    unpack_rest(R, s, lg, B);
}

// The chain of a tile with its operands released two at a time (half as many waits as tile_chain, which the
// Q5_K form keeps): the reads were requested in the order a0..a7, sums, and EXTRA more behind them.
template <int N, class V>
__device__ __forceinline__ void wait_lgkm2(V &r0, V &r1, v16i &acc) {
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(r0), "+v"(r1), "+v"(acc) : "n"(N));
}
template <int EXTRA, class Between, class Next>
__device__ __forceinline__ v16i tile_chain_pairs(TileOperands &T, const BPlanes &B, Between between, Next next) {
    const v16i zi = {0};
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(T.a0), "+v"(T.a1) : "n"(7 + EXTRA));
    v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.H0, zi, 0, 0, 0);
    between(0);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.H1, acc, 0, 0, 0);
    between(1);
    wait_lgkm2<5 + EXTRA>(T.a2, T.a3, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.H2, acc, 0, 0, 0);
    between(2);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.H3, acc, 0, 0, 0);
    between(3);
    wait_lgkm2<3 + EXTRA>(T.a4, T.a5, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.H4, acc, 0, 0, 0);
    between(4);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.H5, acc, 0, 0, 0);
    between(5);
    wait_lgkm2<1 + EXTRA>(T.a6, T.a7, acc);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.H6, acc, 0, 0, 0);
    between(6);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.H7, acc, 0, 0, 0);
    between(7);
    wait_lgkm<0>(T.bs, acc);  // (and the EXTRA reads behind the sums)
    acc = acc << 3;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, B.L0, acc, 0, 0, 0);
    between(8);
    next(0);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, B.L1, acc, 0, 0, 0);
    next(1);
    between(9);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, B.L2, acc, 0, 0, 0);
    next(2);
    between(10);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, B.L3, acc, 0, 0, 0);
    next(3);
    between(11);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a4, B.L4, acc, 0, 0, 0);
    next(4);
    between(12);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a5, B.L5, acc, 0, 0, 0);
    next(5);
    between(13);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a6, B.L6, acc, 0, 0, 0);
    next(6);
    between(14);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a7, B.L7, acc, 0, 0, 0);
    next(7);
    between(15);
    return acc;
}

template <int RG, int KS, int MT, bool Q5 = false>
__global__ __launch_bounds__(512) void gemm_q4_k_pipe_kernel(GemmArgs g) {
    using L = PipeLds<RG, KS, MT, Q5>;
    constexpr int BB = L::BB, PR = BB / 16;          // bytes of a block, its 16-byte pieces
    constexpr int NC = (32 * PR + 63) / 64;          // requests that move a wavefront's 32 rows of a block (the last: half)
    static_assert(32 * PR == 64 * (NC - 1) + 32, "the last request of a block is 32 lanes wide");
    static_assert(NC == 5 || NC == 6, "four requests share one write of M0, the rest follow");
    constexpr int NW = L::NW, NT = L::NT, ROWS = 32 * RG, TM = 32 * MT;
    static_assert(NW == 8 && NT == 4 && (MT == 2 || MT == 4), "eight wavefronts share the four tile slots of a stage");
    extern __shared__ uint4 smem_gemm[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem_gemm);
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_address(lds));
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lg = lane >> 5;
    const int rg = wave % RG, ks = wave / RG;

    // workgroups that share weight rows (different token tiles) sit on one XCD (block id mod 8)
    const int bid = blockIdx.x;
    const int per_group = 8 * g.tok_tiles;
    const int grp = bid / per_group, in_grp = bid % per_group;
    const int row_tile = grp * 8 + (in_grp & 7);
    if (row_tile >= g.row_tiles) return;  // uniform per workgroup
    const int tok0 = (in_grp >> 3) * TM;
    const int nb = g.nb;
    // this workgroup multiplies blocks kb0 .. kb1 - 1, its KS shares `steps` consecutive ones each (a
    // share that runs out of blocks idles through its last steps)
    const int kb0 = nb * (int)blockIdx.y / g.k_split, kb1 = nb * ((int)blockIdx.y + 1) / g.k_split;
    const int steps = (kb1 - kb0 + KS - 1) / KS;
    const int tile0 = tok0 / 32, last_tile = (g.M - 1) / 32;
    auto tile_of = [&](int slot) { return min(tile0 + slot % MT, last_tile); };  // uniform

    // ---- the fetch side.  Every address is a scalar pointer that moves on by one block a step plus a lane
    // offset that never changes, and a stage of the rings is a scalar offset that rotates: a step's requests
    // cost a handful of scalar instructions.  The first four wavefronts -- the ones the SIMDs' arbiters
    // favour (they are the older of each SIMD's two), which otherwise wait at the step's barrier for the
    // other four -- fetch the activations: wavefront f the record of tile slot f (8 KB of quants, 1 KB of
    // sums), wavefronts 0 and 1 the scales of two slots each.  Every wavefront fetches its own weight rows.
    const bool fetches_acts = wave < NT;
    const bool fetches_scales = wave < 2;
    const uint32_t lane16 = (uint32_t)lane * 16;
    const int slot_f = wave & 3, slot_d = (wave & 1) * 2;
    // (a share past its last block keeps requesting that block: nobody multiplies it)
    int next_kb_a = kb0 + (slot_f / MT) * steps;  // the block of this wavefront's activation slot at the next request
    int next_kb_d = kb0 + (slot_d / MT) * steps;
    int next_kb_w = kb0 + ks * steps;
    const uint8_t *src_q = (const uint8_t *)scalar_pointer(reinterpret_cast<const uint8_t *>(g.a.q) +
                                                           ((size_t)tile_of(slot_f) * nb + min(next_kb_a, kb1 - 1)) * 8192);
    const uint8_t *src_s = (const uint8_t *)scalar_pointer(reinterpret_cast<const uint8_t *>(g.a.bs) +
                                                           ((size_t)tile_of(slot_f) * nb + min(next_kb_a, kb1 - 1)) * 1024);
    const uint8_t *src_d = (const uint8_t *)scalar_pointer(reinterpret_cast<const uint8_t *>(g.a.d) +
                                                           ((size_t)tile_of(slot_d) * nb + min(next_kb_d, kb1 - 1)) * 128);
    const uint32_t lane_d = (uint32_t)(lane & 31) * 4 +
                            (lane >= 32 ? (uint32_t)(tile_of(slot_d + 1) - tile_of(slot_d)) * (uint32_t)nb * 128u : 0u);
    // weights: this wavefront's 32 rows x PR sixteen-byte pieces, piece p = 64 * c + lane of chunk c, so that LDS
    // holds the rows back to back.  Rows past the matrix read its last row.  Chunks 1..3 ride on chunk 0's M0
    // with instruction offsets, which move the global address too: their lane offsets are short of it by as
    // much (the pointer is kept 4096 bytes low and every offset 4096 high, so that none goes negative).
    const uint32_t stride = (uint32_t)g.row_stride;
    const int row_base = min(row_tile * ROWS + rg * 32, g.rows - 1);
    uint32_t w_off[NC];
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int p = 64 * c + lane;
        const int r = min(p / PR, g.rows - 1 - row_base);
        w_off[c] = (uint32_t)r * stride + (uint32_t)(p % PR) * 16 + 4096u - (c < 4 ? 1024u * c : 0u);
    }
    const uint8_t *src_w = (const uint8_t *)scalar_pointer(g.W + (size_t)row_base * stride + (size_t)min(next_kb_w, kb1 - 1) * BB - 4096);
    const uint32_t lds_w = lds0 + L::OFF_W + wave * L::W_SLOT;
    // the rings: activations three stages (a step's stage, the next one's, the one being filled), scales four
    uint32_t st_cur = lds0, st_next = lds0 + L::A_STAGE, st_fill = lds0;  // st_fill: where the next request lands
    uint32_t da_fill = lds0 + L::OFF_DA;
    auto fetch_quants = [&](int half) {  // half of the slot's record: 4 KB
        dma16_run<4>(st_fill + slot_f * 8192 + half * 4096, src_q + half * 4096, lane16, lane16, lane16, lane16);
    };
    auto fetch_sums_scales = [&]() {
        dma16_run<1>(st_fill + L::OFF_BS + slot_f * 1024, src_s, lane16, 0, 0, 0);
        if (fetches_scales) dma4(da_fill + slot_d * 128, src_d, lane_d);
    };
    auto acts_fetched = [&]() {  // the request for a step is out: everything moves on to the step after
        const bool adv_a = next_kb_a + 1 < kb1, adv_d = next_kb_d + 1 < kb1;
        next_kb_a++, next_kb_d++;
        src_q += adv_a ? 8192 : 0;
        src_s += adv_a ? 1024 : 0;
        src_d += adv_d ? 128 : 0;
        st_fill = st_fill == lds0 + 2 * L::A_STAGE ? lds0 : st_fill + L::A_STAGE;
        da_fill = da_fill == lds0 + L::OFF_DA + 3 * L::DA_STAGE ? lds0 + L::OFF_DA : da_fill + L::DA_STAGE;
    };
    auto fetch_weights = [&]() {  // NC requests
        dma16_run<4>(lds_w, src_w, w_off[0], w_off[1], w_off[2], w_off[3]);
        if (NC == 6) dma16_run<1>(lds_w + 4096, src_w, w_off[4], 0, 0, 0);
        if (lane < 32) dma16_run<1>(lds_w + (NC - 1) * 1024, src_w, w_off[NC - 1], 0, 0, 0);
        src_w += next_kb_w + 1 < kb1 ? BB : 0;
        next_kb_w++;
    };

    v16f sum[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) sum[mt] = v16f{0.0f};
    BPlanes B;
    PPlanes P;  // (Q5_K only)
    RawBlock R;
    FifthBits F;
    // a raw block leaves this wavefront's slot for registers (Q5_K: the nibbles sit behind the 32 bytes of fifth bits)
    auto read_block = [&]() {
        const uint32_t wa = lds_w + li * BB;
        read_raw(R, wa, wa + (Q5 ? 32 : 0) + 16 * lg);
        if (Q5) {
            read_fifth(F, wa + 16 + 16 * lg);
            wait_raw5<0>(R, F);
        } else {
            wait_raw<0>(R);
        }
    };
    auto unpack = [&]() {
        unpack_block_sel(R, lg, B);
        if (Q5) unpack_fifth(R, F, P);
        fold_mins(B);
    };

    // prologue: activations of steps 0 and 1, weights of step 0; then the weights of step 1
    if (fetches_acts) {
        fetch_quants(0), fetch_quants(1), fetch_sums_scales(), acts_fetched();
    }
    fetch_weights();
    if (steps > 1 && fetches_acts) {
        fetch_quants(0), fetch_quants(1), fetch_sums_scales(), acts_fetched();
    }
    // how many requests of a step's activations this wavefront makes (they stay in flight over the step's end)
    const int acts_requests = fetches_scales ? 10 : fetches_acts ? 9 : 0;
    // where a step's first tile slot of this wavefront's share sits in its stage (lane offsets in)
    const uint32_t rd_q = (uint32_t)(ks * MT) * 8192 + lane16, rd_b = L::OFF_BS + (uint32_t)(ks * MT) * 1024 + lane16;
    const uint32_t rd_d = lds0 + L::OFF_DA + (uint32_t)(ks * MT) * 128 + lg * 16;
    const int my_steps = max(0, min(steps, kb1 - (kb0 + ks * steps)));  // the steps in which this wavefront's share has a block
    TileOperands T;  // the first tile's operands of the step about to run: requested behind the barrier, so that
                     // they travel while the block is unpacked
    wait_vm<0>();
    lds_barrier();
    {
        read_block();
        if (steps > 1) fetch_weights();
        if (my_steps > 0) read_tile<0>(T, st_cur + rd_q, st_cur + rd_b);
        unpack();
    }

    for (int i = 0; i < steps; i++) {
        const bool active = i < my_steps;
        const uint32_t qa = st_cur + rd_q, ba = st_cur + rd_b;
        const uint32_t sa = rd_d + (uint32_t)(i & 3) * L::DA_STAGE;
        const bool more_acts = i + 2 < steps;
        const bool fetch_now = more_acts && fetches_acts;
        if (active) {
            TileOperands Tn;
            TileTail E;
            // One tile after the other; the second half of a tile's chain requests the next tile's operands
            // into the registers it has read for the last time, and carries the tail of the tile before.
            auto run_tile = [&](auto mt_c) {
                constexpr int mt = decltype(mt_c)::value;
                auto between = [&](int j) {
                    if (mt == 0) {
                        if (fetch_now) {
                            if (j == 1) fetch_quants(0);
                            if (j == 3) fetch_quants(1);
                            if (j == 5) fetch_sums_scales(), acts_fetched();
                        }
                    } else {
                        // the scales of the tile before were the last reads requested ahead of this chain:
                        // they have landed once the chain has waited for everything, in front of MFMA 8, and
                        // only from here on may the compiler touch them
                        if (j == 8) wait_scales<0>(E.S);
                        tail_piece(j, E, B, sum[mt > 0 ? mt - 1 : 0]);
                    }
                };
                auto next = [&](int j) {
                    if (mt + 1 < MT) {
                        constexpr int nx = mt + 1 < MT ? mt + 1 : mt;
                        if (j == 0) read_tile_operand<nx, 0>(Tn, qa);
                        if (j == 1) read_tile_operand<nx, 1>(Tn, qa);
                        if (j == 2) read_tile_operand<nx, 2>(Tn, qa);
                        if (j == 3) read_tile_operand<nx, 3>(Tn, qa);
                        if (j == 4) read_tile_operand<nx, 4>(Tn, qa);
                        if (j == 5) read_tile_operand<nx, 5>(Tn, qa);
                        if (j == 6) read_tile_operand<nx, 6>(Tn, qa);
                        if (j == 7) read_tile_operand<nx, 7>(Tn, qa);
                    }
                };
                // (a tile after the first finds four more reads behind its sums: the scales of the tile before)
                constexpr int EXTRA = mt > 0 ? 4 : 0;
                v16i s1;
                if constexpr (Q5) s1 = tile_chain<EXTRA, true>(T, B, between, next, fifth_chain<EXTRA>(T, P));
                else s1 = tile_chain_pairs<EXTRA>(T, B, between, next);
                E.s1 = s1;
                E.bs = T.bs;
                if (mt + 1 < MT) {
                    constexpr int nx = mt + 1 < MT ? mt + 1 : mt;
                    read_tile_sums<nx>(Tn, ba);
                }
                read_tile_scales<mt>(E.S, sa);
                if (mt + 1 < MT) T = Tn;
            };
            run_tile(std::integral_constant<int, 0>());
            if (MT > 1) run_tile(std::integral_constant<int, 1 < MT ? 1 : 0>());
            if (MT > 2) run_tile(std::integral_constant<int, 2 < MT ? 2 : 0>());
            if (MT > 3) run_tile(std::integral_constant<int, 3 < MT ? 3 : 0>());
            // the last tile's tail is exposed
            wait_scales<0>(E.S);
#pragma unroll
            for (int j = 0; j < 16; j++) tail_piece(j, E, B, sum[MT - 1]);
        } else if (fetch_now) {
            fetch_quants(0), fetch_quants(1), fetch_sums_scales(), acts_fetched();
        }
        if (i + 1 < steps) {
            // step i+1's raw weights (requested a step ago) leave their slot, which is refilled at once;
            // the activations of step i+2, younger than they, may stay in flight
            if (!fetch_now) wait_vm<0>();
            else if (acts_requests == 10) wait_vm<10>();
            else wait_vm<9>();
            read_block();
            if (more_acts) fetch_weights();
            lds_barrier();
            st_cur = st_next;
            st_next = st_next == lds0 + 2 * L::A_STAGE ? lds0 : st_next + L::A_STAGE;
            if (i + 1 < my_steps) read_tile<0>(T, st_cur + rd_q, st_cur + rd_b);
            unpack();
        } else {
            lds_barrier();
        }
    }

    // two shares of the blocks: the second half's sums go through LDS and are added onto the first's
    if (KS == 2) {
        float *xch = reinterpret_cast<float *>(lds) + (size_t)rg * MT * 16 * 64;
        if (ks == 1) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int r = 0; r < 16; r++) xch[(mt * 16 + r) * 64 + lane] = sum[mt][r];
        }
        __syncthreads();
        if (ks == 1) return;
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int r = 0; r < 16; r++) sum[mt][r] += xch[(mt * 16 + r) * 64 + lane];
    }
    // store: a lane holds one weight row and 16 tokens per tile
    const int row = row_tile * ROWS + rg * 32 + li;
    float *const dst = g.k_split > 1 ? g.partial + (size_t)blockIdx.y * g.M * g.rows : g.y;
    const int rows_lim = g.rows;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int tok = tok0 + mt * 32 + (r >> 2) * 8 + lg * 4 + (r & 3);
            if (row < rows_lim && tok < g.M) dst[(size_t)tok * g.rows + row] = sum[mt][r];
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
// GATHER: a tile's activation rows are fetched from where their source rows were quantized (plain rows,
// each quantized once however many tiles it is part of) instead of from a record of the grouped order: a
// lane's piece of a record is 16 bytes of one row in either form, so only the lane offsets differ -- the
// source row times the row length, looked up per item from a table in LDS.
template <bool GATHER>
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
    // {expert, rows in use, first row of y} of each of the workgroup's items, filled once: looked up from LDS, an
    // item change costs no global load (whose completion would count in vmcnt, in the middle of the
    // prefetch bookkeeping)
    static constexpr int OFF_ITEMS = OFF_A + A_STAGES * A_STAGE;
    static constexpr int MAX_ITEMS = GATHER ? 64 : 128;
    // GATHER: the source rows of each item's tile, row r of the first half in the low 16 bits of word r and
    // row 32 + r in the high ones
    static constexpr int OFF_SRC = OFF_ITEMS + MAX_ITEMS * 16;
    static constexpr size_t BYTES = (size_t)OFF_SRC + (GATHER ? MAX_ITEMS * 128 : 0);
    static_assert(BYTES <= 160 * 1024, "LDS of a CU");
};

template <bool GATHER>
__global__ __launch_bounds__(512) void gemm_q4_k_stream_kernel(StreamArgs g) {
    using L = StreamLds<GATHER>;
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
        int4 *table = reinterpret_cast<int4 *>(lds + L::OFF_ITEMS);
        for (int i = tid; i < my_items; i += 64 * L::RG) {
            const int4 ti = g.tiles[xcd + 8 * ((slot + i * per_xcd) / per_tile)];
            table[i] = make_int4(ti.x, ti.z, ti.w, 0);
        }
        if (GATHER) {
            uint32_t *src_rows = reinterpret_cast<uint32_t *>(lds + L::OFF_SRC);
            for (int i = tid; i < my_items * 32; i += 64 * L::RG) {
                const int t = xcd + 8 * ((slot + (i >> 5) * per_xcd) / per_tile), r = i & 31;
                const int a = g.gather[t * MOE_TILE + r], b = g.gather[t * MOE_TILE + 32 + r];
                src_rows[i] = (uint32_t)max(a, 0) | ((uint32_t)max(b, 0) << 16);  // (a row not in use: any row will do)
            }
        }
        __syncthreads();
    }
    const uint32_t lds_items = lds_address(lds + L::OFF_ITEMS);
    auto item_info = [&](int ord, int &expert, int &count, int &y_row) {
        v4i v;
        asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_items + ord * 16));
        expert = __builtin_amdgcn_readfirstlane(v.x);
        count = __builtin_amdgcn_readfirstlane(v.y);
        y_row = __builtin_amdgcn_readfirstlane(v.z);
    };

    // ---- the fetch side: a cursor (item, block) three steps ahead of the arithmetic ----
    // weights of a step: this wavefront's 32 rows x 9 sixteen-byte pieces, piece p = 64*c + lane of
    // chunk c (4.5 chunks, 5 loads); activations: quant slice `wave`, plus the sums (wavefront 0) or
    // the scales (wavefront 1).  Addresses are a uniform base that moves with the cursor plus a lane
    // offset that is fixed per item.
    // Per item, kept in registers (recomputing them from the lane number for every request cost ~60 vector
    // instructions a step): the five weight offsets w_off (rows past the matrix, in a last partial row group,
    // fetch the matrix's last piece instead) and the offsets of the activation pieces.
    uint32_t w_off[5] = {0, 0, 0, 0, 0};
    auto opaque_lane = [&]() {  // the lane number as a value the compiler cannot hoist expressions of
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    // activations: quant slice `wave` of each half in use, plus one of the four small pieces: sums
    // (wavefronts 0, 2) and scales (1, 3) of the first (0, 1) and second half (2, 3)
    const bool x_sums = (wave & 1) == 0;
    const bool x_small = wave < 4, x_second = wave >= 2;  // fetches a small piece at all; the second half's
    uint32_t qa_off, qb_off, x_off;
    if (!GATHER) {
        qa_off = (uint32_t)(wave * 1024 + lane * 16);
        qb_off = qa_off + (uint32_t)nb * 8192;
        x_off = x_sums ? (uint32_t)lane * 16 : (uint32_t)(lane & 31) * 4;  // both lane halves fetch the same 32 scales
    }
    const uint8_t *f_w, *f_x;
    const int8_t *f_q;
    const uint32_t lds_src = lds_address(lds + L::OFF_SRC);
    int f_ord = 0, f_kb = 0, f_step = 0;
    bool f_two = false;  // the cursor's tile has rows in its second half
    int issued = 0;      // loads of the fetch most recently issued by this wavefront
    auto point_at = [&](int ord) {  // uniform
        int t, m, rg, expert, count, y_row;
        item_of(ord, t, m, rg);
        item_info(ord, expert, count, y_row);
        f_w = (m ? g.W[1] : g.W[0]) + (size_t)expert * g.rows * g.row_stride;
        const uint32_t stride = (uint32_t)g.row_stride, r0 = (uint32_t)lane % 9;
        const uint32_t off0 = (uint32_t)(rg * (32 * L::RG) + wave * 32 + lane / 9) * stride + r0 * 16;
        const uint32_t last = (uint32_t)(g.rows - 1) * stride + 128;
#pragma unroll
        for (int c = 0; c < 5; c++) {
            // piece p + 64 = 7 rows + 1 piece further on, one more row where the piece index wraps past 8
            w_off[c] = min(off0 + c * (7 * stride + 16) + (r0 + c >= 9 ? stride - Q4_K_BYTES : 0u), last);
            asm volatile("" : "+v"(w_off[c]));
        }
        f_two = count > 32;
        if (GATHER) {
            // piece (row, 16-byte half hk) of quant slice `wave`: bytes 32 * wave + 16 * hk of the row's block;
            // of the sums: 16 * hk of the block's 32 bytes; the scale: the block's 4 bytes
            uint32_t src;  // this lane's source rows of the tile (row lane % 32 of either half)
            asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(src) : "v"(lds_src + ord * 128 + (lane & 31) * 4));
            const uint32_t row_a = src & 0xffffu, row_b = src >> 16, hk = (uint32_t)(lane >> 5) * 16;
            const uint32_t cols = (uint32_t)nb * QK_K, row = x_second ? row_b : row_a;
            qa_off = row_a * cols + (uint32_t)wave * 32 + hk;
            qb_off = row_b * cols + (uint32_t)wave * 32 + hk;
            x_off = x_sums ? row * (uint32_t)nb * 32 + hk : row * (uint32_t)nb * 4;
            asm volatile("" : "+v"(qa_off), "+v"(qb_off), "+v"(x_off));
            f_q = g.src.q;
            f_x = x_sums ? reinterpret_cast<const uint8_t *>(g.src.bs) : reinterpret_cast<const uint8_t *>(g.src.d);
        } else {
            const size_t rec = (size_t)(2 * t + (x_second ? 1 : 0)) * nb;  // the small piece's half
            f_q = g.a.q + (size_t)2 * t * nb * 8192;
            f_x = x_sums ? reinterpret_cast<const uint8_t *>(g.a.bs + rec * 512)
                         : reinterpret_cast<const uint8_t *>(g.a.d + rec * 32);
        }
    };
    auto fetch_acts = [&]() {  // of the cursor's step
        uint8_t *st = lds + L::OFF_A + (f_step & 3) * L::A_STAGE;
        load_to_lds16(f_q + qa_off, st + wave * 1024);
        issued = 1;
        if (f_two) {
            load_to_lds16(f_q + qb_off, st + L::A_HALF + wave * 1024);
            issued = 2;
        }
        if (x_small && (!x_second || f_two)) {
            uint8_t *half = st + (x_second ? L::A_HALF : 0);
            if (x_sums) load_to_lds16(f_x + x_off, half + L::A_BS);
            else load_to_lds4(f_x + x_off, half + L::A_DA);
            issued++;
        }
    };
    auto fetch_weights = [&]() {  // of the cursor's step; moves the cursor on
        uint8_t *st = lds + (f_step & 1) * L::W_STAGE + wave * L::W_WAVE;
#pragma unroll
        for (int c = 0; c < 5; c++)
            if (c < 4 || lane < 32) load_to_lds16(f_w + w_off[c], st + c * 1024);
        issued += 5;
        f_step++;
        f_w += Q4_K_BYTES;
        f_q += GATHER ? QK_K : 8192;
        f_x += GATHER ? (x_sums ? 32 : 4) : (x_sums ? 1024 : 128);
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
    int c_ord = 0, c_kb = 0, c_count = 0, c_y_row = 0;
    int pending = -1, pending_count = 0, pending_y_row = 0;  // item whose results wait to be stored
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
            item_info(c_ord, expert, c_count, c_y_row);
        }
        const BlockScales sc = block_scales(R);
        const int lg_next = opaque_lane() >> 5;
        const ScalePairs sp = scale_pairs(sc);
        multiply_half(st, accF0, B, [&](int i, v16i &) {
            if (i == 0) unpack_pair_free(R.q0, sp.p0, sp.p1, Bnext.H0, Bnext.L0, Bnext.H1, Bnext.L1);
            if (i == 2) unpack_pair_free(R.q1, sp.p2, sp.p3, Bnext.H2, Bnext.L2, Bnext.H3, Bnext.L3);
            if (i == 4) unpack_pair_free(R.q2, sp.p4, sp.p5, Bnext.H4, Bnext.L4, Bnext.H5, Bnext.L5);
            if (i == 6) unpack_pair_free(R.q3, sp.p6, sp.p7, Bnext.H6, Bnext.L6, Bnext.H7, Bnext.L7);
            if (i == 8) unpack_rest(R, sc, lg_next, Bnext);
        });
        if (c_count > 32) multiply_half(st + L::A_HALF, accF1, B, NothingBetween());
        if (++c_kb == nb) {
            pending = c_ord++;
            pending_count = c_count;
            pending_y_row = c_y_row;
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
        float *y = (m ? g.y[1] : g.y[0]) + (size_t)pending_y_row * rows;
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
        unpack_block_sel(R, lg, B0);
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

template <int RG, int KS, int MT, bool Q5 = false>
static int launch_pipe(const GemmArgs &g, unsigned grid, hipStream_t s) {
    constexpr size_t shmem = PipeLds<RG, KS, MT, Q5>::BYTES;
    static_assert(shmem <= 160 * 1024, "LDS of a CU");
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4_k_pipe_kernel<RG, KS, MT, Q5>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(LDS %zu): %s", shmem, hipGetErrorString(e));
        sized = true;
    }
    hipLaunchKernelGGL((gemm_q4_k_pipe_kernel<RG, KS, MT, Q5>), dim3(grid, (unsigned)g.k_split), dim3(512), shmem, s, g);
    FRK_LAUNCH_CHECK("gemm_q4_k_pipe");
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
// The workgroup tile of a batch: 256 rows x 128 tokens when that gives (about) every CU a workgroup,
// else 128 rows x 64 tokens with each row's blocks shared between two wavefronts -- and with those,
// when the grid still fills few of the CUs, a row's blocks split between 2 or 4 workgroups (no finer
// than four blocks each) whose sums are added in order afterwards.
struct Q4KPlan {
    int rows_wg, tok_wg, k_split;
};
static Q4KPlan q4_k_plan(size_t rows, size_t M, size_t nb, bool q5 = false) {
    // (Q5_K: the third plane's 32 registers fit the 128 x 64 form only)
    if (!q5 && M > 64 && ((rows + 255) / 256) * ((M + 127) / 128) >= 200) return {256, 128, 1};
    const size_t grid = (((rows + 127) / 128 + 7) / 8 * 8) * ((M + 63) / 64);
    int ks = 1;
    while (ks < Q4K_MAX_SPLIT && grid * (size_t)ks * 2 <= 256 && nb / (size_t)(ks * 2) >= 4) ks *= 2;
    return {128, 64, ks};
}
// the tiled activations, then room for the parts' sums where the blocks are split
size_t gemm_q4_k_workspace_bytes(size_t M, size_t cols, size_t rows, bool q5) {
    const Q4KPlan p = q4_k_plan(rows, M, cols / QK_K, q5);
    return round_up(q8k_tiled_bytes(M, cols), 256) + (p.k_split > 1 ? (size_t)p.k_split * M * rows * sizeof(float) : 0);
}

// the GEMM proper, over activations already in the tiled form (`partial`: room for the parts' sums)
int launch_gemm_q4_k_acts(const frk_weights *w, Q8KTiled acts, size_t M, float *y, float *partial, hipStream_t s) {
    // the kernel addresses a row group's weights with 32-bit lane offsets
    if ((uint64_t)w->layout.row_stride * 64 >= (1ull << 32))
        return set_error(FRK_ERR_SHAPE, "gemm_q4_k: rows of %zu bytes are beyond the kernel's offsets", w->layout.row_stride);
    GemmArgs g;
    g.a = acts;
    g.W = w->dev;
    g.row_stride = w->layout.row_stride;
    g.rows = (int)w->rows;
    g.nb = (int)(w->cols / QK_K);
    g.M = (int)M;
    g.y = y;
    g.partial = partial;
    const bool q5 = w->kind == FRK_KIND_Q5_K;
    const Q4KPlan p = q4_k_plan(w->rows, M, (size_t)g.nb, q5);
    g.row_tiles = (int)((w->rows + p.rows_wg - 1) / p.rows_wg);
    g.tok_tiles = (int)((M + p.tok_wg - 1) / p.tok_wg);
    g.k_split = p.k_split;
    const unsigned grid = (unsigned)((g.row_tiles + 7) / 8 * 8 * g.tok_tiles);
    if (q5) return launch_pipe<4, 2, 2, true>(g, grid, s);
    return p.rows_wg == 256 ? launch_pipe<8, 1, 4>(g, grid, s) : launch_pipe<4, 2, 2>(g, grid, s);
}

int launch_gemm_q4_k(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s) {
    const Q8KTiled acts = q8k_tiled_carve(ws, M, w->cols);
    int rc = launch_quantize_q8_k_tiled(x, M, w->cols, acts, s);
    if (rc) return rc;
    return launch_gemm_q4_k_acts(w, acts, M, y, reinterpret_cast<float *>((char *)ws + round_up(q8k_tiled_bytes(M, w->cols), 256)), s);
}
// (Q5_K weights take the same entry points: launch_gemm_q4_k_acts looks at the kind)

template <bool GATHER>
static int launch_stream(const StreamArgs &g, int max_tiles, hipStream_t s) {
    using L = StreamLds<GATHER>;
    static int grid = 0;
    if (grid == 0) {
        int dev = 0, cus = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4_k_stream_kernel<GATHER>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)L::BYTES);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "gemm_q4_k_stream setup: %s", hipGetErrorString(e));
        grid = cus < 8 ? 8 : cus / 8 * 8;  // one workgroup per CU, a multiple of the 8 XCDs
    }
    // more workgroups than CUs when a workgroup's share of the largest possible list would not fit
    // its item table
    const size_t most_items = ((size_t)max_tiles + 7) / 8 * g.n_mat * g.row_tiles;
    const unsigned rounds = (unsigned)((most_items + (size_t)(grid / 8) * L::MAX_ITEMS - 1) /
                                       ((size_t)(grid / 8) * L::MAX_ITEMS));
    hipLaunchKernelGGL(gemm_q4_k_stream_kernel<GATHER>, dim3((unsigned)grid * (rounds ? rounds : 1)), dim3(64 * L::RG),
                       L::BYTES, s, g);
    FRK_LAUNCH_CHECK("gemm_q4_k_stream");
    return FRK_OK;
}

bool gemm_q4_k_stream_gathers(size_t src_rows, size_t cols) {
    // a source row is a 16-bit entry of the kernel's table, a row's place a 32-bit lane offset
    return src_rows <= 65535 && src_rows * cols < (1ull << 32);
}

int launch_gemm_q4_k_stream(const frk_weights *w0, const frk_weights *w1, size_t rows_e, Q8KTiled a,
                            const Q8KRows *src, const int *gather, const int4 *tiles, const int *n_tiles,
                            int max_tiles, float *y0, float *y1, hipStream_t s) {
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
    g.src = src ? *src : Q8KRows{nullptr, nullptr, nullptr};
    g.gather = gather;
    return src ? launch_stream<true>(g, max_tiles, s) : launch_stream<false>(g, max_tiles, s);
}

}  // namespace frk
