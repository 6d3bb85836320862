// Batched GEMM for Q6_K weights on the int8 matrix cores:  y[M][rows] = Q8_K(x)[M][cols] . W^T.
// The arithmetic is gemm_q6_k_q8_row / dot_q6_k_q8 (crates/frink-quant/src/lib.rs:1033-1110): per
// 256-wide block the exact integer  isum = sum_g sc_g * sum_{i in g} (q6_i - 32) * a_i  over the
// sixteen 16-weight groups g, then  acc += (d * da) * isum.
//
// How a signed 8-bit scale times a 6-bit code gets through an int8 MFMA.  A lane's 16 bytes of a
// 32x32x32 operand are 16 consecutive weights of one row, i.e. exactly one group: the group's scale
// s is a lane value.  With  s = 16*sh + sl  (sh = s >> 4 in -8..7, sl = s & 15)  and the raw code
// q6 = 8*qu + ql  (qu, ql in 0..7), so that  q6 - 32 = 8*(qu - 4) + ql:
//     s * (q6 - 32) = 128 * sh*(qu-4) + 16 * sh*ql + 8 * sl*(qu-4) + sl*ql
//                   = 8 * (8*HH + HL + LH) + LL
// and the four planes HH = 2*sh*(qu-4) in -56..64, HL = 2*sh*ql in -112..98, LH = sl*(qu-4) in
// -60..45, LL = sl*ql in 0..105 are int8.  One accumulator runs four chains of MFMAs with a shift by
// 3 after the first and before the last.  Half a block (four 32-weight sub-blocks) is unpacked at a time: 16 operand planes,
// 64 registers; the block's two halves add up as integers before the one float step per block.
//
// The planes are built four bytes at a time: a packed 16-bit multiply serves two bytes at once as
// long as no product reaches 256, and the signed planes are formed in a biased form (q6_word).
//
// Data movement is the dense Q4_K kernel's: everything goes global -> LDS with global_load_lds, LDS
// reads are issued from inline assembly with hand-placed waits (the compiler would wait for the whole
// prefetch in front of every read).  Weights are the resident planar rows (ql | qh | sc | d, see
// layout_for): a wavefront stages its own 32 rows -- 128 bytes of ql, 64 of qh, 16 of sc per row and
// block -- in an area only it reads.  A row's 16-byte pieces are stored XOR-swizzled by the row
// number, so that the 32 rows' reads of one logical piece fall in different banks while every
// global access still covers whole rows.  Activations are the tiled Q8_K form (frk_gemm.hip).
#include "frk_device.hpp"

#include <type_traits>

namespace frk {

typedef int q6_v2i __attribute__((ext_vector_type(2)));
typedef int q6_v4i __attribute__((ext_vector_type(4)));
typedef int q6_v16i __attribute__((ext_vector_type(16)));
typedef float q6_v4f __attribute__((ext_vector_type(4)));
typedef float q6_v16f __attribute__((ext_vector_type(16)));
typedef unsigned short q6_us2 __attribute__((ext_vector_type(2)));

struct Q6GemmArgs {
    const uint8_t *W;
    uint32_t row_stride, off_qh, off_sc, off_d;
    int rows, nb, M;
    Q8KTiled a;
    float *y;
    int row_tiles, tok_tiles;
    int k_split;     // 1, or 2/4/8: blockIdx.y takes that share of the blocks and writes its sums to `partial`
    float *partial;  // [k_split][M][rows], added up in order by sum_parts_kernel
    // The grouped (per-expert) form: token tile t (64 rows of the activations and of y) belongs to expert
    // tiles[t].x, whose `rows` weight rows start at row tiles[t].x * rows of W, and has tiles[t].z rows in
    // use; tiles past *n_tiles do nothing.  Null for one matrix.
    const int4 *tiles;
    const int *n_tiles;
};

struct Q6Lds {
    static constexpr int RG = 8, MT = 2;
    static constexpr int A_D = MT * 8192;             // the tiles' quants, then their scales
    static constexpr int A_STAGE = A_D + MT * 128;    // 16640
    static constexpr int W_QH = 32 * 128, W_SC = W_QH + 32 * 64;
    static constexpr int W_WAVE = W_SC + 32 * 16;     // 6656: a wavefront's 32 rows of one block
    static constexpr int W_STAGE = RG * W_WAVE;       // 53248
    static constexpr int OFF_W = 2 * A_STAGE;
    static constexpr size_t BYTES = (size_t)OFF_W + 2 * W_STAGE;  // 139776
};

#define FRK6_DS_READ128(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:" #off : "=v"(dst) : "v"(addr))
#define FRK6_DS_READ64(dst, addr, off) asm volatile("ds_read_b64 %0, %1 offset:" #off : "=v"(dst) : "v"(addr))

struct Q6Raw {  // a lane's share of half a block: two ql pieces, one qh piece, the half's eight scales
    q6_v4i qa, qb, qh;
    q6_v2i sc;
};
struct Q6Planes {
    q6_v4i HH0, HH1, HH2, HH3, HL0, HL1, HL2, HL3, LH0, LH1, LH2, LH3, LL0, LL1, LL2, LL3;
};
struct Q6Ops {  // the four 32-wide activation slices of half a block
    q6_v4i a0, a1, a2, a3;
};

__device__ __forceinline__ uint32_t q6_pk_mul(uint32_t bytes, uint32_t factor) {  // four bytes x one small factor
    q6_us2 a;
    __builtin_memcpy(&a, &bytes, 4);
    const q6_us2 f = {(unsigned short)factor, (unsigned short)factor};
    const q6_us2 r = a * f;
    uint32_t out;
    __builtin_memcpy(&out, &r, 4);
    return out;
}

// What a lane needs of its group's scale s = 16*sh + sl to build the planes' bytes, four at a time.
// With K = 0x80 in every byte, m = 2*|sh| and x, y, z the packed products m*ql, sl*qu, m*qu (all < 128):
//     LL = sl*ql                                                   (as multiplied)
//     LH = sl*(qu-4)      = ((y + (K - 4sl)) ^ K                   (biased by 128, bias removed)
//     HL = 2*sh*ql        = x                       or, sh < 0:  (K - x) ^ K
//     HH = 2*sh*(qu-4)    = (z + (K - 4m)) ^ K      or, sh < 0:  ((K + 4m) - z) ^ K
// and "c - v" is written "(v ^ ~0) + (c + 1)", so that both signs are one xor, one add, one xor with
// lane constants.  No byte ever borrows from or carries into its neighbour: every biased value
// stays within 0x10..0xF0.
struct Q6Scale {
    uint32_t sl, m;           // sl and 2*|sh|
    uint32_t flip;            // ~0 where sh < 0
    uint32_t lh_add;          // K - 4*sl
    uint32_t hl_add, hl_xor;  // 0, 0  or  K + 1, K
    uint32_t hh_add;          // K - 4*m  or  K + 4*m + 1
};
__device__ __forceinline__ Q6Scale q6_scale(int s) {
    const uint32_t K = 0x80808080u;
    const int sh = s >> 4;
    Q6Scale c;
    c.sl = (uint32_t)(s & 15);
    c.m = 2u * (uint32_t)(sh < 0 ? -sh : sh);
    const bool neg = sh < 0;
    c.flip = neg ? 0xffffffffu : 0u;
    c.lh_add = K - (4u * c.sl) * 0x01010101u;
    c.hl_add = neg ? K + 1u : 0u;
    c.hl_xor = neg ? K : 0u;
    c.hh_add = neg ? K + (4u * c.m) * 0x01010101u + 1u : K - (4u * c.m) * 0x01010101u;
    return c;
}
// four codes of one group, given as their low three bits ql and their high three bits qu (a byte
// each) -> their bytes of the four planes
__device__ __forceinline__ void q6_word(uint32_t ql, uint32_t qu, const Q6Scale &c, int &hh, int &hl, int &lh, int &ll) {
    const uint32_t K = 0x80808080u;
    ll = (int)q6_pk_mul(ql, c.sl);
    hl = (int)(((q6_pk_mul(ql, c.m) ^ c.flip) + c.hl_add) ^ c.hl_xor);
    lh = (int)((q6_pk_mul(qu, c.sl) + c.lh_add) ^ K);
    hh = (int)(((q6_pk_mul(qu, c.m) ^ c.flip) + c.hh_add) ^ K);
}

// dequant_q6_k's code assembly (crates/frink-quant/src/lib.rs:519-552) for a lane's 16 columns of
// the half: sub-blocks 0..3 are the weights 128h + 32j + 16lg + (0..15), the code of a weight is
// a nibble of ql (low nibbles: sub-blocks 0 and 1, high: 2 and 3) under two bits of qh (bits 2j..).
// The code is never put together: its low three bits are the nibble's, its high three the nibble's
// top bit under the two bits of qh.  One sub-block per call, so that a caller can spread the four
// between other work.
template <int J>
__device__ __forceinline__ void q6_unpack_sub(const Q6Raw &R, int lg, q6_v4i &HH, q6_v4i &HL, q6_v4i &LH, q6_v4i &LL) {
    const q6_v4i nib = (J & 1) ? R.qb : R.qa;
    // the group's scale: byte 2j + lg of the half's eight
    const uint32_t word = (uint32_t)(J < 2 ? R.sc.x : R.sc.y) >> (8 * lg + 16 * (J & 1));
    const Q6Scale c = q6_scale((int)(int8_t)(word & 0xff));
    auto one = [&](int nw, int hw, int &hh, int &hl, int &lh, int &ll) {
        const uint32_t n = (uint32_t)nw >> (J < 2 ? 0 : 4), h = (uint32_t)hw;
        const uint32_t ql = n & 0x07070707u;
        // bit 0 of qu: the nibble's bit 3; bits 1..2: qh's bits 2J, 2J+1
        const uint32_t top = (n >> 3) & 0x01010101u;
        const uint32_t two = (J == 0 ? (h << 1) : (h >> (2 * J - 1))) & 0x06060606u;
        q6_word(ql, top | two, c, hh, hl, lh, ll);
    };
    int h0, h1, h2, h3, a0, a1, a2, a3, b0, b1, b2, b3, l0, l1, l2, l3;
    one(nib.x, R.qh.x, h0, a0, b0, l0);
    one(nib.y, R.qh.y, h1, a1, b1, l1);
    one(nib.z, R.qh.z, h2, a2, b2, l2);
    one(nib.w, R.qh.w, h3, a3, b3, l3);
    HH = q6_v4i{h0, h1, h2, h3};
    HL = q6_v4i{a0, a1, a2, a3};
    LH = q6_v4i{b0, b1, b2, b3};
    LL = q6_v4i{l0, l1, l2, l3};
}
__device__ __forceinline__ void q6_unpack_half(const Q6Raw &R, int lg, Q6Planes &P) {
    q6_unpack_sub<0>(R, lg, P.HH0, P.HL0, P.LH0, P.LL0);
    q6_unpack_sub<1>(R, lg, P.HH1, P.HL1, P.LH1, P.LL1);
    q6_unpack_sub<2>(R, lg, P.HH2, P.HL2, P.LH2, P.LL2);
    q6_unpack_sub<3>(R, lg, P.HH3, P.HL3, P.LH3, P.LL3);
}

// sum over the half of scale * (code - 32) * activation, for a 32x32 tile: sixteen MFMAs, one accumulator
// between(i) is called after MFMA i has been issued (i = 0..14): what it does shares the gaps of the
// chain, every MFMA of which waits for the one before it.
struct Q6NothingBetween {
    __device__ __forceinline__ void operator()(int) const {}
};
template <class Between = Q6NothingBetween>
__device__ __forceinline__ q6_v16i q6_tile_half(const Q6Ops &T, const Q6Planes &P, Between between = Between()) {
    const q6_v16i zi = {0};
    q6_v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, P.HH0, zi, 0, 0, 0);
    between(0);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, P.HH1, acc, 0, 0, 0);
    between(1);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, P.HH2, acc, 0, 0, 0);
    between(2);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, P.HH3, acc, 0, 0, 0);
    between(3);
    acc = acc << 3;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, P.HL0, acc, 0, 0, 0);
    between(4);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, P.HL1, acc, 0, 0, 0);
    between(5);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, P.HL2, acc, 0, 0, 0);
    between(6);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, P.HL3, acc, 0, 0, 0);
    between(7);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, P.LH0, acc, 0, 0, 0);
    between(8);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, P.LH1, acc, 0, 0, 0);
    between(9);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, P.LH2, acc, 0, 0, 0);
    between(10);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, P.LH3, acc, 0, 0, 0);
    between(11);
    acc = acc << 3;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a0, P.LL0, acc, 0, 0, 0);
    between(12);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a1, P.LL1, acc, 0, 0, 0);
    between(13);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a2, P.LL2, acc, 0, 0, 0);
    between(14);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(T.a3, P.LL3, acc, 0, 0, 0);
    return acc;
}

// A workgroup = 8 wavefronts and 64 activation rows (two 32-row tiles).  WT = 1: 8 row groups of 32
// weight rows, every wavefront multiplies its rows with both tiles.  WT = 2, for matrices with too
// few rows to give every CU one of those: 4 row groups, wavefront w takes row group w % 4 and tile
// w / 4 (both wavefronts of a row group stage the rows for themselves: no sharing, no barrier).
// The operand planes are double-buffered: while one half-block is multiplied, the next one (the
// block's other half, or the next block's first) is unpacked into the other set from inside the
// chain of MFMAs of the wavefront's first tile.
template <int WT>
__global__ __launch_bounds__(512) void gemm_q6_k_mfma_kernel(Q6GemmArgs g) {
    using L = Q6Lds;
    constexpr int RGS = L::RG / WT, MT = L::MT / WT;  // row groups of the workgroup, tiles of a wavefront
    extern __shared__ uint4 smem_q6[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem_q6);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lg = lane >> 5;
    const int rgrp = wave % RGS, tile_first = (wave / RGS) * MT;

    // workgroups that share weight rows (different token tiles) sit on one XCD (block id mod 8)
    const int bid = blockIdx.x;
    const int per_group = 8 * g.tok_tiles;
    const int grp = bid / per_group, in_grp = bid % per_group;
    const int row_tile = grp * 8 + (in_grp & 7);
    if (row_tile >= g.row_tiles) return;  // uniform per workgroup
    const int tok0 = (in_grp >> 3) * (32 * L::MT);
    const int row0 = row_tile * (32 * RGS) + rgrp * 32;  // this wavefront's first weight row
    const int nb = g.nb;  // blocks of a row (strides); this workgroup multiplies blocks kb_begin .. kb_end - 1
    const int kb_begin = nb * (int)blockIdx.y / g.k_split, kb_end = nb * ((int)blockIdx.y + 1) / g.k_split;
    // (never empty: the launcher splits no finer than four blocks a part)
    const int tile0 = tok0 / 32, last_tile = (g.M - 1) / 32;
    uint32_t expert_base = 0;  // byte offset of the expert's first weight row
    int tok_end = g.M;         // first activation row that is not stored
    int y_shift = 0;           // activation row r is stored as row r + y_shift of y
    if (g.tiles) {             // (uniform per workgroup)
        const int t = in_grp >> 3;
        if (t >= *g.n_tiles) return;
        const int4 ti = g.tiles[t];
        expert_base = (uint32_t)ti.x * (uint32_t)g.rows * g.row_stride;
        tok_end = ti.y + ti.z;
        y_shift = ti.w - ti.y;
    }
    auto opaque_lane = [&]() {  // the lane number as a value the compiler cannot hoist expressions of
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    auto row_offset = [&](int r) { return expert_base + (uint32_t)min(row0 + r, g.rows - 1) * g.row_stride; };  // rows past the end repeat the last

    // ---- the prefetch ----
    const uint8_t *Qb = reinterpret_cast<const uint8_t *>(g.a.q);
    const uint32_t d_base = (uint32_t)(reinterpret_cast<const uint8_t *>(g.a.d) - Qb);
    auto tile_rec = [&](int t) { return (uint32_t)min(tile0 + t, last_tile) * (uint32_t)nb; };
    auto issue_acts = [&](int kb) {  // block kb of the workgroup's two tiles
        asm volatile("" : "+s"(kb));
        uint8_t *st = lds + (kb & 1) * L::A_STAGE;
        const uint32_t l = (uint32_t)opaque_lane();
#pragma unroll
        for (int t = 0; t < L::MT; t++)  // slice `wave` of each tile
            load_to_lds16(Qb + ((tile_rec(t) + kb) * 8192 + wave * 1024 + l * 16), st + t * 8192 + wave * 1024);
        if (wave == 0)  // the 32 scales of both tiles, one tile per lane half
            load_to_lds4(Qb + (d_base + (tile_rec((int)(l >> 5)) + kb) * 128 + (l & 31) * 4), st + L::A_D);
    };
    auto issue_weights = [&](int kb) {  // block kb of this wavefront's 32 rows: 4 + 2 + 1 loads
        asm volatile("" : "+s"(kb));
        uint8_t *st = lds + L::OFF_W + (kb & 1) * L::W_STAGE + wave * L::W_WAVE;
        const uint32_t l = (uint32_t)opaque_lane();
#pragma unroll
        for (int i = 0; i < 4; i++) {  // ql: 8 rows a load; piece pp of the LDS row holds piece pp ^ (row & 7)
            const uint32_t r = 8 * i + (l >> 3), piece = (l & 7) ^ (l >> 3);
            load_to_lds16(g.W + (row_offset((int)r) + (uint32_t)kb * 128 + piece * 16), st + i * 1024);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {  // qh: 16 rows a load; piece pp holds piece pp ^ ((row >> 1) & 3)
            const uint32_t r = 16 * i + (l >> 2), piece = (l & 3) ^ ((r >> 1) & 3);
            load_to_lds16(g.W + (row_offset((int)r) + g.off_qh + (uint32_t)kb * 64 + piece * 16), st + L::W_QH + i * 1024);
        }
        if (l < 32) load_to_lds16(g.W + (row_offset((int)l) + g.off_sc + (uint32_t)kb * 16), st + L::W_SC);
    };
    // the block's f16 super-scale d of this lane's row comes straight from memory, a block ahead
    auto load_d = [&](int kb) {
        return *reinterpret_cast<const uint16_t *>(g.W + (row_offset(li) + g.off_d + (uint32_t)min(kb, nb - 1) * 2));
    };

    const uint32_t lds_a = lds_address(lds);
    const uint32_t lds_w = lds_address(lds + L::OFF_W) + wave * L::W_WAVE;
    auto read_raw = [&](int kb, int h) {  // (a block past the last one: whatever its stage holds, for planes nobody uses)
        const int l = opaque_lane(), r = l & 31, k = l >> 5;
        const uint32_t st = lds_w + (kb & 1) * L::W_STAGE;
        const uint32_t pa = (uint32_t)((4 * h + k) ^ (r & 7)), pb = (uint32_t)((4 * h + 2 + k) ^ (r & 7));
        const uint32_t ph = (uint32_t)((2 * h + k) ^ ((r >> 1) & 3));
        Q6Raw R;
        FRK6_DS_READ128(R.qa, st + r * 128 + pa * 16, 0);
        FRK6_DS_READ128(R.qb, st + r * 128 + pb * 16, 0);
        FRK6_DS_READ128(R.qh, st + L::W_QH + r * 64 + ph * 16, 0);
        FRK6_DS_READ64(R.sc, st + L::W_SC + r * 16 + 8 * h, 0);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(R.qa), "+v"(R.qb), "+v"(R.qh), "+v"(R.sc));
        return R;
    };
    auto read_ops = [&](int kb, int h, int t, Q6Ops &T) {
        const uint32_t a = lds_a + (kb & 1) * L::A_STAGE + t * 8192 + h * 4096 + opaque_lane() * 16;
        FRK6_DS_READ128(T.a0, a, 0);
        FRK6_DS_READ128(T.a1, a, 1024);
        FRK6_DS_READ128(T.a2, a, 2048);
        FRK6_DS_READ128(T.a3, a, 3072);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(T.a0), "+v"(T.a1), "+v"(T.a2), "+v"(T.a3));
    };
    // result register r belongs to token 8*(r/4) + 4*(lane/32) + r%4 of the tile
    auto read_scales = [&](int kb, int t, q6_v4f &d0, q6_v4f &d1, q6_v4f &d2, q6_v4f &d3) {
        const uint32_t a = lds_a + (kb & 1) * L::A_STAGE + L::A_D + t * 128 + (opaque_lane() >> 5) * 16;
        FRK6_DS_READ128(d0, a, 0);
        FRK6_DS_READ128(d1, a, 32);
        FRK6_DS_READ128(d2, a, 64);
        FRK6_DS_READ128(d3, a, 96);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(d0), "+v"(d1), "+v"(d2), "+v"(d3));
    };

    q6_v16f accF[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) accF[mt] = q6_v16f{0.0f};

    // prologue: weights of the first two blocks, activations of the first; its first half unpacked
    issue_weights(kb_begin);
    issue_acts(kb_begin);
    if (kb_begin + 1 < kb_end) issue_weights(kb_begin + 1);
    uint32_t d_bits = load_d(kb_begin);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    Q6Planes P0, P1;
    {
        const Q6Raw R = read_raw(kb_begin, 0);
        q6_unpack_half(R, lg, P0);
    }

    // one half-block: multiply with the planes in Pc while the half after it is unpacked into Pn
    q6_v16i X[MT];
    auto half_step = [&](int kb, auto half, const Q6Planes &Pc, Q6Planes &Pn) {
        constexpr int H = decltype(half)::value;
        // the half after this one: this block's second, or the next block's first
        const Q6Raw R = H == 0 ? read_raw(kb, 1) : read_raw(kb + 1, 0);
        // with the block's second half in registers its stage is free for block kb+2
        if (H == 0 && kb + 2 < kb_end) issue_weights(kb + 2);
        const int k = opaque_lane() >> 5;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            Q6Ops T;
            read_ops(kb, H, tile_first + mt, T);
            q6_v16i s;
            if (mt == 0) {
                s = q6_tile_half(T, Pc, [&](int i) {
                    if (i == 1) q6_unpack_sub<0>(R, k, Pn.HH0, Pn.HL0, Pn.LH0, Pn.LL0);
                    if (i == 5) q6_unpack_sub<1>(R, k, Pn.HH1, Pn.HL1, Pn.LH1, Pn.LL1);
                    if (i == 9) q6_unpack_sub<2>(R, k, Pn.HH2, Pn.HL2, Pn.LH2, Pn.LL2);
                    if (i == 13) q6_unpack_sub<3>(R, k, Pn.HH3, Pn.HL3, Pn.LH3, Pn.LL3);
                });
            } else {
                s = q6_tile_half(T, Pc);
            }
            if (H == 0) X[mt] = s;
            else X[mt] = X[mt] + s;
            // (keeps a tile's MFMAs from being scheduled into the next tile's LDS reads)
            asm volatile("" : "+v"(X[mt]));
        }
    };

    for (int kb = kb_begin; kb < kb_end; kb++) {
        const float dw = h2f(d_bits & 0xffffu);  // (before anything new is requested: its load is long done)
        // the activation stage refilled here was last read in iteration kb-1, which every wavefront has left
        if (kb + 1 < kb_end) issue_acts(kb + 1);
        d_bits = load_d(kb + 1);
        half_step(kb, std::integral_constant<int, 0>(), P0, P1);
        half_step(kb, std::integral_constant<int, 1>(), P1, P0);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            q6_v4f d0, d1, d2, d3;
            read_scales(kb, tile_first + mt, d0, d1, d2, d3);
            const q6_v4f dav[4] = {d0, d1, d2, d3};
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int r = c * 4 + e;
                    accF[mt][r] = fmaf(dw * dav[c][e], (float)X[mt][r], accF[mt][r]);
                }
            asm volatile("" : "+v"(accF[mt]));
        }
        // activations of block kb+1 and weights of block kb+2 have landed (block kb+1's did an
        // iteration ago: its first half has just been read)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
    }

    // store: a lane holds one weight row and 16 tokens per tile
    const int row = row0 + li;
    float *const dst = g.k_split > 1 ? g.partial + (size_t)blockIdx.y * g.M * g.rows : g.y;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int tok = tok0 + (tile_first + mt) * 32 + (r >> 2) * 8 + lg * 4 + (r & 3);
            if (row < g.rows && tok < tok_end) dst[(size_t)(tok + y_shift) * g.rows + row] = accF[mt][r];
        }
}

// y = the parts' sums added in the order of the parts: the same bits on every run
__global__ __launch_bounds__(256) void sum_parts_kernel(const float *__restrict__ partial, int parts, size_t n,
                                                        float *__restrict__ y) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float acc = partial[i];
    for (int p = 1; p < parts; p++) acc += partial[(size_t)p * n + i];
    y[i] = acc;
}

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

int launch_sum_parts(const float *partial, int parts, size_t n, float *y, hipStream_t s) {
    hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, partial, parts, n, y);
    FRK_LAUNCH_CHECK("sum of the split GEMM's parts");
    return FRK_OK;
}

// fewer 256-row workgroups than this leave too many CUs idle: split the blocks, or take 128-row ones
constexpr size_t Q6_NARROW_BELOW = 200;
constexpr int Q6_MAX_SPLIT = 8;
// 256 weight rows per workgroup (a block is unpacked once for two tiles) when that gives about every
// CU one.  For a short and wide matrix, or a batch of few token tiles, the blocks are split between 2,
// 4 or 8 workgroups (no finer than four blocks each) whose sums a second kernel adds up in order.
static int q6_k_split(size_t rows, size_t M, size_t nb) {
    const size_t wgs256 = ((rows + 255) / 256) * ((M + 63) / 64);
    int ks = 1;
    while (ks < Q6_MAX_SPLIT && wgs256 < Q6_NARROW_BELOW && wgs256 * ks * 2 <= 256 && nb / (size_t)(ks * 2) >= 4) ks *= 2;
    return ks;
}
// the tiled activations, then room for the parts' sums where the blocks are split
size_t gemm_q6_k_workspace_bytes(size_t M, size_t cols, size_t rows) {
    const int ks = q6_k_split(rows, M, cols / QK_K);
    return round_up(q8k_tiled_bytes(M, cols), 256) + (ks > 1 ? (size_t)ks * M * rows * sizeof(float) : 0);
}

int launch_gemm_q6_k(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s) {
    const Q8KTiled acts = q8k_tiled_carve(ws, M, w->cols);
    int rc = launch_quantize_q8_k_tiled(x, M, w->cols, acts, s);
    if (rc) return rc;
    return launch_gemm_q6_k_acts(w, acts, M, y, reinterpret_cast<float *>((char *)ws + round_up(q8k_tiled_bytes(M, w->cols), 256)), s);
}

// the GEMM proper, over activations already in the tiled form (`partial`: room for the parts' sums)
int launch_gemm_q6_k_acts(const frk_weights *w, Q8KTiled acts, size_t M, float *y, float *partial, hipStream_t s) {
    // the kernel addresses the weights and the tiled activations with 32-bit byte offsets
    if ((uint64_t)w->rows * w->layout.row_stride >= (1ull << 32) || (uint64_t)q8k_tiled_bytes(M, w->cols) >= (1ull << 32))
        return set_error(FRK_ERR_SHAPE, "gemm_q6_k: %zu x %zu weights with %zu activation rows exceed 4 GiB per operand", w->rows,
                         w->cols, M);
    Q6GemmArgs g;
    g.a = acts;
    g.W = w->dev;
    g.row_stride = (uint32_t)w->layout.row_stride;
    g.off_qh = (uint32_t)w->layout.off_a;
    g.off_sc = (uint32_t)w->layout.off_b;
    g.off_d = (uint32_t)w->layout.off_c;
    g.rows = (int)w->rows;
    g.nb = (int)(w->cols / QK_K);
    g.M = (int)M;
    g.y = y;
    g.tok_tiles = (int)((M + 63) / 64);
    // the blocks split between workgroups (q6_k_split), or 128 rows per workgroup where even that
    // leaves most CUs idle
    const size_t wgs256 = ((w->rows + 255) / 256) * (size_t)g.tok_tiles;
    const int ks = q6_k_split(w->rows, M, (size_t)g.nb);
    const bool split = ks > 1;
    const bool narrow = wgs256 < Q6_NARROW_BELOW && !split;
    const int rows_wg = narrow ? 128 : 256;
    g.tiles = nullptr;
    g.n_tiles = nullptr;
    g.k_split = ks;
    g.partial = partial;
    g.row_tiles = (int)((w->rows + rows_wg - 1) / rows_wg);
    const dim3 grid((unsigned)((g.row_tiles + 7) / 8 * 8 * g.tok_tiles), (unsigned)g.k_split);
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q6_k_mfma_kernel<1>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)Q6Lds::BYTES);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q6_k_mfma_kernel<2>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)Q6Lds::BYTES);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(LDS %zu): %s", Q6Lds::BYTES, hipGetErrorString(e));
        sized = true;
    }
    if (narrow) hipLaunchKernelGGL(gemm_q6_k_mfma_kernel<2>, grid, dim3(512), Q6Lds::BYTES, s, g);
    else hipLaunchKernelGGL(gemm_q6_k_mfma_kernel<1>, grid, dim3(512), Q6Lds::BYTES, s, g);
    FRK_LAUNCH_CHECK("gemm_q6_k_mfma");
    if (split) return launch_sum_parts(g.partial, ks, M * w->rows, y, s);
    return FRK_OK;
}

// The grouped form for the MoE down projection: `a` holds max_tiles tiles of 64 activation rows in the
// grouped order, y is [64 * max_tiles][rows_e]; w stacks the experts' rows_e x cols matrices.
int launch_gemm_q6_k_grouped(const frk_weights *w, size_t rows_e, Q8KTiled a, const int4 *tiles, const int *n_tiles,
                             int max_tiles, float *y, hipStream_t s) {
    if ((uint64_t)w->rows * w->layout.row_stride >= (1ull << 32) ||
        (uint64_t)q8k_tiled_bytes((size_t)max_tiles * 64, w->cols) >= (1ull << 32))
        return set_error(FRK_ERR_SHAPE, "grouped gemm_q6_k: %zu x %zu weights with %d tiles exceed 4 GiB per operand", w->rows,
                         w->cols, max_tiles);
    if (max_tiles <= 0) return FRK_OK;
    Q6GemmArgs g;
    g.a = a;
    g.W = w->dev;
    g.row_stride = (uint32_t)w->layout.row_stride;
    g.off_qh = (uint32_t)w->layout.off_a;
    g.off_sc = (uint32_t)w->layout.off_b;
    g.off_d = (uint32_t)w->layout.off_c;
    g.rows = (int)rows_e;
    g.nb = (int)(w->cols / QK_K);
    g.M = max_tiles * 64;
    g.y = y;
    g.tok_tiles = max_tiles;
    g.row_tiles = (int)((rows_e + 255) / 256);
    g.k_split = 1;
    g.partial = nullptr;
    g.tiles = tiles;
    g.n_tiles = n_tiles;
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q6_k_mfma_kernel<1>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)Q6Lds::BYTES);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(LDS %zu): %s", Q6Lds::BYTES, hipGetErrorString(e));
        sized = true;
    }
    const dim3 grid((unsigned)((g.row_tiles + 7) / 8 * 8 * g.tok_tiles), 1u);
    hipLaunchKernelGGL(gemm_q6_k_mfma_kernel<1>, grid, dim3(512), Q6Lds::BYTES, s, g);
    FRK_LAUNCH_CHECK("gemm_q6_k_mfma (grouped)");
    return FRK_OK;
}

}  // namespace frk
