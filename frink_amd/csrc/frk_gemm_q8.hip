// Batched GEMM for Q8_0 weights on the int8 matrix cores:  y[M][rows] = Q8_0(x)[M][cols] . W^T.
// The arithmetic is the reference's batched Q8_0 path (crates/frink-core/src/weight_matrix.rs:2701-2829:
// activations quantized per 32 values by quantize_activations_q8, then the integer dot of
// crates/frink-quant/src/lib.rs:692-733): per 32-wide block the exact integer  isum = sum_i qw_i * qa_i
// and  acc += (dw * da) * isum  in block order.
//
// One v_mfma_i32_32x32x32_i8 is exactly one block of a 32-token x 32-row tile: operand A is 16
// consecutive quants of token lane%32 (k half lane/32), operand B the same of weight row lane%32, and
// both formats already store their quants that way, so nothing is unpacked.  What a block costs is
// its float step: every one of the tile's 1024 sums has its own scale dw[row] * da[token].  That
// outer product is a second, tiny matrix product, and the f16 matrix cores compute it exactly (both
// factors are f16 values, their product has 22 significant bits): v_mfma_f32_32x32x8_f16 with da in
// k = 0 of A, dw in k = 0 of B and zeros elsewhere returns the scales in the very register layout of
// the integer sums.  Left to the vector ALU are a conversion and a fused multiply-add per sum: 32
// instructions a block.
//
// A workgroup of TT x RT wavefronts owns 32*TT tokens x 32*RT rows, one tile per wavefront, and walks
// the columns 256 (8 blocks) at a time: quants go global -> registers -> LDS, two chunks ahead of
// the multiplication; LDS holds the chunks of even and of odd number, so a round needs one barrier.
// An LDS row is 272 bytes -- 256 of quants, so that the 32 rows of a fragment read fall in different
// banks, and the row's eight f16 scales of the chunk in the 16 behind them.
//
// Measured at 4096 x 14336, M = 512 (128-token x 64-row workgroups, one per CU): 115 us.  With the
// float step taken out it is 95 us, with the multiplication taken out 63 us: the 688 MB that the 256
// workgroups pull out of L2 (every chunk of a tile is 48 KB for 4.2 M multiply-adds) cost about as
// much as the vector instructions do, and the two overlap only in part.
#include "frk_device.hpp"

#include <type_traits>

namespace frk {

typedef int q8_v4i __attribute__((ext_vector_type(4)));
typedef int q8_v16i __attribute__((ext_vector_type(16)));
typedef float q8_v16f __attribute__((ext_vector_type(16)));
typedef _Float16 q8_v4h __attribute__((ext_vector_type(4)));
typedef float q8_v4f __attribute__((ext_vector_type(4)));

struct Q8GemmArgs {
    const uint8_t *W;   // resident rows: quants [nb][32] (Q4_0: nibbles [nb][16]), then the f16 scales [nb]
    size_t row_stride, off_d;
    const int8_t *aq;   // [M][cols]
    const uint16_t *ad; // [M][nb rounded up to 8] f16 bits, zeros in the padding
    float *y;           // [M][rows]
    int rows, nb, M;
    int k_split;     // 1, or 2/4/8: blockIdx.z takes that share of the 256-column chunks (whole pairs of them)
    float *partial;  // [k_split][M][rows], added up in order afterwards
    // GROUPED: W stacks the groups' matrices of `rows` rows each; tile blockIdx.y = {group, first row of the grouped
    // order, rows in use, first row of y} multiplies the activation rows src_rows[first + r] (first + r without a list)
    const int4 *tiles;
    const int *n_tiles;
    const int *src_rows;
};

constexpr int Q8_CHUNK_BLOCKS = 8;   // 256 columns a step
constexpr int Q8_LDS_ROW = 272;      // 256 bytes of quants and 16 of padding

struct Q8Scales {  // a lane's eight block scales of one chunk, as f16 bit pairs; zero in lanes 32..63
    uint32_t w0, w1, w2, w3;
};

__device__ __forceinline__ uint32_t q8_pick(const Q8Scales &s, int b) {
    const uint32_t w = (b >> 1) == 0 ? s.w0 : (b >> 1) == 1 ? s.w1 : (b >> 1) == 2 ? s.w2 : s.w3;
    return (b & 1) ? (w >> 16) : (w & 0xffffu);
}

__device__ __forceinline__ q8_v4h q8_as_k0(uint32_t h) {  // {h, 0, 0, 0}
    uint2 u = make_uint2(h, 0u);
    q8_v4h v;
    __builtin_memcpy(&v, &u, 8);
    return v;
}

// quantize_activations_q8, Avx form (crates/frink-quant/src/act_quant.rs:157-189), for the GEMM: the
// same quants as frk_quant.hip's kernel; the block scales leave as the f16 values they are, a token's
// scales padded with zeros to a multiple of eight so that the GEMM reads any chunk's eight in one load.
// Eight lanes per 32-value block.
// GLU: what is quantized is silu(x) * up, element by element (the intermediate in front of a down projection).
template <bool GLU>
__global__ __launch_bounds__(256) void quantize_q8_0_gemm_kernel(const float *__restrict__ x, const float *__restrict__ up, size_t n_blocks,
                                                                 int nb, int8_t *__restrict__ q, uint16_t *__restrict__ d) {
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t b = t >> 3;
    const bool live = b < n_blocks;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = reinterpret_cast<const float4 *>(x)[t];
    if (GLU && live) {
        const float4 u = reinterpret_cast<const float4 *>(up)[t];
        v = make_float4(silu_as_host(v.x) * u.x, silu_as_host(v.y) * u.y, silu_as_host(v.z) * u.z, silu_as_host(v.w) * u.w);
    }
    float amax = fmaxf(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))), 0.0f);
    for (int off = 4; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if (!live) return;
    const float scale = __fdiv_rn(amax, 127.0f);
    const float inv = amax != 0.0f ? __fdiv_rn(127.0f, amax) : 0.0f;
    auto quant = [&](float e) {
        const float r = rintf(e * inv);
        // (f32::clamp keeps a NaN, which `as i8` turns into 0; fmaxf would turn it into -127)
        return (r != r) ? 0 : (int)fminf(fmaxf(r, -127.0f), 127.0f);
    };
    const int q0 = quant(v.x), q1 = quant(v.y), q2 = quant(v.z), q3 = quant(v.w);
    reinterpret_cast<uint32_t *>(q)[t] = (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) |
                                         ((uint32_t)(q2 & 0xff) << 16) | ((uint32_t)(q3 & 0xff) << 24);
    if ((t & 7) == 0) {
        const int stride = (nb + 7) & ~7;
        const size_t tok = b / (size_t)nb;
        const int in_row = (int)(b % (size_t)nb);
        d[tok * stride + in_row] = f2h_bits(scale);
        if (in_row == nb - 1)
            for (int i = nb; i < stride; i++) d[tok * stride + i] = 0;
    }
}

template <int AP, int WP>
struct Q8Stage {  // one chunk's share of a thread on its way from global memory to LDS
    q8_v4i a[AP], w[WP];  // 16-byte pieces of the activation and weight tiles
    q8_v4i s;             // the eight f16 scales of one weight row or token (the first wavefronts only)
};

// Four nibbles of Q4_0 (one per byte of t, already XOR-ed with 8) as the signed bytes nibble - 8:
// n - 8 is the four-bit two's complement value n ^ 8, so bit 3 is copied into bits 4..7 -- 0xF0 per
// byte that has it, as (m << 5) - (m << 1) of the mask m (no byte's 0xF0 reaches its neighbour).
__device__ __forceinline__ int q4_0_bytes(uint32_t t) {
    const uint32_t m = t & 0x08080808u;
    return (int)(t | ((m << 5) - (m << 1)));
}

// Q4: the weights are Q4_0 (dot_q4_0_q8, crates/frink-quant/src/lib.rs:772-796) -- 16 bytes of nibbles a
// block, byte i holding element i low and element i + 16 high -- and become the same signed bytes
// nibble - 8 on their way from the staging registers to LDS; everything behind that is the Q8_0 kernel.
//
// SUB: blocks with an integer scale of their own under a float scale per 256 (IQ4_XS decoded to signed bytes:
// dot_iq4_xs_q8k, crates/frink-quant/src/iq4_xs_q8.rs:50-67), against Q8_K activations -- the 16 bytes behind a
// weight row's chunk hold the eight block scales ls - 32 as signed bytes and the f16 d, a token's hold its f32 d.
// A block's sums are multiplied by its integer scale and added up as integers; once a chunk (one block of 256)
// the integers meet the float scales d_w * d_a, whose outer product a v_mfma_f32_32x32x2f32 returns in the
// registers' layout.
//
// GROUPED: the indexed form (enqueue_mul_mm_grouped_dev, crates/frink-cuda/src/mul_mm_launch.rs:391-470; the MoE
// prefill over experts of these kinds): a workgroup's tokens are one tile of at most 32 * TT rows of one group, the
// activation rows come through a list, and the results go to the tile's rows of y.
template <int TT, int RT, bool Q4, bool SUB = false, bool GROUPED = false>
__global__ __launch_bounds__(64 * TT * RT) void gemm_q8_0_mfma_kernel(Q8GemmArgs g) {
    constexpr int NT = 64 * TT * RT;
    // 16-byte pieces a thread stages per chunk (a piece of Q4_0 nibbles is a whole block)
    constexpr int AP = TT * 512 / NT, WP = (Q4 ? RT * 256 : RT * 512) / NT;
    // two copies of the tiles' chunk: the chunks of even and of odd number
    constexpr int LDS_A = TT * 32 * Q8_LDS_ROW, LDS_COPY = (TT + RT) * 32 * Q8_LDS_ROW;
    extern __shared__ __align__(16) uint8_t q8_lds[];
    uint8_t *const lds_a = q8_lds, *const lds_w = q8_lds + LDS_A;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tt = wave % TT, rt = wave / TT;
    const int row0 = blockIdx.x * (32 * RT);
    int tok0 = blockIdx.y * (32 * TT), tok_end = g.M, y_shift = 0;  // tokens tok0 .. tok_end - 1; token t is row t + y_shift of y
    if (GROUPED) {
        if ((int)blockIdx.y >= *g.n_tiles) return;
        const int4 tile = g.tiles[blockIdx.y];
        g.W += (size_t)tile.x * g.rows * g.row_stride;
        tok0 = tile.y;
        tok_end = tile.y + tile.z;
        y_shift = tile.w - tile.y;
    }
    // the activation row of token t (past the end: the last one again)
    auto act_row = [&](int t) {
        t = max(min(t, tok_end - 1), tok0);
        return GROUPED && g.src_rows ? max(g.src_rows[t], 0) : t;
    };
    const size_t cols = (size_t)g.nb * 32;
    const int n_chunks = (g.nb + Q8_CHUNK_BLOCKS - 1) / Q8_CHUNK_BLOCKS;
    // this workgroup's chunks c0 .. c1 - 1; c0 is even, so that the chunks of even number are the same
    // everywhere
    const int pairs = (n_chunks + 1) / 2;
    const int c0 = 2 * (pairs * (int)blockIdx.z / g.k_split), c1 = min(n_chunks, 2 * (pairs * ((int)blockIdx.z + 1) / g.k_split));

    // The 16-byte pieces this thread stages: piece j is byte 16*p of row r0 + j*NT/16 of either tile.
    const int r0 = tid >> 4, p = tid & 15;
    const int rq = tid >> 3, pq = tid & 7;  // Q4_0: piece j is block pq of row rq + j*NT/8
    const uint8_t *a_src = (const uint8_t *)g.aq;
    const uint8_t *w_src = g.W;
    const int stage_dst = r0 * Q8_LDS_ROW + p * 16;
    // The scales ride in the 16 bytes behind a row's quants in LDS.  Thread i of the first
    // (RT + TT) / 2 wavefronts stages those of weight row i, or of token i - 32 * RT, of the tile.
    const bool stages_scales = wave < (RT + TT) / 2;
    const bool stages_weight_scales = tid < 32 * RT;
    // (SUB: a token's scales are one f32 per chunk, [M][nb / 8])
    const uint8_t *s_src = stages_weight_scales
                               ? g.W + (size_t)min(row0 + tid, g.rows - 1) * g.row_stride + g.off_d
                               : SUB ? (const uint8_t *)g.ad + (size_t)act_row(tok0 + tid - 32 * RT) * (g.nb / 8) * 4
                                     : (const uint8_t *)(g.ad + (size_t)act_row(tok0 + tid - 32 * RT) * ((g.nb + 7) & ~7));
    uint8_t *s_dst = stages_weight_scales ? lds_w + tid * Q8_LDS_ROW + 256 : lds_a + (tid - 32 * RT) * Q8_LDS_ROW + 256;
    const bool low_half = lane < 32;
    const int n_full = g.nb / Q8_CHUNK_BLOCKS;  // chunks of eight whole blocks

    q8_v16f acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    const q8_v16i zero_i = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const q8_v16f zero_f = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    const uint8_t *frag_a = lds_a + (tt * 32 + (lane & 31)) * Q8_LDS_ROW + (lane >> 5) * 16;
    const uint8_t *frag_w = lds_w + (rt * 32 + (lane & 31)) * Q8_LDS_ROW + (lane >> 5) * 16;

    int a_rows[AP];  // the activation rows of this thread's pieces
#pragma unroll
    for (int i = 0; i < AP; i++) a_rows[i] = act_row(tok0 + r0 + i * (NT / 16));
    Q8Scales sa, sw;
    // The loads of a chunk: quant piece i < AP + WP, or (i == AP + WP) the scales.  `whole` says that the
    // chunk is known to be eight whole blocks.
    auto fetch = [&](int i, int chunk, bool whole, Q8Stage<AP, WP> &in) {
        const int blk0 = chunk * Q8_CHUNK_BLOCKS;
        // Rows past the end repeat the last row, and pieces past the row's end its first piece:
        // every load is inside the operand.  What they return meets a zero scale or an output
        // that is not stored.
        const size_t piece = whole || blk0 + (p >> 1) < g.nb ? (size_t)blk0 * 32 + p * 16 : 0;
        if (i < AP) {
            in.a[i] = *reinterpret_cast<const q8_v4i *>(a_src + (size_t)a_rows[i] * cols + piece);
        } else if (i < AP + WP) {
            if (Q4) {
                const int row = min(row0 + rq + (i - AP) * (NT / 8), g.rows - 1);
                const size_t nibbles = whole || blk0 + pq < g.nb ? (size_t)(blk0 + pq) * 16 : 0;
                in.w[i - AP] = *reinterpret_cast<const q8_v4i *>(w_src + (size_t)row * g.row_stride + nibbles);
            } else {
                const int row = min(row0 + r0 + (i - AP) * (NT / 16), g.rows - 1);
                in.w[i - AP] = *reinterpret_cast<const q8_v4i *>(w_src + (size_t)row * g.row_stride + piece);
            }
        } else if (stages_scales) {
            if (SUB && !stages_weight_scales) {
                in.s = q8_v4i{*reinterpret_cast<const int *>(s_src + (size_t)chunk * 4), 0, 0, 0};
            } else if (whole || !stages_weight_scales || blk0 + 8 <= g.nb) {
                // (a token's scales are padded with zeros to whole chunks)
                in.s = *reinterpret_cast<const q8_v4i *>(s_src + (size_t)blk0 * 2);
            } else {  // a weight row's last chunk when it is not a multiple of 256 columns
                const uint16_t *dh = reinterpret_cast<const uint16_t *>(s_src);
                auto wgt = [&](int b) { return blk0 + b < g.nb ? (int)dh[blk0 + b] : 0; };
#pragma unroll
                for (int b = 0; b < 4; b++) in.s[b] = wgt(2 * b) | (wgt(2 * b + 1) << 16);
            }
        }
    };
    // Round c asks for chunk c + 2 (into the registers `in`), multiplies chunk c out of LDS and then
    // moves chunk c + 1 (the registers `out`, asked for a round earlier) into LDS: a load has two
    // rounds to arrive.  Nothing may look at `in` within the round -- that would wait for its loads.
    constexpr int LOADS = AP + WP + 1, LOADS_A_BLOCK = (LOADS + Q8_CHUNK_BLOCKS - 1) / Q8_CHUNK_BLOCKS;
    // In the steady rounds (steady_tag) every condition is known to hold and is not tested (a branch
    // around the loads would make the waits in front of the LDS writes count as if none were issued),
    // and the loads are spread over the blocks of the multiplication: issued together, the eight
    // wavefronts' loads fill the CU's queue and hold up the wavefronts behind them.
    auto round = [&](auto steady_tag, int c, Q8Stage<AP, WP> &out, Q8Stage<AP, WP> &in) {
        constexpr bool STEADY = decltype(steady_tag)::value;
        if (!STEADY && c + 2 < c1) {
#pragma unroll
            for (int i = 0; i < LOADS; i++) fetch(i, c + 2, false, in);
        }
        if (STEADY || (c >= c0 && c < c1)) {
            // A three-stage pipeline over the blocks: the LDS reads of block b + 2, the matrix products
            // of block b + 1 and the float step of block b are issued in that order, so that reads
            // and products run in the shadow of the 32 vector instructions.
            auto frags = [&](int b, q8_v4i &qa, q8_v4i &qw) {
                qa = *reinterpret_cast<const q8_v4i *>(frag_a + (c & 1) * LDS_COPY + b * 32);
                qw = *reinterpret_cast<const q8_v4i *>(frag_w + (c & 1) * LDS_COPY + b * 32);
            };
            auto products = [&](int b, const q8_v4i &qa, const q8_v4i &qw, q8_v16i &isum, q8_v16f &scale) {
                isum = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa, qw, zero_i, 0, 0, 0);
                if (!SUB)
                    scale = __builtin_amdgcn_mfma_f32_32x32x8f16(q8_as_k0(q8_pick(sa, b)), q8_as_k0(q8_pick(sw, b)), zero_f, 0, 0, 0);
            };
            uint32_t ls_lo = 0, ls_hi = 0;  // SUB: this lane's weight row's eight block scales, a signed byte each
            float sub_da = 0.0f, sub_dw = 0.0f;
            {
                const q8_v4i va = *reinterpret_cast<const q8_v4i *>(frag_a + (c & 1) * LDS_COPY - (lane >> 5) * 16 + 256);
                const q8_v4i vw = *reinterpret_cast<const q8_v4i *>(frag_w + (c & 1) * LDS_COPY - (lane >> 5) * 16 + 256);
                if (SUB) {
                    ls_lo = (uint32_t)vw[0], ls_hi = (uint32_t)vw[1];
                    sub_da = low_half ? __uint_as_float((uint32_t)va[0]) : 0.0f;
                    sub_dw = low_half ? h2f((uint32_t)vw[2] & 0xffffu) : 0.0f;
                }
                sa = Q8Scales{low_half ? (uint32_t)va[0] : 0u, low_half ? (uint32_t)va[1] : 0u, low_half ? (uint32_t)va[2] : 0u,
                              low_half ? (uint32_t)va[3] : 0u};
                sw = Q8Scales{low_half ? (uint32_t)vw[0] : 0u, low_half ? (uint32_t)vw[1] : 0u, low_half ? (uint32_t)vw[2] : 0u,
                              low_half ? (uint32_t)vw[3] : 0u};
            }
            q8_v16i iacc = zero_i;
            q8_v4i qa1, qw1, qa2, qw2;
            q8_v16i isum_next;
            q8_v16f scale_next;
            frags(0, qa1, qw1);
            frags(1, qa2, qw2);
            products(0, qa1, qw1, isum_next, scale_next);
            qa1 = qa2, qw1 = qw2;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < Q8_CHUNK_BLOCKS; b++) {
                const q8_v16i isum = isum_next;
                const q8_v16f scale = scale_next;
                if (b + 2 < Q8_CHUNK_BLOCKS) frags(b + 2, qa2, qw2);
                if (b + 1 < Q8_CHUNK_BLOCKS) products(b + 1, qa1, qw1, isum_next, scale_next);
                if (STEADY) {
#pragma unroll
                    for (int i = b * LOADS_A_BLOCK; i < (b + 1) * LOADS_A_BLOCK && i < LOADS; i++) fetch(i, c + 2, true, in);
                }
                if (SUB) {
                    // |ls| <= 32 and |isum| <= 32 * 127 * 127: 24-bit factors, and eight blocks' products fit 32 bits
                    const int ls = (int)(int8_t)(((b < 4 ? ls_lo : ls_hi) >> (8 * (b & 3))) & 0xff);
#pragma unroll
                    for (int r = 0; r < 16; r++) iacc[r] = __mul24(isum[r], ls) + iacc[r];
                    if (b == Q8_CHUNK_BLOCKS - 1) {
                        const q8_v16f dd = __builtin_amdgcn_mfma_f32_32x32x2f32(sub_da, sub_dw, zero_f, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[r] = __builtin_fmaf(dd[r], (float)iacc[r], acc[r]);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[r] = __builtin_fmaf(scale[r], (float)isum[r], acc[r]);
                }
                if (b + 2 < Q8_CHUNK_BLOCKS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // LDS reads
                if (b + 1 < Q8_CHUNK_BLOCKS) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // MFMAs
                // keeps the float step here: sunk towards the loop's end it would leave every
                // block's matrix results alive at once
                asm volatile("" : "+v"(acc));
                if (SUB) asm volatile("" : "+v"(iacc));
                __builtin_amdgcn_sched_barrier(0);
                qa1 = qa2, qw1 = qw2;
            }
        }
        if (STEADY || (c + 1 >= c0 && c + 1 < c1)) {
            // chunk c + 1 goes into the copy that chunk c - 1 was read from: every wavefront finished
            // with that before the barrier that ended the last round
            const int to = ((c + 1) & 1) * LDS_COPY;
#pragma unroll
            for (int j = 0; j < AP; j++) *reinterpret_cast<q8_v4i *>(lds_a + to + stage_dst + j * (NT / 16) * Q8_LDS_ROW) = out.a[j];
#pragma unroll
            for (int j = 0; j < WP; j++) {
                if (Q4) {
                    const q8_v4i v = out.w[j];
                    q8_v4i lo, hi;
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const uint32_t wv = (uint32_t)v[k];
                        lo[k] = q4_0_bytes((wv & 0x0f0f0f0fu) ^ 0x08080808u);
                        hi[k] = q4_0_bytes(((wv >> 4) & 0x0f0f0f0fu) ^ 0x08080808u);
                    }
                    uint8_t *dst = lds_w + to + (rq + j * (NT / 8)) * Q8_LDS_ROW + pq * 32;
                    *reinterpret_cast<q8_v4i *>(dst) = lo;
                    *reinterpret_cast<q8_v4i *>(dst + 16) = hi;
                } else {
                    *reinterpret_cast<q8_v4i *>(lds_w + to + stage_dst + j * (NT / 16) * Q8_LDS_ROW) = out.w[j];
                }
            }
            if (stages_scales) *reinterpret_cast<q8_v4i *>(s_dst + to) = out.s;
        }
        lds_barrier();  // one barrier a round (it does not wait for the loads on their way)
    };
    Q8Stage<AP, WP> even, odd;  // the chunks of either parity on their way
    const std::false_type any;
    const std::true_type steady;
    round(any, c0 - 2, odd, even);
    round(any, c0 - 1, even, odd);
    int c = c0;
    for (; c + 3 < min(n_full, c1); c += 2) {  // the chunks these rounds ask for, c + 2 and c + 3, are whole and ours
        round(steady, c, odd, even);
        round(steady, c + 1, even, odd);
    }
    for (; c < c1; c += 2) {
        round(any, c, odd, even);
        round(any, c + 1, even, odd);
    }

    // D register r of lane l is token 8*(r/4) + 4*(l/32) + r%4, weight row l%32 of the tile
    const int row = row0 + rt * 32 + (lane & 31);
    float *const dst = g.k_split > 1 ? g.partial + (size_t)blockIdx.z * g.M * g.rows : g.y;
    if (row < g.rows) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int tok = tok0 + tt * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (tok < tok_end) dst[(size_t)(tok + y_shift) * g.rows + row] = acc[r];
        }
    }
}

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

constexpr int Q8_MAX_SPLIT = 8;
// A small grid (few token tiles, a short matrix) splits the chunks of a row between 2, 4 or 8
// workgroups, no finer than two pairs of chunks each; their sums are added in order afterwards.
static int q8_0_split(size_t rows, size_t M, size_t nb32) {
    const size_t wgs = M > 32 ? ((rows + 63) / 64) * ((M + 127) / 128) : (rows + 31) / 32;
    const size_t pairs = ((nb32 + Q8_CHUNK_BLOCKS - 1) / Q8_CHUNK_BLOCKS + 1) / 2;
    int ks = 1;
    const size_t fill = M > 32 ? 256 : 1024;  // (the one-wavefront workgroups of the thinnest batches: four per CU)
    while (ks < Q8_MAX_SPLIT && wgs * ks * 2 <= fill && pairs / (size_t)(ks * 2) >= 2) ks *= 2;
    return ks;
}
// the quantized activations, their scales, and room for the parts' sums where the chunks are split
size_t gemm_q8_0_workspace_bytes(size_t M, size_t cols, size_t rows) {
    const int ks = q8_0_split(rows, M, cols / 32);
    return round_up(M * cols, 256) + round_up(M * round_up(cols / 32, 8) * 2, 256) + (ks > 1 ? (size_t)ks * M * rows * sizeof(float) : 0);
}

static int launch_q8_mfma(Q8GemmArgs g, bool q4, bool sub, hipStream_t s);

int launch_gemm_q8_0(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s) {
    return launch_gemm_q8_0_planar(w->dev, w->layout.row_stride, w->layout.off_a, w->rows, w->cols, w->kind == FRK_KIND_Q4_0, x, M, y,
                                   ws, s);
}

// The same over any rows in the planar form -- quants [nb][32] (q4: nibbles [nb][16]), then the f16 scales [nb] at
// off_d of every row: the resident Q8_0 / Q4_0 matrices, and other 32-element kinds decoded into that form.
int launch_gemm_q8_0_planar(const uint8_t *W, size_t row_stride, size_t off_d, size_t rows, size_t cols, bool q4, const float *x,
                            size_t M, float *y, void *ws, hipStream_t s) {
    if (M > (size_t)1 << 30 || rows > (size_t)1 << 30)
        return set_error(FRK_ERR_SHAPE, "gemm_q8_0: %zu activation rows x %zu weight rows is too many", M, rows);
    struct {
        size_t rows, cols;
    } dims = {rows, cols};
    const auto *w = &dims;
    int8_t *aq = (int8_t *)ws;
    uint16_t *ad = (uint16_t *)((char *)ws + round_up(M * w->cols, 256));
    const size_t n_blocks = M * (w->cols / 32);
    hipLaunchKernelGGL(quantize_q8_0_gemm_kernel<false>, dim3((unsigned)((n_blocks * 8 + 255) / 256)), dim3(256), 0, s, x,
                       (const float *)nullptr, n_blocks, (int)(w->cols / 32), aq, ad);
    FRK_LAUNCH_CHECK("quantize_q8_0_gemm");
    Q8GemmArgs g;
    g.W = W;
    g.row_stride = row_stride;
    g.off_d = off_d;
    g.aq = aq;
    g.ad = ad;
    g.y = y;
    g.rows = (int)w->rows;
    g.nb = (int)(w->cols / 32);
    g.M = (int)M;
    g.partial = reinterpret_cast<float *>((char *)ws + round_up(M * w->cols, 256) + round_up(M * round_up(w->cols / 32, 8) * 2, 256));
    g.tiles = nullptr;
    g.n_tiles = nullptr;
    g.src_rows = nullptr;
    return launch_q8_mfma(g, q4, false, s);
}

// The kernel over operands that are ready: the widest token tile the batch fills; two row tiles per workgroup
// with it, one wavefront a workgroup for the thinnest batches, whose grids are small.  g.partial: room for the
// parts' sums where the chunks are split (q8_0_split).
static int launch_q8_mfma(Q8GemmArgs g, bool q4, bool sub, hipStream_t s) {
    auto lds_bytes = [](int tt, int rt) { return (size_t)2 * (tt + rt) * 32 * Q8_LDS_ROW; };
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        const void *big[6] = {reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<4, 2, false>),
                              reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<4, 2, true>),
                              reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<2, 2, false>),
                              reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<2, 2, true>),
                              reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<4, 2, false, true>),
                              reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<2, 2, false, true>)};
        for (int i = 0; i < 6; i++) {
            hipError_t e = hipFuncSetAttribute(big[i], hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(4, 2));
            if (e != hipSuccess)
                return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(LDS %zu): %s", lds_bytes(4, 2), hipGetErrorString(e));
        }
        sized = true;
    }
    const size_t rows = (size_t)g.rows, M = (size_t)g.M;
    const int ks = q8_0_split(rows, M, (size_t)g.nb);
    g.k_split = ks;
    const unsigned kz = (unsigned)ks;
#define FRK_GO(TT, RT, grid, threads)                                                                                        \
    do {                                                                                                                     \
        if (sub) hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<TT, RT, false, true>), grid, dim3(threads), lds_bytes(TT, RT), s, g); \
        else if (q4) hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<TT, RT, true>), grid, dim3(threads), lds_bytes(TT, RT), s, g);  \
        else hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<TT, RT, false>), grid, dim3(threads), lds_bytes(TT, RT), s, g);         \
    } while (0)
    if (M > 64) {
        const dim3 grid((unsigned)((rows + 63) / 64), (unsigned)((M + 127) / 128), kz);
        FRK_GO(4, 2, grid, 512);
    } else if (M > 32) {
        const dim3 grid((unsigned)((rows + 63) / 64), 1u, kz);
        FRK_GO(2, 2, grid, 256);
    } else {
        const dim3 grid((unsigned)((rows + 31) / 32), 1u, kz);
        FRK_GO(1, 1, grid, 64);
    }
#undef FRK_GO
    FRK_LAUNCH_CHECK("gemm_q8_0_mfma");
    if (ks > 1) return launch_sum_parts(g.partial, ks, M * rows, g.y, s);
    return FRK_OK;
}

// Rows of signed bytes with an integer scale per 32 and an f16 scale per 256 in the slots behind the quants (SUB
// above) against Q8_K activations: quants aq [M][cols], scales ad [M][cols / 256].  `partial`: room for
// gemm_sub_partial_bytes.
size_t gemm_sub_partial_bytes(size_t M, size_t cols, size_t rows) {
    const int ks = q8_0_split(rows, M, cols / 32);
    return ks > 1 ? (size_t)ks * M * rows * sizeof(float) : 0;
}
int launch_gemm_sub_planar(const uint8_t *W, size_t row_stride, size_t off_d, size_t rows, size_t cols, const int8_t *aq,
                           const float *ad, size_t M, float *y, void *partial, hipStream_t s) {
    if (M > (size_t)1 << 30 || rows > (size_t)1 << 30 || cols % QK_K)
        return set_error(FRK_ERR_SHAPE, "gemm_sub: %zu activation rows x %zu weight rows x %zu columns", M, rows, cols);
    Q8GemmArgs g;
    g.W = W;
    g.row_stride = row_stride;
    g.off_d = off_d;
    g.aq = aq;
    g.ad = reinterpret_cast<const uint16_t *>(ad);
    g.y = y;
    g.rows = (int)rows;
    g.nb = (int)(cols / 32);
    g.M = (int)M;
    g.partial = (float *)partial;
    g.tiles = nullptr;
    g.n_tiles = nullptr;
    g.src_rows = nullptr;
    return launch_q8_mfma(g, false, true, s);
}

// The grouped form over decoded rows (Q8_0 planar form, or with sub = true the form with integer block scales): W
// stacks the groups' matrices of rows_g rows; tiles / n_tiles as grouped_tiles and moe_group write them (tiles of at
// most 64 rows); activation row of grouped row r: src_rows[r], or r itself without a list.  aq / ad: the activations'
// quants and scales as the plain forms above take them ([..][cols]; f16 per 32 padded to eights, or f32 per 256).
int launch_gemm_planar_grouped(const uint8_t *W, size_t row_stride, size_t off_d, size_t rows_g, size_t cols, bool sub,
                               const int8_t *aq, const void *ad, const int *src_rows, const int4 *tiles, const int *n_tiles,
                               size_t max_tiles, float *y, hipStream_t s) {
    if (rows_g > (size_t)1 << 30 || max_tiles > 65535 || (sub && cols % QK_K))
        return set_error(FRK_ERR_SHAPE, "grouped gemm: %zu rows a group, %zu tiles, %zu columns", rows_g, max_tiles, cols);
    if (max_tiles == 0) return FRK_OK;
    Q8GemmArgs g;
    g.W = W;
    g.row_stride = row_stride;
    g.off_d = off_d;
    g.aq = aq;
    g.ad = reinterpret_cast<const uint16_t *>(ad);
    g.y = y;
    g.rows = (int)rows_g;
    g.nb = (int)(cols / 32);
    g.M = 0;
    g.k_split = 1;
    g.partial = nullptr;
    g.tiles = tiles;
    g.n_tiles = n_tiles;
    g.src_rows = src_rows;
    // 64 tokens x 128 rows a workgroup where the groups have the rows for it: a tile's bytes per multiply-add are what
    // bounds this kernel (32 MXFP4 experts top-4 of 2880/2880 at 512 tokens: 207 -> 137 us a projection), 64 x 64 else
    auto lds_bytes = [](int rt) { return (size_t)2 * (2 + rt) * 32 * Q8_LDS_ROW; };
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        const void *k[4] = {reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<2, 2, false, false, true>),
                            reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<2, 2, false, true, true>),
                            reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<2, 4, false, false, true>),
                            reinterpret_cast<const void *>(&gemm_q8_0_mfma_kernel<2, 4, false, true, true>)};
        for (int i = 0; i < 4; i++) {
            hipError_t e = hipFuncSetAttribute(k[i], hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(i < 2 ? 2 : 4));
            if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(LDS %zu): %s", lds_bytes(4), hipGetErrorString(e));
        }
        sized = true;
    }
    if (rows_g > 64) {
        const dim3 grid((unsigned)((rows_g + 127) / 128), (unsigned)max_tiles, 1u);
        if (sub) hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<2, 4, false, true, true>), grid, dim3(512), lds_bytes(4), s, g);
        else hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<2, 4, false, false, true>), grid, dim3(512), lds_bytes(4), s, g);
    } else {
        const dim3 grid((unsigned)((rows_g + 63) / 64), (unsigned)max_tiles, 1u);
        if (sub) hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<2, 2, false, true, true>), grid, dim3(256), lds_bytes(2), s, g);
        else hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<2, 2, false, false, true>), grid, dim3(256), lds_bytes(2), s, g);
    }
    FRK_LAUNCH_CHECK("gemm_planar_grouped");
    return FRK_OK;
}

// quantize_activations_q8 for the kernels above: quants [rows][cols], f16 scales [rows][cols / 32 rounded up to 8]
size_t q8_0_gemm_acts_bytes(size_t rows, size_t cols) { return round_up(rows * cols, 256) + round_up(rows * round_up(cols / 32, 8) * 2, 256); }
// (with `up`: silu(x) * up is what is quantized)
int launch_quantize_q8_0_gemm(const float *x, const float *up, size_t rows, size_t cols, int8_t *q, uint16_t *d, hipStream_t s) {
    const size_t n_blocks = rows * (cols / 32);
    if (n_blocks == 0) return FRK_OK;
    const dim3 grid((unsigned)((n_blocks * 8 + 255) / 256));
    if (up) hipLaunchKernelGGL(quantize_q8_0_gemm_kernel<true>, grid, dim3(256), 0, s, x, up, n_blocks, (int)(cols / 32), q, d);
    else hipLaunchKernelGGL(quantize_q8_0_gemm_kernel<false>, grid, dim3(256), 0, s, x, up, n_blocks, (int)(cols / 32), q, d);
    FRK_LAUNCH_CHECK("quantize_q8_0_gemm");
    return FRK_OK;
}

}  // namespace frk
