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
// the integer sums.  Left to the vector ALU are a conversion and a fused multiply-add per sum -- 32
// instructions a block, which is what bounds the kernel (an MFMA pair takes about 50 clocks, the 32
// instructions 128).
//
// A workgroup of TT x RT wavefronts owns 32*TT tokens x 32*RT rows, one tile per wavefront, and walks
// the columns 256 (8 blocks) at a time: quants go global -> registers -> LDS (rows padded to 272
// bytes so that the 32 rows of a fragment read fall in different banks), the next chunk's loads are
// in flight while the current one is multiplied.  A wavefront reads its own rows' 8 scales of the
// chunk straight from global memory, one chunk ahead as well.
#include "frk_device.hpp"

namespace frk {

typedef int q8_v4i __attribute__((ext_vector_type(4)));
typedef int q8_v16i __attribute__((ext_vector_type(16)));
typedef float q8_v16f __attribute__((ext_vector_type(16)));
typedef _Float16 q8_v4h __attribute__((ext_vector_type(4)));
typedef float q8_v4f __attribute__((ext_vector_type(4)));

struct Q8GemmArgs {
    const uint8_t *W;   // resident rows: quants [nb][32], then the f16 scales [nb]
    size_t row_stride, off_d;
    const int8_t *aq;   // [M][cols]
    const float *ad;    // [M][nb], every value an f16 value
    float *y;           // [M][rows]
    int rows, nb, M;
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

template <int TT, int RT>
__global__ __launch_bounds__(64 * TT * RT) void gemm_q8_0_mfma_kernel(Q8GemmArgs g) {
    constexpr int NT = 64 * TT * RT;
    constexpr int AP = TT * 512 / NT, WP = RT * 512 / NT;  // 16-byte pieces a thread stages per chunk
    __shared__ __align__(16) uint8_t lds_a[TT * 32 * Q8_LDS_ROW];
    __shared__ __align__(16) uint8_t lds_w[RT * 32 * Q8_LDS_ROW];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tt = wave % TT, rt = wave / TT;
    const int tok0 = blockIdx.y * (32 * TT), row0 = blockIdx.x * (32 * RT);
    const size_t cols = (size_t)g.nb * 32;
    const int n_chunks = (g.nb + Q8_CHUNK_BLOCKS - 1) / Q8_CHUNK_BLOCKS;

    // The 16-byte pieces this thread stages: piece j is byte 16*p of row r0 + j*NT/16 of either tile.
    const int r0 = tid >> 4, p = tid & 15;
    const uint8_t *a_src = (const uint8_t *)g.aq;
    const uint8_t *w_src = g.W;
    const int stage_dst = r0 * Q8_LDS_ROW + p * 16;
    // the wavefront's own tile: token and weight row of this lane's operand fragments and scales
    const int my_tok = min(tok0 + tt * 32 + (lane & 31), g.M - 1);
    const int my_row = min(row0 + rt * 32 + (lane & 31), g.rows - 1);
    const float *da_src = g.ad + (size_t)my_tok * g.nb;
    const uint8_t *dw_src = g.W + (size_t)my_row * g.row_stride + g.off_d;
    const bool low_half = lane < 32;
    const bool da_vec = (g.nb & 3) == 0;  // a token's scales then start 16-byte aligned

    q8_v16f acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    const q8_v16i zero_i = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const q8_v16f zero_f = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    const uint8_t *frag_a = lds_a + (tt * 32 + (lane & 31)) * Q8_LDS_ROW + (lane >> 5) * 16;
    const uint8_t *frag_w = lds_w + (rt * 32 + (lane & 31)) * Q8_LDS_ROW + (lane >> 5) * 16;

    Q8Scales sa = {0u, 0u, 0u, 0u}, sw = {0u, 0u, 0u, 0u};
    // round c multiplies chunk c while chunk c + 1 is on its way into registers; round -1 only fetches
    for (int c = -1; c < n_chunks; c++) {
        const bool more = c + 1 < n_chunks;
        // vector values, not structs (a struct picked by a condition goes through memory), and nothing
        // here may look at what a load returns: that would wait for it before the multiplication
        q8_v4i a_reg[AP], w_reg[WP], dw_raw = {0, 0, 0, 0};
        q8_v4f da_lo = {0.f, 0.f, 0.f, 0.f}, da_hi = {0.f, 0.f, 0.f, 0.f};
        if (more) {
            const int blk0 = (c + 1) * Q8_CHUNK_BLOCKS;
            // Rows past the end repeat the last row, and pieces past the row's end its first piece:
            // every load is inside the operand.  What they return meets a zero scale or an
            // output that is not stored.
            const size_t piece = blk0 + (p >> 1) < g.nb ? (size_t)blk0 * 32 + p * 16 : 0;
#pragma unroll
            for (int j = 0; j < AP; j++) {
                const int tok = min(tok0 + r0 + j * (NT / 16), g.M - 1);
                a_reg[j] = *reinterpret_cast<const q8_v4i *>(a_src + (size_t)tok * cols + piece);
            }
#pragma unroll
            for (int j = 0; j < WP; j++) {
                const int row = min(row0 + r0 + j * (NT / 16), g.rows - 1);
                w_reg[j] = *reinterpret_cast<const q8_v4i *>(w_src + (size_t)row * g.row_stride + piece);
            }
            // scales: blocks past the end count as zero
            if (blk0 + 8 <= g.nb) {
                if (da_vec) {
                    da_lo = *reinterpret_cast<const q8_v4f *>(da_src + blk0);
                    da_hi = *reinterpret_cast<const q8_v4f *>(da_src + blk0 + 4);
                } else {
#pragma unroll
                    for (int b = 0; b < 4; b++) da_lo[b] = da_src[blk0 + b], da_hi[b] = da_src[blk0 + 4 + b];
                }
                dw_raw = *reinterpret_cast<const q8_v4i *>(dw_src + (size_t)blk0 * 2);
            } else {  // the last chunk of a row that is not a multiple of 256 columns
                const uint16_t *dh = reinterpret_cast<const uint16_t *>(dw_src);
                auto act = [&](int b) { return blk0 + b < g.nb ? da_src[blk0 + b] : 0.0f; };
                auto wgt = [&](int b) { return blk0 + b < g.nb ? (int)dh[blk0 + b] : 0; };
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    da_lo[b] = act(b), da_hi[b] = act(4 + b);
                    dw_raw[b] = wgt(2 * b) | (wgt(2 * b + 1) << 16);
                }
            }
        }
        if (c >= 0) {
            // the matrix cores run one block ahead of the float step
            auto products = [&](int b, q8_v16i &isum, q8_v16f &scale) {
                const q8_v4i qa = *reinterpret_cast<const q8_v4i *>(frag_a + b * 32);
                const q8_v4i qw = *reinterpret_cast<const q8_v4i *>(frag_w + b * 32);
                isum = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa, qw, zero_i, 0, 0, 0);
                scale = __builtin_amdgcn_mfma_f32_32x32x8f16(q8_as_k0(q8_pick(sa, b)), q8_as_k0(q8_pick(sw, b)), zero_f, 0, 0, 0);
            };
            q8_v16i isum_next;
            q8_v16f scale_next;
            products(0, isum_next, scale_next);
#pragma unroll
            for (int b = 0; b < Q8_CHUNK_BLOCKS; b++) {
                const q8_v16i isum = isum_next;
                const q8_v16f scale = scale_next;
                if (b + 1 < Q8_CHUNK_BLOCKS) products(b + 1, isum_next, scale_next);
#pragma unroll
                for (int r = 0; r < 16; r++) acc[r] = __builtin_fmaf(scale[r], (float)isum[r], acc[r]);
                // keeps the float step here: sunk towards the loop's end it would leave every
                // block's matrix results alive at once
                asm volatile("" : "+v"(acc));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (!more) break;
        __syncthreads();  // every wavefront has read the chunk in LDS
#pragma unroll
        for (int j = 0; j < AP; j++) *reinterpret_cast<q8_v4i *>(lds_a + stage_dst + j * (NT / 16) * Q8_LDS_ROW) = a_reg[j];
#pragma unroll
        for (int j = 0; j < WP; j++) *reinterpret_cast<q8_v4i *>(lds_w + stage_dst + j * (NT / 16) * Q8_LDS_ROW) = w_reg[j];
        auto pair = [](float lo, float hi) { return (uint32_t)f2h_bits(lo) | ((uint32_t)f2h_bits(hi) << 16); };
        sa = Q8Scales{low_half ? pair(da_lo[0], da_lo[1]) : 0u, low_half ? pair(da_lo[2], da_lo[3]) : 0u,
                      low_half ? pair(da_hi[0], da_hi[1]) : 0u, low_half ? pair(da_hi[2], da_hi[3]) : 0u};
        sw = Q8Scales{low_half ? (uint32_t)dw_raw[0] : 0u, low_half ? (uint32_t)dw_raw[1] : 0u,
                      low_half ? (uint32_t)dw_raw[2] : 0u, low_half ? (uint32_t)dw_raw[3] : 0u};
        __syncthreads();
    }

    // D register r of lane l is token 8*(r/4) + 4*(l/32) + r%4, weight row l%32 of the tile
    const int row = row0 + rt * 32 + (lane & 31);
    if (row < g.rows) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int tok = tok0 + tt * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (tok < g.M) g.y[(size_t)tok * g.rows + row] = acc[r];
        }
    }
}

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

size_t gemm_q8_0_workspace_bytes(size_t M, size_t cols) {
    return round_up(M * cols, 256) + round_up(M * (cols / 32) * 4, 256);
}

int launch_gemm_q8_0(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s) {
    if (M > (size_t)1 << 30 || w->rows > (size_t)1 << 30)
        return set_error(FRK_ERR_SHAPE, "gemm_q8_0: %zu activation rows x %zu weight rows is too many", M, w->rows);
    int8_t *aq = (int8_t *)ws;
    float *ad = (float *)((char *)ws + round_up(M * w->cols, 256));
    int rc = launch_quantize_q8_0(x, M * w->cols, aq, ad, s);
    if (rc) return rc;
    Q8GemmArgs g;
    g.W = w->dev;
    g.row_stride = w->layout.row_stride;
    g.off_d = w->layout.off_a;
    g.aq = aq;
    g.ad = ad;
    g.y = y;
    g.rows = (int)w->rows;
    g.nb = (int)(w->cols / 32);
    g.M = (int)M;
    // the widest token tile the batch fills; two row tiles per workgroup with it, one wavefront a
    // workgroup for the thinnest batches, whose grids are small
    if (M > 64) {
        const dim3 grid((unsigned)((w->rows + 63) / 64), (unsigned)((M + 127) / 128));
        hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<4, 2>), grid, dim3(512), 0, s, g);
    } else if (M > 32) {
        const dim3 grid((unsigned)((w->rows + 63) / 64), 1u);
        hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<2, 2>), grid, dim3(256), 0, s, g);
    } else {
        const dim3 grid((unsigned)((w->rows + 31) / 32), 1u);
        hipLaunchKernelGGL((gemm_q8_0_mfma_kernel<1, 1>), grid, dim3(64), 0, s, g);
    }
    FRK_LAUNCH_CHECK("gemm_q8_0_mfma");
    return FRK_OK;
}

}  // namespace frk
