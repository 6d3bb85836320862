// Prefill / batched GEMM over Q4_K weights on the int8 matrix cores:
//   y[tok][row] = sum_k W[row][k] * x[tok][k],  x quantized per token to Q8_K first.
//
// Arithmetic is dot_q4_k_q8's (crates/frink-quant/src/lib.rs:822-869), regrouped so that a whole
// 256-weight block accumulates in int32 inside the MFMA:
//   sum_j sc_j * isum_j      with sc_j = 8*sh_j + sl_j (sh, sl < 8): a weight row's block becomes two
//                            int8 operand planes  H = sh_j * q  and  L = sl_j * q  (each < 106), so
//                            sum = 8 * (acts . H) + (acts . L), exact, no per-sub-block rescale;
//   sum_j m_j * bsum_j       the activation's 16-wide sums are split as bsum = 64*hi + lo (both int8)
//                            and multiplied by the 6-bit mins on the K=16 MFMA: 64*(hi . m) + (lo . m).
// Per block and output the epilogue is then  acc += da * (d * S1 - dmin * S2)  in f32.
// (Scaling each sub-block's product after a K=32 MFMA instead -- one v_mad_i32_i24 per result and
// sub-block -- was measured slower here: it is bound by the vector ALU and needs more registers.)
//
// MFMA operand roles: A = activations (tile row = token), B = weights (tile column = weight row), so
// a lane's 16 results share one weight row (its d, dmin are per-lane values) and span 16 tokens.
// Operand layout of v_mfma_i32_32x32x32_i8 (checked on the device): lane l holds, for row/column
// l % 32, the 16 k-values 16*(l/32) .. +15; result register r of lane l is
// D[8*(r/4) + 4*(l/32) + r%4][l % 32].
#include "frk_device.hpp"

namespace frk {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned short us2 __attribute__((ext_vector_type(2)));

constexpr int GM_LDW = 272;  // LDS bytes per token and block: 256 quants + 16 of padding (bank spread)

// Activation side: Q8_K quantization plus the base-64 digits of the 16-wide sums.
// One wavefront per 256-value block.
__global__ __launch_bounds__(256) void quantize_q8_k_gemm_kernel(const float *__restrict__ x, size_t n_blocks,
                                                                 int8_t *__restrict__ q, float *__restrict__ d,
                                                                 int8_t *__restrict__ bs_hi,
                                                                 int8_t *__restrict__ bs_lo) {
    const int lane = threadIdx.x & 63;
    const size_t b = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= n_blocks) return;
    const float4 v = reinterpret_cast<const float4 *>(x + b * QK_K)[lane];
    float dd;
    int bs;
    const uint32_t packed = quantize_q8_k_lane(v, dd, bs);
    reinterpret_cast<uint32_t *>(q + b * QK_K)[lane] = packed;
    if ((lane & 3) == 0) {
        bs_hi[b * 16 + (lane >> 2)] = (int8_t)(bs >> 6);  // floor(bs / 64) in [-32, 31]
        bs_lo[b * 16 + (lane >> 2)] = (int8_t)(bs & 63);
    }
    if (lane == 0) d[b] = dd;
}

struct GemmArgs {
    const uint8_t *W;
    size_t row_stride;
    int rows, nb, M;
    const int8_t *aq;     // [M][nb*256]
    const float *ad;      // [M][nb]
    const int8_t *bs_hi;  // [M][nb*16]
    const int8_t *bs_lo;
    float *y;             // [M][rows]
    int row_tiles, tok_tiles;
    // grouped (per-expert) form: tile t covers output rows first..first+count of expert e, whose
    // weights are rows [e*rows, (e+1)*rows) of W; activation row of output row p is gather[p]
    // (p itself when gather is null).  Tiles past *n_tiles exit at once.
    const int4 *tiles;    // {expert, first, count, 0}
    const int *n_tiles;
    const int *gather;
};

// One block's worth of global loads in flight: a lane's weights and a thread's share of the
// activation tile, requested one block-iteration before they are needed.
struct GemmPrefetch {
    uint4 wh, wq0, wq1, wq2, wq3;  // header, the lane's 16-byte half of each 32-byte nibble pair
    uint4 sa0, sa1, sa2, sa3, sdig;
    float sda;
};

// A wavefront owns 32 weight rows and keeps their current block in registers, already unpacked
// into MFMA B operands (a lane holds k = 16g..16g+15 of row l%32 for each of the 8 sub-blocks).
// The workgroup has 4*WT wavefronts: four row groups (128 rows) times WT token groups of 32*MT
// tokens; they share an activation tile of 32*MT*WT tokens staged through LDS.  Nothing but
// activations goes through LDS.  With WT = 2 there are two wavefronts per SIMD, so one's epilogue
// arithmetic runs under the other's MFMAs.
template <int MT, int WT, bool GROUPED>
__global__ __launch_bounds__(256 * WT) void gemm_q4_k_mfma_kernel(GemmArgs g) {
    constexpr int TM = 32 * MT * WT;  // tokens per workgroup
    static_assert(TM * 4 <= 256, "activation staging assumes one pass of 256 threads");
    constexpr int OFF_DIG = TM * GM_LDW;
    constexpr int OFF_DA = OFF_DIG + TM * 32;
    constexpr int STAGE = OFF_DA + TM * 4;
    extern __shared__ uint4 smem_gemm[];
    uint8_t *lds = reinterpret_cast<uint8_t *>(smem_gemm);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lg = lane >> 5;

    const int bid = blockIdx.x;
    int row_tile, tok0, n_tok, w_first_row;
    if (GROUPED) {
        row_tile = bid % g.row_tiles;
        const int t = bid / g.row_tiles;
        if (t >= *g.n_tiles) return;  // uniform per workgroup
        const int4 ti = g.tiles[t];
        tok0 = ti.y;
        n_tok = ti.y + ti.z;  // one past the last output row of this tile
        w_first_row = ti.x * g.rows;
    } else {
        // workgroups that share weight rows (different token tiles) sit on one XCD (block id mod 8)
        const int per_group = 8 * g.tok_tiles;
        const int grp = bid / per_group, in_grp = bid % per_group;
        row_tile = grp * 8 + (in_grp & 7);
        if (row_tile >= g.row_tiles) return;  // uniform per workgroup
        tok0 = (in_grp >> 3) * TM;
        n_tok = g.M;
        w_first_row = 0;
    }
    const int wtok = wave >> 2;  // token group of this wavefront
    const int row = row_tile * 128 + (wave & 3) * 32 + li;
    const int K = g.nb * QK_K;
    // activation row that feeds output row tok0 + t (clamped into the tile)
    auto act_row = [&](int t) {
        const int p = min(tok0 + min(t, TM - 1), n_tok - 1);
        return (GROUPED && g.gather) ? g.gather[p] : p;
    };

    // weight side: this lane's row, bytes 16*lg.. of every 32-byte nibble pair
    const uint8_t *wrow = g.W + (size_t)(w_first_row + min(row, g.rows - 1)) * g.row_stride;
    // activation side: thread t moves the 64 bytes (t & 3) of token t >> 2, 16 digit bytes of
    // token t >> 1 and the block scale of token t
    const int8_t *s_src = g.aq + (size_t)act_row(tid >> 2) * K + (tid & 3) * 64;
    const int8_t *d_src = ((tid & 1) ? g.bs_lo : g.bs_hi) + (size_t)act_row(tid >> 1) * g.nb * 16;
    const float *a_src = g.ad + (size_t)act_row(tid) * g.nb;

    auto issue_loads = [&](GemmPrefetch &pf, int kb) {
        const uint8_t *blk = wrow + (size_t)kb * Q4_K_BYTES;
        pf.wh = *reinterpret_cast<const uint4 *>(blk);
        pf.wq0 = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * lg);
        pf.wq1 = *reinterpret_cast<const uint4 *>(blk + 48 + 16 * lg);
        pf.wq2 = *reinterpret_cast<const uint4 *>(blk + 80 + 16 * lg);
        pf.wq3 = *reinterpret_cast<const uint4 *>(blk + 112 + 16 * lg);
        const uint4 *src = reinterpret_cast<const uint4 *>(s_src + (size_t)kb * QK_K);
        pf.sa0 = src[0];
        pf.sa1 = src[1];
        pf.sa2 = src[2];
        pf.sa3 = src[3];
        pf.sdig = *reinterpret_cast<const uint4 *>(d_src + (size_t)kb * 16);
        pf.sda = a_src[kb];
    };
    auto store_stage = [&](const GemmPrefetch &pf, int stage) {
        uint8_t *st = lds + stage * STAGE;
        if (tid < TM * 4) {
            uint4 *dst = reinterpret_cast<uint4 *>(st + (tid >> 2) * GM_LDW + (tid & 3) * 64);
            dst[0] = pf.sa0;
            dst[1] = pf.sa1;
            dst[2] = pf.sa2;
            dst[3] = pf.sa3;
        }
        if (tid < TM * 2) *reinterpret_cast<uint4 *>(st + OFF_DIG + (tid >> 1) * 32 + (tid & 1) * 16) = pf.sdig;
        if (tid < TM) *reinterpret_cast<float *>(st + OFF_DA + tid * 4) = pf.sda;
    };

    // the current block of this lane's row as MFMA operands
    v4i bH[8], bL[8];
    long mB;
    float wd, wdmin;
    auto unpack = [&](const GemmPrefetch &pf) {
        const uint4 wh = pf.wh;
        const uint32_t sc_lo = wh.y & 0x3f3f3f3fu, m_lo = wh.z & 0x3f3f3f3fu;
        const uint32_t sc_hi = (wh.w & 0x0f0f0f0fu) | (((wh.y >> 6) & 0x03030303u) << 4);
        const uint32_t m_hi = ((wh.w >> 4) & 0x0f0f0f0fu) | (((wh.z >> 6) & 0x03030303u) << 4);
        // one nibble pair: 16 bytes -> the lane's H and L operands of sub-blocks 2p and 2p+1
        auto pair = [&](const uint4 q, const uint32_t scw, v4i &H0, v4i &L0, v4i &H1, v4i &L1) {
            const uint32_t s0 = scw & 0xff, s1 = (scw >> 8) & 0xff;
            const us2 h0 = {(unsigned short)(s0 >> 3), (unsigned short)(s0 >> 3)};
            const us2 l0 = {(unsigned short)(s0 & 7), (unsigned short)(s0 & 7)};
            const us2 h1 = {(unsigned short)(s1 >> 3), (unsigned short)(s1 >> 3)};
            const us2 l1 = {(unsigned short)(s1 & 7), (unsigned short)(s1 & 7)};
            auto one = [&](const uint32_t w, int &o0, int &o1, int &o2, int &o3) {
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
            H0 = v4i{a0, b0, c0, d0};  // sub-block 2p: low nibbles
            L0 = v4i{a1, b1, c1, d1};
            H1 = v4i{a2, b2, c2, d2};  // sub-block 2p+1: high nibbles
            L1 = v4i{a3, b3, c3, d3};
        };
        pair(pf.wq0, sc_lo, bH[0], bL[0], bH[1], bL[1]);
        pair(pf.wq1, sc_lo >> 16, bH[2], bL[2], bH[3], bL[3]);
        pair(pf.wq2, sc_hi, bH[4], bL[4], bH[5], bL[5]);
        pair(pf.wq3, sc_hi >> 16, bH[6], bL[6], bH[7], bL[7]);
        // mins of the four sub-blocks whose 16-wide groups are 8*lg .. 8*lg+7, each twice
        const uint32_t mw = lg ? m_hi : m_lo;
        const uint32_t mlo = __builtin_amdgcn_perm(0, mw, 0x01010000u), mhi = __builtin_amdgcn_perm(0, mw, 0x03030202u);
        mB = (long)(((unsigned long)mhi << 32) | mlo);
        wd = h2f(wh.x & 0xffffu);
        wdmin = h2f(wh.x >> 16);
    };

    float accF[MT][16];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) accF[mt][r] = 0.0f;

    auto compute_block = [&](int kb) {
        const uint8_t *st = lds + (kb & 1) * STAGE;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const int t0 = (wtok * MT + mt) * 32;  // first token of this tile within the stage
            const uint8_t *arow = st + (t0 + li) * GM_LDW + 16 * lg;
            const v16i z = {0};
            // all of the tile's LDS reads go out before the first MFMA needs one
            v4i a[8];
#pragma unroll
            for (int ks = 0; ks < 8; ks++) a[ks] = *reinterpret_cast<const v4i *>(arow + ks * 32);
            const uint8_t *drow = st + OFF_DIG + (t0 + li) * 32 + 8 * lg;
            const long dgh = *reinterpret_cast<const long *>(drow);
            const long dgl = *reinterpret_cast<const long *>(drow + 16);
            v16i accH, accL;
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                if (ks == 0) {
                    accH = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks], bH[ks], z, 0, 0, 0);
                    accL = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks], bL[ks], z, 0, 0, 0);
                } else {
                    accH = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks], bH[ks], accH, 0, 0, 0);
                    accL = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks], bL[ks], accL, 0, 0, 0);
                }
            }
            const v16i Dh = __builtin_amdgcn_mfma_i32_32x32x16_i8(dgh, mB, z, 0, 0, 0);
            const v16i Dl = __builtin_amdgcn_mfma_i32_32x32x16_i8(dgl, mB, z, 0, 0, 0);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float4 da4 = *reinterpret_cast<const float4 *>(st + OFF_DA + (t0 + 4 * lg + 8 * c) * 4);
                const float dav[4] = {da4.x, da4.y, da4.z, da4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int r = c * 4 + e;
                    const int s1 = (accH[r] << 3) + accL[r];
                    const int s2 = (Dh[r] << 6) + Dl[r];
                    const float v = wd * (float)s1 - wdmin * (float)s2;
                    accF[mt][r] = fmaf(dav[e], v, accF[mt][r]);
                }
            }
        }
    };

    // prologue: block 0 staged and unpacked, block 1 in flight
    GemmPrefetch pf;
    issue_loads(pf, 0);
    store_stage(pf, 0);
    unpack(pf);
    if (g.nb > 1) issue_loads(pf, 1);
    lds_barrier();

    for (int kb = 0; kb < g.nb; kb++) {
        compute_block(kb);
        if (kb + 1 < g.nb) {
            store_stage(pf, (kb + 1) & 1);  // the other stage: nobody reads it during this iteration
            unpack(pf);
            if (kb + 2 < g.nb) issue_loads(pf, kb + 2);
        }
        lds_barrier();
    }

    // store: a lane holds one weight row and 16 tokens per tile
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int tok = tok0 + (wtok * MT + mt) * 32 + (r >> 2) * 8 + lg * 4 + (r & 3);
            if (row < g.rows && tok < n_tok) g.y[(size_t)tok * g.rows + row] = accF[mt][r];
        }
}

// ------------------------------------------------------------------ launchers

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

size_t gemm_q4_k_workspace_bytes(size_t M, size_t cols) {
    const size_t n = M * cols;
    return round_up(n, 256) + round_up(n / QK_K * 4, 256) + 2 * round_up(n / 16, 256);
}

int launch_gemm_q4_k(const frk_weights *w, const float *x, size_t M, float *y, void *ws, hipStream_t s) {
    const size_t n = M * w->cols;
    int8_t *q = (int8_t *)ws;
    float *d = (float *)((char *)ws + round_up(n, 256));
    int8_t *bh = (int8_t *)((char *)d + round_up(n / QK_K * 4, 256));
    int8_t *bl = bh + round_up(n / 16, 256);
    int rc = launch_quantize_q8_k_gemm(x, n, q, d, bh, bl, s);
    if (rc) return rc;

    GemmArgs g;
    g.W = w->dev;
    g.row_stride = w->layout.row_stride;
    g.rows = (int)w->rows;
    g.nb = (int)(w->cols / QK_K);
    g.M = (int)M;
    g.aq = q;
    g.ad = d;
    g.bs_hi = bh;
    g.bs_lo = bl;
    g.y = y;
    g.tiles = nullptr;
    g.n_tiles = nullptr;
    g.gather = nullptr;
    g.row_tiles = (int)((w->rows + 127) / 128);
    const int wt = M > 32 ? 2 : 1;  // token groups per workgroup, one 32-token tile per wavefront
    const int tm = 32 * wt;
    g.tok_tiles = (int)((M + tm - 1) / tm);
    const int groups = (g.row_tiles + 7) / 8;
    const unsigned grid = (unsigned)(groups * 8 * g.tok_tiles);
    const size_t shmem = 2 * ((size_t)tm * GM_LDW + (size_t)tm * 36);
    if (wt == 2) hipLaunchKernelGGL((gemm_q4_k_mfma_kernel<1, 2, false>), dim3(grid), dim3(512), shmem, s, g);
    else hipLaunchKernelGGL((gemm_q4_k_mfma_kernel<1, 1, false>), dim3(grid), dim3(256), shmem, s, g);
    FRK_LAUNCH_CHECK("gemm_q4_k_mfma");
    return FRK_OK;
}


int launch_quantize_q8_k_gemm(const float *x, size_t n, int8_t *q, float *d, int8_t *bs_hi, int8_t *bs_lo,
                              hipStream_t s) {
    const size_t nblk = n / QK_K;
    if (nblk == 0) return FRK_OK;
    hipLaunchKernelGGL(quantize_q8_k_gemm_kernel, dim3((unsigned)((nblk + 3) / 4)), dim3(256), 0, s, x, nblk, q, d,
                       bs_hi, bs_lo);
    FRK_LAUNCH_CHECK("quantize_q8_k_gemm");
    return FRK_OK;
}

// Grouped GEMM over the experts stacked in `w` (expert e = rows [e*rows_e, (e+1)*rows_e)):
// y[p][rows_e] for every output row p listed in the tiles (32 rows per tile at most).
int launch_gemm_q4_k_grouped(const frk_weights *w, size_t rows_e, const int8_t *aq, const float *ad,
                             const int8_t *bs_hi, const int8_t *bs_lo, const int4 *tiles, const int *n_tiles,
                             int max_tiles, const int *gather, float *y, hipStream_t s) {
    GemmArgs g;
    g.W = w->dev;
    g.row_stride = w->layout.row_stride;
    g.rows = (int)rows_e;
    g.nb = (int)(w->cols / QK_K);
    g.M = 0;
    g.aq = aq;
    g.ad = ad;
    g.bs_hi = bs_hi;
    g.bs_lo = bs_lo;
    g.y = y;
    g.tiles = tiles;
    g.n_tiles = n_tiles;
    g.gather = gather;
    g.row_tiles = (int)((rows_e + 127) / 128);
    g.tok_tiles = max_tiles;
    const unsigned grid = (unsigned)(g.row_tiles * max_tiles);
    const size_t shmem = 2 * ((size_t)32 * GM_LDW + (size_t)32 * 36);
    hipLaunchKernelGGL((gemm_q4_k_mfma_kernel<1, 1, true>), dim3(grid), dim3(256), shmem, s, g);
    FRK_LAUNCH_CHECK("gemm_q4_k_grouped");
    return FRK_OK;
}

}  // namespace frk
