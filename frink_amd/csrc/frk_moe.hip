// MoE expert FFN for a batch of tokens, the device form of Decoder::moe_ffn_batch
// (crates/frink-models/src/decoder/ffn_batch.rs:343-434):
//   bucket (token, slot) pairs by expert  ->  gate/up grouped GEMM over gathered token rows
//   ->  silu(gate)*up, quantized to Q8_K  ->  down grouped GEMM  ->  out[tok] = sum_e w * down
// with each token's experts added in ascending expert id, as the reference's expert loop does.
#include "frk_device.hpp"

namespace frk {

// route_top_k_softmax (crates/frink-moe/src/lib.rs:567-589): one wavefront per token.  The
// exponentials are computed in parallel, the softmax denominator is then summed by one lane in
// index order (the reference's sequential f32 sum); among equal probabilities the lowest index
// wins (the reference's unstable sort leaves that case undefined).  n_experts <= 1024, k <= 64.
__global__ __launch_bounds__(64) void route_top_k_softmax_kernel(const float *__restrict__ logits, int batch,
                                                                 int n_experts, int k, int norm,
                                                                 int32_t *__restrict__ ids,
                                                                 float *__restrict__ weights) {
    __shared__ float prob[1024];
    __shared__ float s_sum;
    const int b = blockIdx.x, lane = threadIdx.x;
    const float *l = logits + (size_t)b * n_experts;
    float mx = -INFINITY;
    for (int i = lane; i < n_experts; i += 64) mx = fmaxf(mx, l[i]);
    mx = wave_max(mx);
    for (int i = lane; i < n_experts; i += 64) prob[i] = expf(l[i] - mx);
    __syncthreads();
    if (lane == 0) {
        float sum = 0.0f;
        for (int i = 0; i < n_experts; i++) sum += prob[i];
        s_sum = sum;
    }
    __syncthreads();
    const float sum = s_sum;
    for (int i = lane; i < n_experts; i += 64) prob[i] = __fdiv_rn(prob[i], sum);
    __syncthreads();
    float top_sum = 0.0f, mine = 0.0f;  // lane s keeps the s-th weight
    for (int s = 0; s < k; s++) {
        // wave argmax: larger probability, then smaller index
        float best = -1.0f;
        int best_i = 0x7fffffff;
        for (int i = lane; i < n_experts; i += 64) {
            const float p = prob[i];
            if (p > best) {
                best = p;
                best_i = i;
            }
        }
#pragma unroll
        for (int m = 1; m < 64; m <<= 1) {
            const float ob = __shfl_xor(best, m);
            const int oi = __shfl_xor(best_i, m);
            if (ob > best || (ob == best && oi < best_i)) {
                best = ob;
                best_i = oi;
            }
        }
        if (lane == 0) {
            ids[(size_t)b * k + s] = best_i;
            prob[best_i] = -2.0f;  // taken
        }
        if (lane == s) mine = best;
        top_sum += best;  // same order in every lane: the reference's sum over the k weights
        __syncthreads();
    }
    if (lane < k) weights[(size_t)b * k + lane] = norm ? __fdiv_rn(mine, top_sum) : mine;
}

// Exclusive scan over the workgroup's 1024 threads (16 wavefronts); `total` gets the sum.
__device__ __forceinline__ int block_exclusive_scan(int v, int *wave_tot, int &total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = v;
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const int o = __shfl_up(inc, m);
        if (lane >= m) inc += o;
    }
    if (lane == 63) wave_tot[wave] = inc;
    __syncthreads();
    int base = 0, tot = 0;
    for (int w = 0; w < 16; w++) {
        const int t = wave_tot[w];
        if (w < wave) base += t;
        tot += t;
    }
    __syncthreads();
    total = tot;
    return base + inc - v;
}

// Buckets the batch*k (token, slot) pairs by expert, tokens ascending inside a bucket.
//   group_off[E+1]   bucket boundaries in the grouped order
//   gather[pairs]    token of each grouped position
//   pos_of[pairs]    grouped position of pair (tok*k + slot); -1 for an id outside [0, E)
//   tiles / n_tiles  the buckets cut into runs of at most MOE_TILE positions for the grouped GEMM
// One workgroup of 1024 threads; E <= 1024.  Pairs are taken 1024 at a time in pair order (which
// is token-major); a pair's place in its bucket is the count of earlier pairs of that expert:
// those of earlier rounds (run), of earlier wavefronts of this round (a prefix over the
// per-wavefront counts) and of lower lanes of its own wavefront.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t *__restrict__ ids, int pairs, int k,
                                                         int n_experts, int *__restrict__ group_off,
                                                         int *__restrict__ gather, int *__restrict__ pos_of,
                                                         int4 *__restrict__ tiles, int *__restrict__ n_tiles) {
    __shared__ int cnt[1024];
    __shared__ int off[1024];
    __shared__ int run[1024];
    __shared__ unsigned short wcnt[16][1024];
    __shared__ int wave_tot[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    cnt[tid] = 0;
    run[tid] = 0;
    __syncthreads();
    for (int p = tid; p < pairs; p += 1024) {
        const int e = ids[p];
        if (e >= 0 && e < n_experts) atomicAdd(&cnt[e], 1);
        else pos_of[p] = -1;
    }
    __syncthreads();
    {
        const int c = tid < n_experts ? cnt[tid] : 0;
        const int nt = (c + MOE_TILE - 1) / MOE_TILE;
        int total, total_tiles;
        const int o = block_exclusive_scan(c, wave_tot, total);
        const int t = block_exclusive_scan(nt, wave_tot, total_tiles);
        off[tid] = o;
        if (tid < n_experts) {
            group_off[tid] = o;
            for (int i = 0; i < nt; i++) tiles[t + i] = make_int4(tid, o + MOE_TILE * i, min(MOE_TILE, c - MOE_TILE * i), 0);
        }
        if (tid == 0) {
            group_off[n_experts] = total;
            *n_tiles = total_tiles;
        }
    }
    for (int p0 = 0; p0 < pairs; p0 += 1024) {
        for (int w = 0; w < 16; w++) wcnt[w][tid] = 0;
        __syncthreads();
        const int p = p0 + tid;
        int e = p < pairs ? ids[p] : -1;
        if (e >= n_experts) e = -1;
        int rank = 0, same = 0;
        for (int j = 0; j < 64; j++) {
            const int ej = __shfl(e, j);
            same += (ej == e);
            rank += (ej == e && j < lane);
        }
        if (e >= 0 && rank == 0) wcnt[wave][e] = (unsigned short)same;
        __syncthreads();
        int before = 0;
        if (e >= 0)
            for (int w = 0; w < wave; w++) before += wcnt[w][e];
        if (e >= 0) {
            const int pos = off[e] + run[e] + before + rank;
            gather[pos] = p / k;
            pos_of[p] = pos;
        }
        __syncthreads();
        {
            int tot = 0;
            for (int w = 0; w < 16; w++) tot += wcnt[w][tid];
            run[tid] += tot;
        }
        __syncthreads();
    }
}

// GluAct::Swiglu (crates/frink-core/src/matmul.rs:634-650): act = gate / (1 + exp(-gate)) * up, quantized
// straight to Q8_K (with the GEMM's digit split) -- the down projection quantizes its own input
// in the reference too (ffn_batch.rs:405-415).  One wavefront per 256 values.
__global__ __launch_bounds__(256) void swiglu_quantize_kernel(const float *__restrict__ gate,
                                                              const float *__restrict__ up, size_t n_blocks,
                                                              int8_t *__restrict__ q, float *__restrict__ d,
                                                              _Float16 *__restrict__ bsf) {
    const int lane = threadIdx.x & 63;
    const size_t b = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= n_blocks) return;
    const float4 gv = reinterpret_cast<const float4 *>(gate + b * QK_K)[lane];
    const float4 uv = reinterpret_cast<const float4 *>(up + b * QK_K)[lane];
    // exp in double, rounded once to f32: the correctly rounded value, which is what a host libm's
    // expf returns in all but a vanishing share of cases, so the quantizer below sees the same input
    auto silu = [](float x) { return __fdiv_rn(x, 1.0f + (float)exp(-(double)x)); };
    const float4 v = make_float4(silu(gv.x) * uv.x, silu(gv.y) * uv.y, silu(gv.z) * uv.z, silu(gv.w) * uv.w);
    float dd;
    int bs;
    const uint32_t packed = quantize_q8_k_lane(v, dd, bs);
    reinterpret_cast<uint32_t *>(q + b * QK_K)[lane] = packed;
    if ((lane & 3) == 0) {
        bsf[b * 16 + (lane >> 2)] = (_Float16)bs;
    }
    if (lane == 0) d[b] = dd;
}

// silu(gate) * up, elementwise (frink_core::matmul::swiglu, crates/frink-core/src/matmul.rs:634-650;
// glu_mul_device in crates/frink-cuda/src/matvec_launch.rs:551-570)
__global__ __launch_bounds__(256) void swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                                     size_t n, float *__restrict__ act) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i];
    act[i] = __fdiv_rn(g, 1.0f + (float)exp(-(double)g)) * up[i];
}

int launch_swiglu(const float *gate, const float *up, size_t n, float *act, hipStream_t s);

// out[tok] = sum over the token's slots, ascending expert id, of w * down[pos]: the order of the
// reference's expert loop (ffn_batch.rs:388-423), each term a separate multiply and add.
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ down, const int32_t *__restrict__ ids,
                                                          const float *__restrict__ weights,
                                                          const int *__restrict__ pos_of, int k, int hidden,
                                                          float *__restrict__ out) {
    __shared__ int s_pos[64];
    __shared__ float s_w[64];
    const int tok = blockIdx.x;
    if (threadIdx.x == 0) {
        int order[64];
        for (int s = 0; s < k; s++) order[s] = s;
        for (int a = 1; a < k; a++) {  // insertion sort by expert id
            const int v = order[a];
            int j = a - 1;
            while (j >= 0 && ids[(size_t)tok * k + order[j]] > ids[(size_t)tok * k + v]) {
                order[j + 1] = order[j];
                j--;
            }
            order[j + 1] = v;
        }
        for (int s = 0; s < k; s++) {
            s_pos[s] = pos_of[(size_t)tok * k + order[s]];
            s_w[s] = weights[(size_t)tok * k + order[s]];
        }
    }
    __syncthreads();
    for (int h = threadIdx.x * 4; h < hidden; h += blockDim.x * 4) {
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int s = 0; s < k; s++) {
            if (s_pos[s] < 0) continue;
            const float4 v = *reinterpret_cast<const float4 *>(down + (size_t)s_pos[s] * hidden + h);
            const float w = s_w[s];
            acc.x += w * v.x;
            acc.y += w * v.y;
            acc.z += w * v.z;
            acc.w += w * v.w;
        }
        *reinterpret_cast<float4 *>(out + (size_t)tok * hidden + h) = acc;
    }
}

#define FRK_LAUNCH_CHECK(what)                                                                          \
    do {                                                                                                \
        hipError_t e_ = hipGetLastError();                                                              \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

int launch_swiglu(const float *gate, const float *up, size_t n, float *act, hipStream_t s) {
    hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, gate, up, n, act);
    FRK_LAUNCH_CHECK("swiglu");
    return FRK_OK;
}

int launch_route_top_k_softmax(const float *logits, int batch, int n_experts, int k, int norm, int32_t *ids,
                               float *weights, hipStream_t s) {
    hipLaunchKernelGGL(route_top_k_softmax_kernel, dim3(batch), dim3(64), 0, s, logits, batch, n_experts, k,
                       norm, ids, weights);
    FRK_LAUNCH_CHECK("route_top_k_softmax");
    return FRK_OK;
}

struct MoeScratch {
    int8_t *xq;  // Q8_K of the token rows; bsums as f16
    _Float16 *xb;
    float *xd;
    float *gate_out, *up_out, *down_out;
    int8_t *aq;  // Q8_K of silu(gate)*up
    _Float16 *ab;
    float *ad;
    int *group_off, *gather, *pos_of, *n_tiles;
    int4 *tiles;
};

// Carves the workspace; with base == nullptr the returned pointers are offsets and `end` the size.
static MoeScratch moe_carve(void *base, size_t batch, int k, int n_experts, int hidden, int ffn, size_t *end) {
    const size_t pairs = batch * (size_t)k;
    char *p = (char *)base;
    auto take = [&](size_t bytes) {
        char *r = p;
        p += round_up(bytes, 256);
        return r;
    };
    MoeScratch m;
    m.xq = (int8_t *)take(batch * hidden);
    m.xb = (_Float16 *)take(batch * hidden / 16 * 2);
    m.xd = (float *)take(batch * hidden / QK_K * 4);
    m.gate_out = (float *)take(pairs * ffn * 4);
    m.up_out = (float *)take(pairs * ffn * 4);
    m.down_out = (float *)take(pairs * hidden * 4);
    m.aq = (int8_t *)take(pairs * ffn);
    m.ab = (_Float16 *)take(pairs * ffn / 16 * 2);
    m.ad = (float *)take(pairs * ffn / QK_K * 4);
    m.group_off = (int *)take((n_experts + 1) * 4);
    m.gather = (int *)take(pairs * 4);
    m.pos_of = (int *)take(pairs * 4);
    m.n_tiles = (int *)take(256);
    m.tiles = (int4 *)take((pairs / MOE_TILE + n_experts + 1) * 16);
    if (end) *end = (size_t)(p - (char *)base);
    return m;
}

size_t moe_workspace_bytes(size_t batch, int k, int n_experts, int hidden, int ffn) {
    size_t end = 0;
    (void)moe_carve(nullptr, batch, k, n_experts, hidden, ffn, &end);
    return end;
}

// Test hook: copies out what the last launch_moe_ffn of this shape left in `ws` (null = skip).
// Rows are in grouped order; pos_of[tok*k + slot] is the row of a (token, slot) pair.
int moe_copy_intermediates(void *ws, size_t batch, int k, int n_experts, int hidden, int ffn, float *gate_out,
                           float *up_out, int8_t *act_q, float *act_d, int32_t *pos_of, hipStream_t s) {
    const MoeScratch m = moe_carve(ws, batch, k, n_experts, hidden, ffn, nullptr);
    const size_t pairs = batch * (size_t)k;
    auto copy = [&](void *dst, const void *src, size_t bytes) -> int {
        if (!dst) return FRK_OK;
        hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s);
        return e == hipSuccess ? FRK_OK : set_error(FRK_ERR_HIP, "hipMemcpyAsync: %s", hipGetErrorString(e));
    };
    int rc = copy(gate_out, m.gate_out, pairs * ffn * 4);
    if (!rc) rc = copy(up_out, m.up_out, pairs * ffn * 4);
    if (!rc) rc = copy(act_q, m.aq, pairs * ffn);
    if (!rc) rc = copy(act_d, m.ad, pairs * ffn / QK_K * 4);
    if (!rc) rc = copy(pos_of, m.pos_of, pairs * 4);
    return rc;
}

int launch_moe_ffn(const frk_weights *gate, const frk_weights *up, const frk_weights *down, int n_experts,
                   const float *x, size_t batch, const int32_t *ids, const float *weights, int k, float *out,
                   void *ws, hipStream_t s) {
    const int hidden = (int)gate->cols, ffn = (int)down->cols;
    const size_t pairs = batch * (size_t)k;
    const MoeScratch m = moe_carve(ws, batch, k, n_experts, hidden, ffn, nullptr);
    const int max_tiles = (int)(pairs / MOE_TILE + n_experts);

    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 0, s, ids, (int)pairs, k, n_experts, m.group_off, m.gather,
                       m.pos_of, m.tiles, m.n_tiles);
    FRK_LAUNCH_CHECK("moe_group");
    int rc = launch_quantize_q8_k_gemm(x, batch * hidden, m.xq, m.xd, m.xb, s);
    if (rc) return rc;
    // gate and up read the same quantized token rows through the gather list
    rc = launch_gemm_q4_k_grouped(gate, (size_t)ffn, m.xq, m.xd, m.xb, m.tiles, m.n_tiles, max_tiles, m.gather,
                                  m.gate_out, s);
    if (rc) return rc;
    rc = launch_gemm_q4_k_grouped(up, (size_t)ffn, m.xq, m.xd, m.xb, m.tiles, m.n_tiles, max_tiles, m.gather,
                                  m.up_out, s);
    if (rc) return rc;
    const size_t ablk = pairs * ffn / QK_K;
    hipLaunchKernelGGL(swiglu_quantize_kernel, dim3((unsigned)((ablk + 3) / 4)), dim3(256), 0, s, m.gate_out, m.up_out,
                       ablk, m.aq, m.ad, m.ab);
    FRK_LAUNCH_CHECK("swiglu_quantize");
    rc = launch_gemm_q4_k_grouped(down, (size_t)hidden, m.aq, m.ad, m.ab, m.tiles, m.n_tiles, max_tiles, nullptr,
                                  m.down_out, s);
    if (rc) return rc;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)batch), dim3(256), 0, s, m.down_out, ids, weights, m.pos_of, k,
                       hidden, out);
    FRK_LAUNCH_CHECK("moe_combine");
    return FRK_OK;
}

}  // namespace frk
