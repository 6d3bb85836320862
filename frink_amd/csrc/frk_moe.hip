// MoE expert FFN for a batch of tokens, the device form of Decoder::moe_ffn_batch
// (crates/frink-models/src/decoder/ffn_batch.rs:343-434):
//   bucket (token, slot) pairs by expert  ->  gate/up grouped GEMM over gathered token rows
//   ->  silu(gate)*up, quantized to Q8_K  ->  down grouped GEMM  ->  out[tok] = sum_e w * down
// with each token's experts added in the order the reference adds them (moe_combine_kernel).
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
    __shared__ uint64_t table[32];
    const int b = blockIdx.x, lane = threadIdx.x;
    const float *l = logits + (size_t)b * n_experts;
    // This kernel is one wavefront and as long as its chain of dependent steps: the exponential's table is asked
    // for beside the logits (not when the first exponent is known), a lane's candidates stay in registers (expert
    // i lives in lane i % 64, register i / 64), and the ids leave in one store at the end.
    const uint64_t entry = EXPF_TABLE[lane & 31];
    float p[16];
#pragma unroll
    for (int j = 0; j < 16; j++) p[j] = lane + 64 * j < n_experts ? l[lane + 64 * j] : -INFINITY;
    table[lane & 31] = entry;
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 16; j++) mx = fmaxf(mx, p[j]);
    mx = wave_max(mx);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 16; j++)
        if (64 * j < n_experts) {  // uniform
            p[j] = expf_as_libm(p[j] - mx, table);  // (a host's bits, as the reference's f32::exp gives them)
            if (lane + 64 * j < n_experts) prob[lane + 64 * j] = p[j];
        }
    __syncthreads();
    float sum = 0.0f;  // every lane adds all of them in index order, as the reference does: no broadcast afterwards
    for (int i = 0; i < n_experts; i++) sum += prob[i];
#pragma unroll
    for (int j = 0; j < 16; j++) p[j] = lane + 64 * j < n_experts ? __fdiv_rn(p[j], sum) : -2.0f;  // (-2: no candidate)
    float top_sum = 0.0f, mine = 0.0f;  // lane s keeps the s-th weight
    int mine_i = 0;
    for (int s = 0; s < k; s++) {
        // argmax over the wavefront: larger probability, then smaller index
        float best = -1.0f;
        int best_i = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < 16; j++)
            if (p[j] > best) best = p[j], best_i = lane + 64 * j;
        // (two maxima, mostly DPP: the largest probability, then the smallest index among the lanes that hold it --
        // an index up to 1024 is exact as a float)
        const float top = wave_max(best);
        best_i = n_experts - (int)wave_max(best == top ? (float)(n_experts - best_i) : -1.0f);
#pragma unroll
        for (int j = 0; j < 16; j++)
            if (best_i == lane + 64 * j) p[j] = -2.0f;  // taken
        if (lane == s) mine = top, mine_i = best_i;
        top_sum += top;  // same order in every lane: the reference's sum over the k weights
    }
    if (lane < k) {
        ids[(size_t)b * k + lane] = mine_i;
        weights[(size_t)b * k + lane] = norm ? __fdiv_rn(mine, top_sum) : mine;
    }
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

// Buckets the batch*k (token, slot) pairs by expert, pairs ascending inside a bucket (which is tokens
// ascending: pairs are token-major).  A bucket is cut into tiles of MOE_TILE rows; tile t is rows
// [MOE_TILE*t, MOE_TILE*(t+1)) of the grouped order and belongs to one expert, so the order has gaps.
// Tiles with more than 32 rows in use come first: they cost the grouped GEMM twice the arithmetic of
// the others, and its workgroups, which deal the tile list out among themselves round-robin, then
// get an even share of both kinds.
//   group_off[E+1]   bucket boundaries in the order without the gaps
//   gather[max_rows] token of each row of the grouped order, -1 in a gap and past the last tile
//   pos_of[pairs]    row of pair (tok*k + slot); -1 for an id outside [0, E)
//   cpos_of[pairs]   the pair's place in the order without the gaps
//   tiles / n_tiles  {expert, first row, rows in use, first row of the GEMMs' output (the same row)} per tile
// One workgroup of 1024 threads; E <= 1024.  No atomic decides an order: a round takes `round`
// pairs, marks pair j of expert e as bit j of row e of a bit matrix in LDS (an OR, so the result
// does not depend on who comes first; the matrix is stored word-major so that the per-expert
// pass below is free of bank conflicts), and a pair's rank in its bucket is the number of set bits
// before its own in that row plus the bucket's count from earlier rounds.
constexpr int GROUP_BIT_WORDS = 16384;  // 64 KB of bits: round = 524288 / E pairs (a multiple of 32)
struct GroupLds {
    uint32_t bits[GROUP_BIT_WORDS];
    unsigned short before[GROUP_BIT_WORDS];  // set bits of the row in the words before this one
    int cnt[1024], off_cmp[1024], run[1024];
    int tile_big[1024], n_big[1024], tile_small[1024], seg_sum[1024];  // first heavy tile, their number, the light tile
    int wave_tot[16];
};
struct GroupArgs {
    const int32_t *ids;
    int pairs, k, n_experts;
    int *group_off, *gather, *pos_of, *cpos_of;
    int4 *tiles;
    int *n_tiles;
    int max_rows;
};
__device__ __forceinline__ void moe_group(const GroupArgs &a) {
    const int32_t *__restrict__ ids = a.ids;
    const int pairs = a.pairs, k = a.k, n_experts = a.n_experts, max_rows = a.max_rows;
    int *__restrict__ group_off = a.group_off, *__restrict__ gather = a.gather, *__restrict__ pos_of = a.pos_of;
    int *__restrict__ cpos_of = a.cpos_of, *__restrict__ n_tiles = a.n_tiles;
    int4 *__restrict__ tiles = a.tiles;
    extern __shared__ uint4 smem_group[];
    GroupLds &L = *reinterpret_cast<GroupLds *>(smem_group);
    const int tid = threadIdx.x;
    L.cnt[tid] = 0;
    L.run[tid] = 0;
    for (int r = tid; r < max_rows; r += 1024) gather[r] = -1;
    __syncthreads();
    // the first 4096 ids stay in registers for all three passes (each pass from memory costs a
    // round trip this one-workgroup kernel has nothing to hide behind)
    int held[4];
#pragma unroll
    for (int i = 0; i < 4; i++) held[i] = tid + 1024 * i < pairs ? ids[tid + 1024 * i] : -1;
    auto id_of = [&](int p) {  // p = tid (mod 1024)
        const int i = p >> 10;
        return i == 0 ? held[0] : i == 1 ? held[1] : i == 2 ? held[2] : i == 3 ? held[3] : ids[p];
    };
    for (int p = tid; p < pairs; p += 1024) {
        const int e = id_of(p);
        if (e >= 0 && e < n_experts) atomicAdd(&L.cnt[e], 1);
        else pos_of[p] = cpos_of[p] = -1;
    }
    __syncthreads();
    {
        const int c = tid < n_experts ? L.cnt[tid] : 0;
        const int nt = (c + MOE_TILE - 1) / MOE_TILE;
        const int last = c - MOE_TILE * (nt - 1);  // rows in use of the last tile (nt > 0)
        const int big = nt == 0 ? 0 : nt - 1 + (last > 32);
        const int small = nt - big;  // 0 or 1
        int total, total_big, total_small;
        const int o = block_exclusive_scan(c, L.wave_tot, total);
        const int tb = block_exclusive_scan(big, L.wave_tot, total_big);
        const int ts = total_big + block_exclusive_scan(small, L.wave_tot, total_small);
        L.off_cmp[tid] = o;
        L.tile_big[tid] = tb;
        L.n_big[tid] = big;
        L.tile_small[tid] = ts;
        if (tid < n_experts) {
            group_off[tid] = o;
            for (int i = 0; i < nt; i++) {
                const int t = i < big ? tb + i : ts;
                const int used = min(MOE_TILE, c - MOE_TILE * i);
                tiles[t] = make_int4(tid, MOE_TILE * t, used, MOE_TILE * t);
            }
        }
        if (tid == 0) {
            group_off[n_experts] = total;
            *n_tiles = total_big + total_small;
        }
    }
    // words per row; `before` is 16 bits wide, so a round stays below 65536 pairs
    const int rw = max(1, min(min(GROUP_BIT_WORDS / n_experts, 2047), (pairs + 31) / 32));
    const int round = rw * 32;
    for (int p0 = 0; p0 < pairs; p0 += round) {
        for (int i = tid; i < rw * n_experts; i += 1024) L.bits[i] = 0;
        __syncthreads();
        for (int j = tid; j < round && p0 + j < pairs; j += 1024) {
            const int e = (p0 & 1023) == 0 ? id_of(p0 + j) : ids[p0 + j];
            if (e >= 0 && e < n_experts) atomicOr(&L.bits[(j >> 5) * n_experts + e], 1u << (j & 31));
        }
        __syncthreads();
        {
            // prefix of the set bits along every row: the row's words are cut into `segs` runs, one
            // thread each
            const int segs = max(1, 1024 / n_experts), ws = (rw + segs - 1) / segs;
            const int e = tid % n_experts, seg = tid / n_experts;
            const int w0 = min(rw, seg * ws), w1 = min(rw, w0 + ws);
            int sum = 0;
            if (seg < segs)
                for (int w = w0; w < w1; w++) sum += __popc(L.bits[w * n_experts + e]);
            L.seg_sum[tid] = sum;
            __syncthreads();
            if (seg < segs) {
                int run = 0;
                for (int s2 = 0; s2 < seg; s2++) run += L.seg_sum[s2 * n_experts + e];
                for (int w = w0; w < w1; w++) {
                    L.before[w * n_experts + e] = (unsigned short)run;
                    run += __popc(L.bits[w * n_experts + e]);
                }
                if (seg == segs - 1) L.cnt[e] = run;  // this pass's pairs of the expert
            }
        }
        __syncthreads();
        for (int j = tid; j < round && p0 + j < pairs; j += 1024) {
            const int p = p0 + j;
            const int e = (p0 & 1023) == 0 ? id_of(p) : ids[p];
            if (e >= 0 && e < n_experts) {
                const int w = (j >> 5) * n_experts + e;
                const int rank = L.run[e] + L.before[w] + __popc(L.bits[w] & ((1u << (j & 31)) - 1u));
                const int j = rank / MOE_TILE;
                const int pos = MOE_TILE * (j < L.n_big[e] ? L.tile_big[e] + j : L.tile_small[e]) + rank % MOE_TILE;
                gather[pos] = p / k;
                pos_of[p] = pos;
                cpos_of[p] = L.off_cmp[e] + rank;
            }
        }
        __syncthreads();
        if (tid < n_experts) L.run[tid] += L.cnt[tid];
        __syncthreads();
    }
}
__global__ __launch_bounds__(1024) void moe_group_kernel(GroupArgs a) { moe_group(a); }

// The bucketing and the quantization of the token rows do not depend on each other: in one launch, workgroup
// 0 buckets while the others quantize (quantize_activations_q8_k, crates/frink-quant/src/act_quant.rs:69-104;
// a wavefront per 256-value block) every token row ONCE, into plain rows that the grouped GEMM gathers from
// -- instead of a launch that waits for the bucketing and then quantizes every (token, slot) pair's copy.
__global__ __launch_bounds__(1024) void moe_group_quantize_kernel(GroupArgs a, const float *__restrict__ x, int n_blocks,
                                                                  Q8KRows out) {
    if (blockIdx.x == 0) {
        moe_group(a);
        return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int b = ((int)blockIdx.x - 1) * 16 + wave; b < n_blocks; b += ((int)gridDim.x - 1) * 16) {
        const float4 v = reinterpret_cast<const float4 *>(x + (size_t)b * QK_K)[lane];
        float dd;
        int bs;
        const uint32_t packed = quantize_q8_k_lane(v, dd, bs);
        reinterpret_cast<uint32_t *>(out.q + (size_t)b * QK_K)[lane] = packed;
        if ((lane & 3) == 0) out.bs[(size_t)b * 16 + (lane >> 2)] = (_Float16)bs;
        if (lane == 0) out.d[b] = dd;
    }
}

// The grouped GEMM with the groups given (enqueue_mul_mm_grouped_dev, crates/frink-cuda/src/mul_mm_launch.rs:391-470):
// pairs group_off[g] .. group_off[g+1]-1 belong to group g and pair p reads activation row gather[p] (row p without
// a gather list).  This cuts the groups into the tiles the grouped kernels walk -- {group, first row of the grouped
// order, rows in use, first pair}: the kernels store tile row r as row (first pair + r) of y, so y comes out as
// [pairs][rows] without gaps -- and lists every tile row's source row (-1: not in use).  Tiles with more than 32
// rows in use first, as in moe_group.  One workgroup of 1024 threads, at most 1024 groups.
struct GroupedTilesArgs {
    const int32_t *group_off, *gather;  // gather may be null
    int n_groups, pairs, x_rows, max_rows;
    int *src_rows;  // [max_rows]
    int4 *tiles;
    int *n_tiles;
};
struct GroupedTilesLds {
    int off[1025], tile_big[1024], n_big[1024], tile_small[1024];
    int wave_tot[16];
};
__device__ __forceinline__ void grouped_tiles(const GroupedTilesArgs &a) {
    __shared__ GroupedTilesLds L;
    const int tid = threadIdx.x;
    for (int r = tid; r < a.max_rows; r += 1024) a.src_rows[r] = -1;
    // (offsets outside 0 .. pairs or out of order: clamped, so that no tile row points outside the lists)
    for (int g = tid; g <= a.n_groups; g += 1024) L.off[g] = min(max(a.group_off[g], 0), a.pairs);
    __syncthreads();
    {
        const int c = tid < a.n_groups ? max(L.off[tid + 1] - L.off[tid], 0) : 0;
        const int nt = (c + MOE_TILE - 1) / MOE_TILE;
        const int last = c - MOE_TILE * (nt - 1);
        const int big = nt == 0 ? 0 : nt - 1 + (last > 32);
        const int small = nt - big;  // 0 or 1
        int total_big, total_small;
        const int tb = block_exclusive_scan(big, L.wave_tot, total_big);
        const int ts = total_big + block_exclusive_scan(small, L.wave_tot, total_small);
        L.tile_big[tid] = tb;
        L.n_big[tid] = big;
        L.tile_small[tid] = ts;
        for (int i = 0; i < nt; i++) {
            const int t = i < big ? tb + i : ts;
            a.tiles[t] = make_int4(tid, MOE_TILE * t, min(MOE_TILE, c - MOE_TILE * i), L.off[tid] + MOE_TILE * i);
        }
        if (tid == 0) *a.n_tiles = total_big + total_small;
    }
    __syncthreads();
    for (int p = tid; p < a.pairs; p += 1024) {
        int lo = 0, hi = a.n_groups;  // the group g with off[g] <= p < off[g+1]: the last g with off[g] <= p
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (L.off[mid] <= p) lo = mid;
            else hi = mid;
        }
        const int rank = p - L.off[lo];
        if (rank < 0 || p >= L.off[lo + 1]) continue;  // (a pair before the first group or in a clamped hole)
        const int i = rank / MOE_TILE;
        const int t = i < L.n_big[lo] ? L.tile_big[lo] + i : L.tile_small[lo];
        const int src = a.gather ? a.gather[p] : p;
        a.src_rows[MOE_TILE * t + rank % MOE_TILE] = min(max(src, 0), a.x_rows - 1);
    }
}
__global__ __launch_bounds__(1024) void grouped_tiles_kernel(GroupedTilesArgs a) { grouped_tiles(a); }
// the same beside the quantization of the activation rows, as in moe_group_quantize_kernel
__global__ __launch_bounds__(1024) void grouped_tiles_quantize_kernel(GroupedTilesArgs a, const float *__restrict__ x, int n_blocks,
                                                                      Q8KRows out) {
    if (blockIdx.x == 0) {
        grouped_tiles(a);
        return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int b = ((int)blockIdx.x - 1) * 16 + wave; b < n_blocks; b += ((int)gridDim.x - 1) * 16) {
        const float4 v = reinterpret_cast<const float4 *>(x + (size_t)b * QK_K)[lane];
        float dd;
        int bs;
        const uint32_t packed = quantize_q8_k_lane(v, dd, bs);
        reinterpret_cast<uint32_t *>(out.q + (size_t)b * QK_K)[lane] = packed;
        if ((lane & 3) == 0) out.bs[(size_t)b * 16 + (lane >> 2)] = (_Float16)bs;
        if (lane == 0) out.d[b] = dd;
    }
}

// GluAct::Swiglu (crates/frink-core/src/matmul.rs:634-650): act = gate / (1 + exp(-gate)) * up, quantized
// straight to Q8_K in the tiled form -- the down projection quantizes its own input in the
// reference too (ffn_batch.rs:405-415).  One workgroup per record (32 rows of the grouped order x
// one block), eight wavefronts of four rows each (measured at 512 tokens x top-8 of 128 experts, 2048/768:
// 12.8 us; sixteen wavefronts 13.6, four 16.2 -- the kernel is about as long as one wavefront's chain of
// tile entry -> loads -> exponentials -> record, times the rounds its workgroups need to become resident).
// Rows past a tile's rows in use become zeros, records without rows in use are skipped.
constexpr int SWIGLU_WAVES = 8;
__global__ __launch_bounds__(64 * SWIGLU_WAVES) void swiglu_quantize_kernel(const float *__restrict__ gate,
                                                                            const float *__restrict__ up, int nb,
                                                                            const int4 *__restrict__ tiles,
                                                                            const int *__restrict__ n_tiles, Q8KTiled out) {
    __shared__ Q8KRecordLds L;
    const int t32 = blockIdx.x / nb, kb = blockIdx.x % nb, lane = threadIdx.x & 63;
    static_assert(MOE_TILE == 64, "a tile is two records");
    const int4 tile = tiles[t32 >> 1];  // (the list is as long as the grid needs, entries past *n_tiles unwritten)
    const int used = t32 >> 1 < *n_tiles ? tile.z - 32 * (t32 & 1) : 0;  // rows in use come first in a tile
    if (used <= 0) return;
    __shared__ uint64_t table[32];
    if (threadIdx.x < 32) table[threadIdx.x] = EXPF_TABLE[threadIdx.x];
    __syncthreads();
    auto silu = [&](float x) { return silu_as_host(x, table); };  // (the quantizer sees a host's bits)
    quantize_q8k_record<SWIGLU_WAVES>(out, (size_t)t32 * nb + kb, L, [&](int r) {
        if (r >= used) return make_float4(0.f, 0.f, 0.f, 0.f);
        const size_t src = ((size_t)(t32 * 32 + r) * nb + kb) * QK_K;
        const float4 gv = reinterpret_cast<const float4 *>(gate + src)[lane];
        const float4 uv = reinterpret_cast<const float4 *>(up + src)[lane];
        return make_float4(silu(gv.x) * uv.x, silu(gv.y) * uv.y, silu(gv.z) * uv.z, silu(gv.w) * uv.w);
    });
}

// silu(gate) * up, elementwise (frink_core::matmul::swiglu, crates/frink-core/src/matmul.rs:634-650;
// glu_mul_device in crates/frink-cuda/src/matvec_launch.rs:551-570)
// (act may be gate: every element is read before it is written, by the thread that writes it)
__global__ __launch_bounds__(256) void swiglu_kernel(const float *gate, const float *__restrict__ up, size_t n, float *act) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i];
    act[i] = silu_as_host(g) * up[i];
}
// four elements a thread, for lengths and addresses that are multiples of four floats
__global__ __launch_bounds__(256) void swiglu4_kernel(const float4 *gate, const float4 *__restrict__ up, size_t n4, float4 *act) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4 g = gate[i], u = up[i];
    act[i] = make_float4(silu_as_host(g.x) * u.x, silu_as_host(g.y) * u.y, silu_as_host(g.z) * u.z, silu_as_host(g.w) * u.w);
}

int launch_swiglu(const float *gate, const float *up, size_t n, float *act, hipStream_t s);

// out[tok] = sum over the token's slots of w * down[pos], each term a separate multiply and add, in the
// order the reference adds them for a batch of this size: its bucket path (32 tokens and more,
// ffn_batch.rs:355, 388-423) walks the experts in ascending id; below that every position runs alone and
// combine_expert_outputs (crates/frink-moe/src/lib.rs:1246-1263) adds the slots in routing order.
// A slot whose id is outside [0, n_experts) contributes nothing.
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ down, const int32_t *__restrict__ ids,
                                                          const float *__restrict__ weights,
                                                          const int *__restrict__ pos_of, int k, int hidden,
                                                          int n_experts, int by_expert_id, float *__restrict__ out) {
    __shared__ int s_pos[64];
    __shared__ float s_w[64];
    __shared__ int s_id[64];
    const int tok = blockIdx.x, tid = threadIdx.x;
    // (the slot's three entries are asked for together: this kernel is as long as its chain of dependent loads)
    int mine = 0, pos = 0;
    float w = 0.0f;
    if (tid < k) {
        mine = ids[(size_t)tok * k + tid];
        pos = pos_of ? pos_of[(size_t)tok * k + tid] : tok * k + tid;  // (no map: rows in pair order)
        w = weights[(size_t)tok * k + tid];
        s_id[tid] = mine;
    }
    __syncthreads();
    if (tid < k) {
        int rank = tid;
        if (by_expert_id) {  // place in the ascending order of expert ids, equal ids in slot order
            rank = 0;
            for (int j = 0; j < k; j++) rank += (s_id[j] < mine) || (s_id[j] == mine && j < tid);
        }
        s_pos[rank] = (mine >= 0 && mine < n_experts) ? pos : -1;
        s_w[rank] = w;
    }
    __syncthreads();
    for (int h = (blockIdx.y * blockDim.x + threadIdx.x) * 4; h < hidden; h += gridDim.y * blockDim.x * 4) {
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        // eight slots' rows are asked for together and then added in order (one at a time, a token's eight
        // experts were eight trips to memory in a row: 7 us of a 19 us layer at one token)
        for (int s0 = 0; s0 < k; s0 += 8) {
            float4 v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int p = s0 + j < k ? s_pos[s0 + j] : -1;
                v[j] = *reinterpret_cast<const float4 *>(down + (size_t)max(p, 0) * hidden + h);  // (no slot: row 0, not added)
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (s0 + j < k && s_pos[s0 + j] >= 0) {  // uniform across the workgroup
                    const float w = s_w[s0 + j];
                    acc.x += w * v[j].x;
                    acc.y += w * v[j].y;
                    acc.z += w * v[j].z;
                    acc.w += w * v[j].w;
                }
            }
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
    if (n == 0) return FRK_OK;
    const bool by_four = n % 4 == 0 && ((reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) | reinterpret_cast<uintptr_t>(act)) & 15) == 0;
    if (by_four)
        hipLaunchKernelGGL(swiglu4_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, s, reinterpret_cast<const float4 *>(gate),
                           reinterpret_cast<const float4 *>(up), n / 4, reinterpret_cast<float4 *>(act));
    else
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
    Q8KTiled xa;                          // the token rows in the grouped order, Q8_K
    float *gate_out, *up_out, *down_out;  // rows in the grouped order (with its gaps)
    Q8KTiled act;                         // Q8_K of silu(gate)*up
    Q8KRows xr;                           // Q8_K of the token rows (the gathering form; shares xa's room)
    int *group_off, *gather, *pos_of, *cpos_of, *n_tiles;
    int4 *tiles;
};

// rows of the grouped order at most: every bucket may end in a partly used tile
static size_t moe_max_rows(size_t pairs, int n_experts) {
    return (pairs / MOE_TILE + (size_t)n_experts) * MOE_TILE;
}

// Carves the workspace; with base == nullptr the returned pointers are offsets and `end` the size.
static MoeScratch moe_carve(void *base, size_t batch, int k, int n_experts, int hidden, int ffn, size_t *end) {
    const size_t pairs = batch * (size_t)k, rows = moe_max_rows(pairs, n_experts);
    char *p = (char *)base;
    auto take = [&](size_t bytes) {
        char *r = p;
        p += round_up(bytes, 256);
        return r;
    };
    MoeScratch m;
    {
        // the token rows' Q8_K in one of two forms: gathered into the grouped order, or plain
        const size_t nb = (size_t)hidden / QK_K;
        const size_t plain = round_up(batch * hidden, 256) + round_up(batch * nb * 32, 256) + batch * nb * 4;
        char *room = take(std::max(q8k_tiled_bytes(rows, hidden), plain));
        m.xa = q8k_tiled_carve(room, rows, hidden);
        m.xr.q = (int8_t *)room;
        m.xr.bs = (_Float16 *)(room + round_up(batch * hidden, 256));
        m.xr.d = (float *)(room + round_up(batch * hidden, 256) + round_up(batch * nb * 32, 256));
    }
    m.gate_out = (float *)take(rows * ffn * 4);
    m.up_out = (float *)take(rows * ffn * 4);
    m.down_out = (float *)take(rows * hidden * 4);
    m.act = q8k_tiled_carve(take(q8k_tiled_bytes(rows, ffn)), rows, ffn);
    m.group_off = (int *)take((n_experts + 1) * 4);
    m.gather = (int *)take(rows * 4);
    m.pos_of = (int *)take(pairs * 4);
    m.cpos_of = (int *)take(pairs * 4);
    m.n_tiles = (int *)take(256);
    m.tiles = (int4 *)take((rows / MOE_TILE + 1) * 16);
    if (end) *end = (size_t)(p - (char *)base);
    return m;
}

size_t moe_workspace_bytes(size_t batch, int k, int n_experts, int hidden, int ffn) {
    size_t end = 0;
    (void)moe_carve(nullptr, batch, k, n_experts, hidden, ffn, &end);
    return end;
}

// Test hook: one workgroup per (token, slot) pair copies the pair's rows of the intermediates to
// the pair's place in the grouped order without gaps (null outputs are skipped).
__global__ __launch_bounds__(256) void moe_export_kernel(MoeScratch m, int ffn, float *__restrict__ gate_out,
                                                         float *__restrict__ up_out, int8_t *__restrict__ act_q,
                                                         float *__restrict__ act_d, int32_t *__restrict__ pos) {
    const int pair = blockIdx.x, tid = threadIdx.x;
    const int src = m.pos_of[pair], dst = m.cpos_of[pair];
    if (pos && tid == 0) pos[pair] = dst;
    if (src < 0) return;
    const int nb = ffn / QK_K;
    for (int i = tid; i < ffn; i += 256) {
        if (gate_out) gate_out[(size_t)dst * ffn + i] = m.gate_out[(size_t)src * ffn + i];
        if (up_out) up_out[(size_t)dst * ffn + i] = m.up_out[(size_t)src * ffn + i];
        if (act_q) act_q[(size_t)dst * ffn + i] = m.act.q[q8k_tiled_index(nb, src, i / QK_K, i % QK_K)];
    }
    if (act_d)
        for (int i = tid; i < nb; i += 256)
            act_d[(size_t)dst * nb + i] = m.act.d[((size_t)(src >> 5) * nb + i) * 32 + (src & 31)];
}

// Copies out what the last launch_moe_ffn of this shape left in `ws`: row i of every output is the
// i-th (token, slot) pair in the order experts ascending, tokens ascending; pos[tok*k + slot] = i.
int moe_copy_intermediates(void *ws, size_t batch, int k, int n_experts, int hidden, int ffn, float *gate_out,
                           float *up_out, int8_t *act_q, float *act_d, int32_t *pos_of, hipStream_t s) {
    const MoeScratch m = moe_carve(ws, batch, k, n_experts, hidden, ffn, nullptr);
    const size_t pairs = batch * (size_t)k;
    hipLaunchKernelGGL(moe_export_kernel, dim3((unsigned)pairs), dim3(256), 0, s, m, ffn, gate_out, up_out, act_q, act_d,
                       pos_of);
    FRK_LAUNCH_CHECK("moe_export");
    return FRK_OK;
}

// The per-token path (cpu_moe_topk_parallel_slots / run_expert, crates/frink-models/src/decoder/
// moe_host.rs:102-203, crates/frink-moe/src/lib.rs:1068-1165): with a token or a few, every (token,
// slot) pair reads its expert's three matrices alone, so the layer is three launches of decode
// kernels -- gate, up and silu(g)*u of all pairs; down of all pairs, each quantizing its own
// intermediate; the weighted sum in routing order -- instead of the six of the grouped path.
// (Q4_K gate and up experts; the down experts Q4_K, or Q6_K with rows of at most 4096 columns)
bool moe_takes_per_token_path(size_t batch, size_t hidden, size_t ffn, int down_kind) {
    const bool down_ok = down_kind == FRK_KIND_Q4_K || (down_kind == FRK_KIND_Q6_K && ffn <= 4096);
    return down_ok && batch <= MOE_PER_TOKEN_MAX_BATCH && hidden <= FUSED_GEMV_MAX_COLS && ffn <= FUSED_GEMV_MAX_COLS;
}
static int launch_moe_ffn_per_token(const frk_weights *gate, const frk_weights *up, const frk_weights *down,
                                    int n_experts, const float *x, size_t batch, const int32_t *ids,
                                    const float *weights, int k, float *out, const MoeScratch &m, hipStream_t s) {
    const int hidden = (int)gate->cols, ffn = (int)down->cols;
    float *act = m.gate_out;  // [batch*k][ffn]
    int rc = launch_gemv_q4_k_experts(gate, up, n_experts, (size_t)ffn, x, (size_t)hidden, ids, batch, (size_t)k, act, s);
    if (rc) return rc;
    rc = down->kind == FRK_KIND_Q6_K
             ? launch_gemv_q6_k_experts(down, n_experts, (size_t)hidden, act, (size_t)ffn, ids, batch * (size_t)k, m.down_out, s)
             : launch_gemv_q4_k_experts(down, nullptr, n_experts, (size_t)hidden, act, (size_t)ffn, ids, batch * (size_t)k, 1,
                                        m.down_out, s);
    if (rc) return rc;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)batch, (unsigned)((hidden + 1023) / 1024)), dim3(256), 0, s, m.down_out, ids, weights,
                       (const int *)nullptr, k, hidden, n_experts, (int)(batch >= MOE_BUCKET_ORDER_FROM), out);
    FRK_LAUNCH_CHECK("moe_combine");
    return FRK_OK;
}

int launch_moe_ffn(const frk_weights *gate, const frk_weights *up, const frk_weights *down, int n_experts,
                   const float *x, size_t batch, const int32_t *ids, const float *weights, int k, float *out,
                   void *ws, hipStream_t s) {
    const int hidden = (int)gate->cols, ffn = (int)down->cols;
    const size_t pairs = batch * (size_t)k, rows = moe_max_rows(pairs, n_experts);
    const MoeScratch m = moe_carve(ws, batch, k, n_experts, hidden, ffn, nullptr);
    const int max_tiles = (int)(rows / MOE_TILE);
    if (moe_takes_per_token_path(batch, (size_t)hidden, (size_t)ffn, down->kind))
        return launch_moe_ffn_per_token(gate, up, down, n_experts, x, batch, ids, weights, k, out, m, s);

    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_group_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GroupLds));
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_group_quantize_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GroupLds));
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(moe_group): %s", hipGetErrorString(e));
        sized = true;
    }
    const GroupArgs ga{ids, (int)pairs, k, n_experts, m.group_off, m.gather, m.pos_of, m.cpos_of, m.tiles, m.n_tiles, (int)rows};
    int rc;
    if (gemm_q4_k_stream_gathers(batch, (size_t)hidden)) {
        // every token row quantized once, beside the bucketing; the gate/up GEMM gathers its tiles' rows
        const size_t n_blocks = batch * ((size_t)hidden / QK_K);
        const unsigned quantizers = (unsigned)std::min<size_t>((n_blocks + 15) / 16, 512);
        hipLaunchKernelGGL(moe_group_quantize_kernel, dim3(1 + quantizers), dim3(1024), sizeof(GroupLds), s, ga, x,
                           (int)n_blocks, m.xr);
        FRK_LAUNCH_CHECK("moe_group_quantize");
        rc = launch_gemm_q4_k_stream(gate, up, (size_t)ffn, m.xa, &m.xr, m.gather, m.tiles, m.n_tiles, max_tiles, m.gate_out,
                                     m.up_out, s);
    } else {
        hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), sizeof(GroupLds), s, ga);
        FRK_LAUNCH_CHECK("moe_group");
        // the token rows, gathered into the grouped order and quantized; gate and up share them
        rc = launch_quantize_q8_k_gather(x, (size_t)hidden, m.gather, rows, m.xa, s);
        if (rc) return rc;
        rc = launch_gemm_q4_k_stream(gate, up, (size_t)ffn, m.xa, nullptr, nullptr, m.tiles, m.n_tiles, max_tiles, m.gate_out,
                                     m.up_out, s);
    }
    if (rc) return rc;
    hipLaunchKernelGGL(swiglu_quantize_kernel, dim3((unsigned)(rows / 32 * (ffn / QK_K))), dim3(64 * SWIGLU_WAVES), 0, s,
                       m.gate_out, m.up_out, ffn / QK_K, m.tiles, m.n_tiles, m.act);
    FRK_LAUNCH_CHECK("swiglu_quantize");
    // (a Q4_K_M checkpoint keeps some layers' down experts in Q6_K: the matrix-core Q6_K kernel, by tile)
    rc = down->kind == FRK_KIND_Q6_K
             ? launch_gemm_q6_k_grouped(down, (size_t)hidden, m.act, m.tiles, m.n_tiles, max_tiles, m.down_out, s)
             : launch_gemm_q4_k_stream(down, nullptr, (size_t)hidden, m.act, nullptr, nullptr, m.tiles, m.n_tiles, max_tiles,
                                       m.down_out, nullptr, s);
    if (rc) return rc;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)batch, (unsigned)((hidden + 1023) / 1024)), dim3(256), 0, s, m.down_out, ids, weights, m.pos_of, k,
                       hidden, n_experts, (int)(batch >= MOE_BUCKET_ORDER_FROM), out);
    FRK_LAUNCH_CHECK("moe_combine");
    return FRK_OK;
}

// The grouped GEMM as an entry of its own.  Scratch: the activations' Q8_K (plain rows, or gathered into the
// grouped order when the kernel cannot address the plain rows or the weights are Q6_K), the tile list and the
// tile rows' source rows.
struct GroupedScratch {
    Q8KTiled xa;
    Q8KRows xr;
    int *src_rows, *n_tiles;
    int4 *tiles;
};
static GroupedScratch grouped_carve(void *base, size_t n_groups, size_t x_rows, size_t pairs, size_t cols, size_t *end) {
    const size_t rows = moe_max_rows(pairs, (int)n_groups), nb = cols / QK_K;
    char *p = (char *)base;
    auto take = [&](size_t bytes) {
        char *r = p;
        p += round_up(bytes, 256);
        return r;
    };
    GroupedScratch m;
    const size_t plain = round_up(x_rows * cols, 256) + round_up(x_rows * nb * 32, 256) + x_rows * nb * 4;
    char *room = take(std::max(q8k_tiled_bytes(rows, cols), plain));
    m.xa = q8k_tiled_carve(room, rows, cols);
    m.xr.q = (int8_t *)room;
    m.xr.bs = (_Float16 *)(room + round_up(x_rows * cols, 256));
    m.xr.d = (float *)(room + round_up(x_rows * cols, 256) + round_up(x_rows * nb * 32, 256));
    m.src_rows = (int *)take(rows * 4);
    m.n_tiles = (int *)take(256);
    m.tiles = (int4 *)take((rows / MOE_TILE + 1) * 16);
    if (end) *end = (size_t)(p - (char *)base);
    return m;
}
size_t grouped_gemm_workspace_bytes(size_t n_groups, size_t x_rows, size_t pairs, size_t cols) {
    size_t end = 0;
    (void)grouped_carve(nullptr, n_groups, x_rows, pairs, cols, &end);
    return end;
}
int launch_gemm_grouped(const frk_weights *w, size_t n_groups, const int32_t *group_off, const int32_t *gather,
                        const float *x, size_t x_rows, size_t pairs, float *y, void *ws, hipStream_t s) {
    const size_t rows_g = w->rows / n_groups, cols = w->cols, rows = moe_max_rows(pairs, (int)n_groups);
    const GroupedScratch m = grouped_carve(ws, n_groups, x_rows, pairs, cols, nullptr);
    const int max_tiles = (int)(rows / MOE_TILE);
    const GroupedTilesArgs ta{group_off, gather, (int)n_groups, (int)pairs, (int)x_rows, (int)rows, m.src_rows, m.tiles, m.n_tiles};
    if (w->kind == FRK_KIND_Q4_K && gemm_q4_k_stream_gathers(x_rows, cols)) {
        const size_t n_blocks = x_rows * (cols / QK_K);
        const unsigned quantizers = (unsigned)std::min<size_t>((n_blocks + 15) / 16, 512);
        hipLaunchKernelGGL(grouped_tiles_quantize_kernel, dim3(1 + quantizers), dim3(1024), 0, s, ta, x, (int)n_blocks, m.xr);
        FRK_LAUNCH_CHECK("grouped_tiles_quantize");
        return launch_gemm_q4_k_stream(w, nullptr, rows_g, m.xa, &m.xr, m.src_rows, m.tiles, m.n_tiles, max_tiles, y, nullptr, s);
    }
    hipLaunchKernelGGL(grouped_tiles_kernel, dim3(1), dim3(1024), 0, s, ta);
    FRK_LAUNCH_CHECK("grouped_tiles");
    int rc = launch_quantize_q8_k_gather(x, cols, m.src_rows, rows, m.xa, s);
    if (rc) return rc;
    return w->kind == FRK_KIND_Q6_K
               ? launch_gemm_q6_k_grouped(w, rows_g, m.xa, m.tiles, m.n_tiles, max_tiles, y, s)
               : launch_gemm_q4_k_stream(w, nullptr, rows_g, m.xa, nullptr, nullptr, m.tiles, m.n_tiles, max_tiles, y, nullptr, s);
}

// Experts in Q5_0 / IQ4_XS / MXFP4 (run_expert takes any WeightMatrix, crates/frink-moe/src/lib.rs:1068-1165; gpt-oss
// keeps its experts in MXFP4): every (token, slot) pair is a job of the integer decode kernel -- gate and up over the
// token's quantized activation, silu(g) * u, that row quantized, down -- and the weighted sum in the reference's order
// for the batch size.  Q8_0 activation blocks for Q5_0 and MXFP4 projections, Q8_K for IQ4_XS ones.  (A batch of
// hundreds of tokens would read an expert's matrices once per pair here: from 32 tokens on the layer takes the
// bucketed path below instead, where the kinds have a decoded form.)
struct UnitsActs {
    int8_t *q;
    float *d;
    int16_t *bsums;  // Q8_K only
};
static size_t units_acts_bytes(size_t rows, size_t cols) {
    return round_up(rows * cols, 256) + round_up(rows * cols / 32 * 4, 256) + round_up(rows * cols / 16 * 2, 256);
}
static UnitsActs units_acts_carve(char *base, size_t rows, size_t cols) {
    UnitsActs a;
    a.q = (int8_t *)base;
    a.d = (float *)(base + round_up(rows * cols, 256));
    a.bsums = (int16_t *)(base + round_up(rows * cols, 256) + round_up(rows * cols / 32 * 4, 256));
    return a;
}
static int quantize_for_units(int kind, const float *x, size_t n, const UnitsActs &a, hipStream_t s) {
    return kind == FRK_KIND_IQ4_XS ? launch_quantize_q8_k(x, n, a.q, a.d, a.bsums, s) : launch_quantize_q8_0(x, n, a.q, a.d, s);
}
size_t moe_units_workspace_bytes(size_t batch, int k, int hidden, int ffn) {
    const size_t pairs = batch * (size_t)k;
    return units_acts_bytes(batch, hidden) + 2 * round_up(pairs * ffn * 4, 256) + units_acts_bytes(pairs, ffn) +
           round_up(pairs * hidden * 4, 256);
}
int launch_moe_ffn_units(const frk_weights *gate, const frk_weights *up, const frk_weights *down, int n_experts, const float *x,
                         size_t batch, const int32_t *ids, const float *weights, int k, float *out, void *ws, hipStream_t s) {
    const int hidden = (int)gate->cols, ffn = (int)down->cols;
    const size_t pairs = batch * (size_t)k;
    char *p = (char *)ws;
    const UnitsActs xa = units_acts_carve(p, batch, hidden);
    p += units_acts_bytes(batch, hidden);
    float *g_out = (float *)p;
    p += round_up(pairs * ffn * 4, 256);
    float *u_out = (float *)p;
    p += round_up(pairs * ffn * 4, 256);
    const UnitsActs aa = units_acts_carve(p, pairs, ffn);
    p += units_acts_bytes(pairs, ffn);
    float *d_out = (float *)p;
    int rc = quantize_for_units(gate->kind, x, batch * (size_t)hidden, xa, s);
    if (rc) return rc;
    // five launches: the tokens quantized; gate and up of every pair; silu(g) * u quantized; down; the weighted sum
    rc = launch_gemv_units_int_jobs(gate, up, (size_t)ffn, n_experts, ids, pairs, k, xa.q, xa.d, g_out, u_out, s);
    if (rc) return rc;
    rc = down->kind == FRK_KIND_IQ4_XS ? launch_swiglu_quantize_q8_k(g_out, u_out, pairs * (size_t)ffn, aa.q, aa.d, aa.bsums, s)
                                      : launch_swiglu_quantize_q8_0(g_out, u_out, pairs * (size_t)ffn, aa.q, aa.d, s);
    if (rc) return rc;
    rc = launch_gemv_units_int_jobs(down, nullptr, (size_t)hidden, n_experts, ids, pairs, 1, aa.q, aa.d, d_out, nullptr, s);
    if (rc) return rc;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)batch, (unsigned)((hidden + 1023) / 1024)), dim3(256), 0, s, d_out, ids, weights,
                       (const int *)nullptr, k, hidden, n_experts, (int)(batch >= MOE_BUCKET_ORDER_FROM), out);
    FRK_LAUNCH_CHECK("moe_combine");
    return FRK_OK;
}

// The same layer from 32 tokens on, when every projection's kind has a decoded form the matrix cores read (Q5_0;
// MXFP4 with scales that are f16 values; IQ4_XS): the reference's bucket path (crates/frink-models/src/decoder/
// ffn_batch.rs:343-434) -- the pairs bucketed by expert, every expert's rows read once -- with the experts decoded
// into signed bytes in the call's scratch memory and the grouped form of the Q8_0 matrix-core kernel.  The
// activations are quantized per token (gate and up) and per grouped row (down) exactly as the per-pair jobs
// quantize them, and the integers are the same: the two paths differ in the order of the float additions only.
bool moe_units_takes_grouped_path(const frk_weights *gate, const frk_weights *up, const frk_weights *down, size_t batch) {
    return batch >= MOE_BUCKET_ORDER_FROM && units_have_planar_form(gate) && units_have_planar_form(up) && units_have_planar_form(down);
}
struct UnitsGroupedScratch {
    uint8_t *gate_w, *up_w, *down_w;  // decoded experts
    char *x_acts, *a_acts;            // quantized token rows; quantized intermediate rows (grouped order)
    float *gate_out, *up_out, *down_out;
    int *group_off, *gather, *pos_of, *cpos_of, *n_tiles;
    int4 *tiles;
};
// room for a batch of rows quantized either way: Q8_0 blocks in the GEMM's form, or Q8_K (quants, scales, sums)
static size_t units_grouped_acts_bytes(size_t rows, size_t cols) {
    const size_t q8k = round_up(rows * cols, 256) + round_up(rows * cols / QK_K * 4 + 4, 256) + round_up(rows * cols / 16 * 2 + 2, 256);
    return std::max(q8_0_gemm_acts_bytes(rows, cols), q8k);
}
static UnitsGroupedScratch units_grouped_carve(void *base, size_t batch, int k, int n_experts, int hidden, int ffn, size_t *end) {
    const size_t pairs = batch * (size_t)k, rows = moe_max_rows(pairs, n_experts);
    char *p = (char *)base;
    auto take = [&](size_t bytes) {
        char *r = p;
        p += round_up(bytes, 256);
        return r;
    };
    UnitsGroupedScratch m;
    m.gate_w = (uint8_t *)take(units_planar_bytes((size_t)n_experts * ffn, hidden));
    m.up_w = (uint8_t *)take(units_planar_bytes((size_t)n_experts * ffn, hidden));
    m.down_w = (uint8_t *)take(units_planar_bytes((size_t)n_experts * hidden, ffn));
    m.x_acts = take(units_grouped_acts_bytes(batch, hidden));
    m.a_acts = take(units_grouped_acts_bytes(rows, ffn));
    m.gate_out = (float *)take(rows * ffn * 4);
    m.up_out = (float *)take(rows * ffn * 4);
    m.down_out = (float *)take(rows * hidden * 4);
    m.group_off = (int *)take((n_experts + 1) * 4);
    m.gather = (int *)take(rows * 4);
    m.pos_of = (int *)take(pairs * 4);
    m.cpos_of = (int *)take(pairs * 4);
    m.n_tiles = (int *)take(256);
    m.tiles = (int4 *)take((rows / MOE_TILE + 1) * 16);
    if (end) *end = (size_t)(p - (char *)base);
    return m;
}
size_t moe_units_grouped_workspace_bytes(size_t batch, int k, int n_experts, int hidden, int ffn) {
    size_t end = 0;
    (void)units_grouped_carve(nullptr, batch, k, n_experts, hidden, ffn, &end);
    return end;
}
// rows x cols floats quantized into `room` for a projection of `kind`; the pointers the grouped GEMM takes
struct UnitsGroupedActs {
    const int8_t *q;
    const void *d;
};
// (with `up`: silu(x) * up is what is quantized)
static int quantize_for_units_grouped(int kind, const float *x, const float *up, size_t rows, size_t cols, char *room,
                                      UnitsGroupedActs *a, hipStream_t s) {
    int8_t *q = (int8_t *)room;
    a->q = q;
    if (kind == FRK_KIND_IQ4_XS) {
        float *d = (float *)(room + round_up(rows * cols, 256));
        int16_t *bs = (int16_t *)(room + round_up(rows * cols, 256) + round_up(rows * cols / QK_K * 4 + 4, 256));
        a->d = d;
        return up ? launch_swiglu_quantize_q8_k(x, up, rows * cols, q, d, bs, s) : launch_quantize_q8_k(x, rows * cols, q, d, bs, s);
    }
    uint16_t *d = (uint16_t *)(room + round_up(rows * cols, 256));
    a->d = d;
    return launch_quantize_q8_0_gemm(x, up, rows, cols, q, d, s);
}
// The grouped GEMM as an entry of its own over groups of these kinds: the tile list, the stack decoded, the
// activation rows quantized once (Q8_0 blocks, or Q8_K for IQ4_XS), the grouped kernel gathering through the list.
struct GroupedUnitsScratch {
    uint8_t *decoded;
    char *acts;
    int *src_rows, *n_tiles;
    int4 *tiles;
};
static GroupedUnitsScratch grouped_units_carve(void *base, size_t n_groups, size_t w_rows, size_t x_rows, size_t pairs, size_t cols,
                                               size_t *end) {
    const size_t rows = moe_max_rows(pairs, (int)n_groups);
    char *p = (char *)base;
    auto take = [&](size_t bytes) {
        char *r = p;
        p += round_up(bytes, 256);
        return r;
    };
    GroupedUnitsScratch m;
    m.decoded = (uint8_t *)take(units_planar_bytes(w_rows, cols));
    m.acts = take(units_grouped_acts_bytes(x_rows, cols));
    m.src_rows = (int *)take(rows * 4);
    m.n_tiles = (int *)take(256);
    m.tiles = (int4 *)take((rows / MOE_TILE + 1) * 16);
    if (end) *end = (size_t)(p - (char *)base);
    return m;
}
size_t grouped_units_workspace_bytes(size_t n_groups, size_t w_rows, size_t x_rows, size_t pairs, size_t cols) {
    size_t end = 0;
    (void)grouped_units_carve(nullptr, n_groups, w_rows, x_rows, pairs, cols, &end);
    return end;
}
int launch_gemm_grouped_units(const frk_weights *w, size_t n_groups, const int32_t *group_off, const int32_t *gather, const float *x,
                              size_t x_rows, size_t pairs, float *y, void *ws, hipStream_t s) {
    const size_t rows_g = w->rows / n_groups, cols = w->cols, rows = moe_max_rows(pairs, (int)n_groups);
    const GroupedUnitsScratch m = grouped_units_carve(ws, n_groups, w->rows, x_rows, pairs, cols, nullptr);
    const GroupedTilesArgs ta{group_off, gather, (int)n_groups, (int)pairs, (int)x_rows, (int)rows, m.src_rows, m.tiles, m.n_tiles};
    hipLaunchKernelGGL(grouped_tiles_kernel, dim3(1), dim3(1024), 0, s, ta);
    FRK_LAUNCH_CHECK("grouped_tiles");
    const uint8_t *decoded = nullptr;
    int rc = units_decoded(w, m.decoded, s, &decoded);
    if (rc) return rc;
    UnitsGroupedActs xa;
    rc = quantize_for_units_grouped(w->kind, x, nullptr, x_rows, cols, m.acts, &xa, s);
    if (rc) return rc;
    const Layout l = layout_for(FRK_KIND_Q8_0, cols);
    return launch_gemm_planar_grouped(decoded, l.row_stride, l.off_a, rows_g, cols, w->kind == FRK_KIND_IQ4_XS, xa.q, xa.d, m.src_rows,
                                      m.tiles, m.n_tiles, rows / MOE_TILE, y, s);
}

int launch_moe_ffn_units_grouped(const frk_weights *gate, const frk_weights *up, const frk_weights *down, int n_experts,
                                 const float *x, size_t batch, const int32_t *ids, const float *weights, int k, float *out,
                                 void *ws, hipStream_t s) {
    const int hidden = (int)gate->cols, ffn = (int)down->cols;
    const size_t pairs = batch * (size_t)k, rows = moe_max_rows(pairs, n_experts), max_tiles = rows / MOE_TILE;
    const UnitsGroupedScratch m = units_grouped_carve(ws, batch, k, n_experts, hidden, ffn, nullptr);
    static bool sized = false;  // a benign race: every thread sets the same attribute
    if (!sized) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_group_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GroupLds));
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFuncSetAttribute(moe_group): %s", hipGetErrorString(e));
        sized = true;
    }
    const GroupArgs ga{ids, (int)pairs, k, n_experts, m.group_off, m.gather, m.pos_of, m.cpos_of, m.tiles, m.n_tiles, (int)rows};
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), sizeof(GroupLds), s, ga);
    FRK_LAUNCH_CHECK("moe_group");
    const uint8_t *gate_w = nullptr, *up_w = nullptr, *down_w = nullptr;
    int rc = units_decoded(gate, m.gate_w, s, &gate_w);
    if (rc) return rc;
    rc = units_decoded(up, m.up_w, s, &up_w);
    if (rc) return rc;
    rc = units_decoded(down, m.down_w, s, &down_w);
    if (rc) return rc;
    UnitsGroupedActs xa, aa;
    rc = quantize_for_units_grouped(gate->kind, x, nullptr, batch, (size_t)hidden, m.x_acts, &xa, s);
    if (rc) return rc;
    const Layout lg = layout_for(FRK_KIND_Q8_0, (size_t)hidden), ld = layout_for(FRK_KIND_Q8_0, (size_t)ffn);
    rc = launch_gemm_planar_grouped(gate_w, lg.row_stride, lg.off_a, (size_t)ffn, (size_t)hidden, gate->kind == FRK_KIND_IQ4_XS, xa.q,
                                    xa.d, m.gather, m.tiles, m.n_tiles, max_tiles, m.gate_out, s);
    if (rc) return rc;
    rc = launch_gemm_planar_grouped(up_w, lg.row_stride, lg.off_a, (size_t)ffn, (size_t)hidden, up->kind == FRK_KIND_IQ4_XS, xa.q,
                                    xa.d, m.gather, m.tiles, m.n_tiles, max_tiles, m.up_out, s);
    if (rc) return rc;
    // silu(gate) * up, quantized in the same launch (rows of the grouped order that no pair uses hold whatever the
    // memory held: nothing reads their results)
    rc = quantize_for_units_grouped(down->kind, m.gate_out, m.up_out, rows, (size_t)ffn, m.a_acts, &aa, s);
    if (rc) return rc;
    rc = launch_gemm_planar_grouped(down_w, ld.row_stride, ld.off_a, (size_t)hidden, (size_t)ffn, down->kind == FRK_KIND_IQ4_XS, aa.q,
                                    aa.d, nullptr, m.tiles, m.n_tiles, max_tiles, m.down_out, s);
    if (rc) return rc;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)batch, (unsigned)((hidden + 1023) / 1024)), dim3(256), 0, s, m.down_out, ids,
                       weights, m.pos_of, k, hidden, n_experts, 1, out);
    FRK_LAUNCH_CHECK("moe_combine");
    return FRK_OK;
}

}  // namespace frk
