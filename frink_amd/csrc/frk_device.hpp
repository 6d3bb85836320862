// Device-side helpers shared by the kernels: f16 conversion, dot4, DPP reductions and the Q8_K
// block quantizer.
#pragma once

#include "frk_internal.hpp"

namespace frk {

__device__ __forceinline__ float h2f(uint32_t bits16) {
    _Float16 v;
    uint16_t h = (uint16_t)bits16;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;  // exact, subnormals included
}

__device__ __forceinline__ uint16_t f2h_bits(float f) {
    _Float16 v = (_Float16)f;  // round to nearest even
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// v (op) lane-permuted v, the permutation given by a DPP control word
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}

// Workgroup barrier that publishes LDS writes but does NOT wait for outstanding global loads.
// __syncthreads() is a full fence: it drains vmcnt too, which would stall every wavefront until
// all the weight loads it prefetched have landed.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// global_load_lds: every lane names its own global source; the wavefront's 64 pieces of BYTES
// (4 or 16) bytes land in LDS at lds_chunk + BYTES * lane, without passing through registers.
// Completion is counted by vmcnt like any other global load.  lds_chunk must be wavefront-uniform.
// (The builtin exists in the device pass only, hence the guard.)
__device__ __forceinline__ void load_to_lds16(const void *src, void *lds_chunk) {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void *)lds_chunk, 16, 0, 0);
#endif
}
__device__ __forceinline__ void load_to_lds4(const void *src, void *lds_chunk) {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void *)lds_chunk, 4, 0, 0);
#endif
}

// global_load_lds from a wavefront-uniform base (scalar registers) plus a 32-bit lane offset; the 64
// lanes' pieces land at lds_uniform + 16 (or 4) * lane.  Counted by vmcnt.
// (readfirstlane costs nothing on a value the compiler already keeps in scalar registers and makes the
// operands scalar where its uniformity analysis gives up)
__device__ __forceinline__ const void *scalar_pointer(const void *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const void *>(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ void dma16(uint32_t lds_uniform, const void *base_uniform, uint32_t lane_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_uniform)), "v"(lane_off), "s"(scalar_pointer(base_uniform))
                 : "memory");
}
// Loads with the non-temporal bit, for weights a decode step fetches once (see dma16_nt for what the bit buys).
typedef uint32_t nt_u4_t __attribute__((ext_vector_type(4)));
typedef uint32_t nt_u2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 stream_load16(const void *p) {
    const nt_u4_t v = __builtin_nontemporal_load(reinterpret_cast<const nt_u4_t *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 stream_load8(const void *p) {
    const nt_u2_t v = __builtin_nontemporal_load(reinterpret_cast<const nt_u2_t *>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint16_t stream_load2(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const uint16_t *>(p));
}
// The same with the non-temporal bit: for data fetched once per launch (a decode step's weights).  Measured on
// the bare fetch of 33 MB in 9 KB spans, cache-cold: 5.97 us per launch with the bit, 6.45 without.
__device__ __forceinline__ void dma16_nt(uint32_t lds_uniform, const void *base_uniform, uint32_t lane_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_uniform)), "v"(lane_off), "s"(scalar_pointer(base_uniform))
                 : "memory");
}
__device__ __forceinline__ void dma4(uint32_t lds_uniform, const void *base_uniform, uint32_t lane_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_uniform)), "v"(lane_off), "s"(scalar_pointer(base_uniform))
                 : "memory");
}
// the 32-bit LDS address of a pointer into shared memory, for LDS instructions written as inline assembly
__device__ __forceinline__ uint32_t lds_address(const void *p) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
#else
    return 0;
#endif
}

// a 32-bit LDS store the compiler does not see (its LDS address from lds_address)
__device__ __forceinline__ void lds_store32(uint32_t addr, uint32_t value) {
    asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(value) : "memory");
}

typedef uint32_t lds_u4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_store128(uint32_t addr, lds_u4 value) {
    asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"(value) : "memory");
}

constexpr int DPP_QUAD_XOR1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141;  // lane i <- lane 7-i of its group of 8
constexpr int DPP_ROW_MIRROR = 0x140;   // lane i <- lane 15-i of its row of 16

// Sum over the LPR lanes (8, 16, 32 or 64) that share a row; every lane ends with the total.
template <int LPR>
__device__ __forceinline__ float part_sum(float v) {
    v += dpp_f<DPP_QUAD_XOR1>(v);
    v += dpp_f<DPP_QUAD_XOR2>(v);
    v += dpp_f<DPP_HALF_MIRROR>(v);
    if (LPR >= 16) v += dpp_f<DPP_ROW_MIRROR>(v);
    if (LPR >= 32) v += __shfl_xor(v, 16);
    if (LPR >= 64) v += __shfl_xor(v, 32);
    return v;
}

// Max over all 64 lanes.  max is exact, so any fold order gives the reference's amax.
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR2>(v));
    v = fmaxf(v, dpp_f<DPP_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f<DPP_ROW_MIRROR>(v));  // every lane of a row of 16 holds its row's maximum
    // across the rows without a trip through LDS: the row before's last lane into rows 1 and 3, lane 31 into rows 2
    // and 3 (row_bcast15 / row_bcast31, other rows keep their value), and lane 63's total read out as a scalar
#if defined(__HIP_DEVICE_COMPILE__)
    const int r1 = __builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x142, 0xa, 0xf, false);
    v = fmaxf(v, __int_as_float(r1));
    const int r2 = __builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x143, 0xc, 0xf, false);
    v = fmaxf(v, __int_as_float(r2));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
#else
    return v;
#endif
}

// expf the way glibc computes it (2.28 and later, every architecture: sysdeps/ieee754/flt-32/e_expf.c, the
// algorithm of ARM's optimized routines): in double, exp(x) = 2^(k/32) * 2^(r/32) with k = round(32 x / ln 2),
// 2^(k/32) from a table of 32 correctly rounded values (the exponent added to the table entry's bits) and a
// cubic for the rest, rounded to f32 once.  Rust's f32::exp is the platform's expf (the reference's silu:
// crates/frink-core/src/matmul.rs:634-650), so this returns a Linux host's bits (a build of glibc that fuses
// the cubic's multiply-adds differs in the double's last bits, which reaches the f32 in about one value in
// 2^29) at a third of the instructions of a correctly rounded double exp.
__constant__ const uint64_t EXPF_TABLE[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};
// In two steps, so that a caller can fetch the table entries of several values at once: the reduction
// (r and the integer k, whose low five bits select the entry) and the rest.  Outside the range where the
// result is a finite, non-zero f32 glibc returns inf, 0 or (just above the underflow threshold, its "may
// underflow" path) the smallest subnormal; a NaN comes out of the arithmetic as a NaN.
struct ExpfReduced {
    double r;
    uint32_t k;
};
__device__ __forceinline__ ExpfReduced expf_reduce(float x) {
    constexpr double INV_LN2_N = 0x1.71547652b82fep+0 * 32.0, SHIFT = 0x1.8p+52;
    const double z = INV_LN2_N * (double)x;
    double kd = z + SHIFT;  // the integer nearest to z sits in the low bits
    const uint32_t k = (uint32_t)__double_as_longlong(kd);
    kd -= SHIFT;
    return {z - kd, k};
}
__device__ __forceinline__ float expf_finish(float x, const ExpfReduced &a, uint64_t entry) {
    constexpr double N = 32.0;
    constexpr double C0 = 0x1.c6af84b912394p-5 / N / N / N, C1 = 0x1.ebfce50fac4f3p-3 / N / N, C2 = 0x1.62e42ff0c52d6p-1 / N;
    const double s = __longlong_as_double((long long)(entry + ((uint64_t)a.k << 47)));
    const double p = C0 * a.r + C1;
    const double r2 = a.r * a.r;
    double y = C2 * a.r + 1.0;
    y = p * r2 + y;
    float e = (float)(y * s);
    if (x > 0x1.62e42ep6f) e = INFINITY;
    if (x < -0x1.9d1d9ep6f) e = x < -0x1.9fe368p6f ? 0.0f : 0x1p-149f;
    return e;
}
// (`table`: EXPF_TABLE or a copy of it)
__device__ __forceinline__ float expf_as_libm(float x, const uint64_t *table = EXPF_TABLE) {
    const ExpfReduced a = expf_reduce(x);
    return expf_finish(x, a, table[a.k & 31]);
}
// x * sigmoid(x) as the reference's hosts compute it: x / (1 + expf(-x)), each step rounded to f32
__device__ __forceinline__ float silu_as_host(float x, const uint64_t *table = EXPF_TABLE) {
    return __fdiv_rn(x, 1.0f + expf_as_libm(-x, table));
}

// quantize_activations_q8_k (crates/frink-quant/src/act_quant.rs:69-104) for one 256-value block
// held four consecutive values per lane by one wavefront.  Returns the lane's four quants packed
// little-endian; d_out is the block scale (same in every lane); bsum16 is the sum of the 16-wide
// group this lane belongs to (same in the four lanes of a quad).
// BRANCHES false: an all-zero block is a select at the end instead of a branch around the arithmetic (the
// same results: 127 / 0 is an infinity whose products are dropped by the select, and 1 / inf is the zero
// scale), so that a wavefront quantizing several blocks can interleave their dependent chains.
template <bool BRANCHES = true>
__device__ __forceinline__ uint32_t quantize_q8_k_lane(float4 v, float &d_out, int &bsum16) {
    // f32::max ignores a NaN operand, as fmaxf does, and the fold starts from 0: a block of NaNs has the maximum 0
    const float amax = wave_max(fmaxf(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))), 0.0f));
    int q0 = 0, q1 = 0, q2 = 0, q3 = 0;
    d_out = 0.0f;
    if (!BRANCHES || amax != 0.0f) {  // uniform across the wavefront
        const float iscale = __fdiv_rn(127.0f, amax);
        auto quant = [&](float e) {
            const float r = rintf(iscale * e);  // round half to even
            // a NaN becomes 0: f32::clamp keeps it and `as i8` makes it 0 (fmaxf would turn it into -127)
            return (r != r || (!BRANCHES && amax == 0.0f)) ? 0 : (int)fminf(fmaxf(r, -127.0f), 127.0f);
        };
        q0 = quant(v.x);
        q1 = quant(v.y);
        q2 = quant(v.z);
        q3 = quant(v.w);
        d_out = __fdiv_rn(1.0f, iscale);
    }
    int s = q0 + q1 + q2 + q3;
    s += dpp_i<DPP_QUAD_XOR1>(s);
    s += dpp_i<DPP_QUAD_XOR2>(s);
    bsum16 = s;
    return (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) |
           ((uint32_t)(q3 & 0xff) << 24);
}

// One record of the tiled Q8_K form (32 rows x one 256-wide block) by a workgroup of WAVES wavefronts
// (4, 8 or 16): wavefront w quantizes rows 32/WAVES * w .. (`load(r)` returns this lane's four values of
// row r, zeros for a row that does not exist; all of a wavefront's loads are in flight before its
// first row is quantized), the record is put together in LDS and leaves as three contiguous copies
// -- quantizing straight into the tiled form would write it in 4-byte pieces.  These kernels are
// bound by latency: few records want many wavefronts each, many records small workgroups.
struct Q8KRecordLds {
    uint32_t q[2048];
    _Float16 bs[512];
    float d[32];
};
template <int WAVES, class Load>
__device__ __forceinline__ void quantize_q8k_record(const Q8KTiled &a, size_t rec, Q8KRecordLds &L, Load load) {
    constexpr int RPW = 32 / WAVES;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float4 v[RPW];
#pragma unroll
    for (int i = 0; i < RPW; i++) v[i] = load(wave * RPW + i);
    // the lane's four values are k = 4*lane..: 32-wide slice lane/8, 16-byte half (lane/4)%2 of it
    const int ks = lane >> 3, half = (lane >> 2) & 1, g = lane >> 2;
#pragma unroll
    for (int i = 0; i < RPW; i++) {
        const int r = wave * RPW + i;
        float dd;
        int bs;
        const uint32_t packed = quantize_q8_k_lane(v[i], dd, bs);
        L.q[ks * 256 + (half * 32 + r) * 4 + (lane & 3)] = packed;
        if ((lane & 3) == 0) L.bs[((g >> 3) * 32 + r) * 8 + (g & 7)] = (_Float16)bs;
        if (lane == 0) L.d[r] = dd;
    }
    __syncthreads();
    uint4 *dq = reinterpret_cast<uint4 *>(a.q + rec * 8192);
    const uint4 *sq = reinterpret_cast<const uint4 *>(L.q);
    for (int i = tid; i < 512; i += 64 * WAVES) dq[i] = sq[i];
    if (tid < 64) reinterpret_cast<uint4 *>(a.bs + rec * 512)[tid] = reinterpret_cast<const uint4 *>(L.bs)[tid];
    if (tid < 32) a.d[rec * 32 + tid] = L.d[tid];
}
// where quant k of (row, block kb) lives in the tiled form
__device__ __forceinline__ size_t q8k_tiled_index(int nb, int row, int kb, int k) {
    const size_t rec = (size_t)(row >> 5) * nb + kb;
    return rec * 8192 + (k >> 5) * 1024 + (((k >> 4) & 1) * 32 + (row & 31)) * 16 + (k & 15);
}

}  // namespace frk
