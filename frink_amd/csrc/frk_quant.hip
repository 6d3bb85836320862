// Bit-exact kernels: activation quantizers (Q8_K, Q8_0 Avx form), dequantizers, and the one-time
// byte permutation of Q6_K / Q8_0 rows into 16-byte-aligned planes.
//
// This file must be compiled with -ffp-contract=off: the reference rounds every f32 operation
// separately (d*sc, dmin*m, d1*nib, the subtraction), and a fused multiply-add changes low bits.
#include <algorithm>

#include "frk_device.hpp"

namespace frk {

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;  // exact, subnormals included
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    _Float16 v = (_Float16)f;  // round to nearest even
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

// ---- quantize_activations_q8_k (crates/frink-quant/src/act_quant.rs:69-104) ----
// One wavefront per 256-value block, four consecutive values per lane.
// GLU: what is quantized is silu(x) * up, element by element (GluAct::Swiglu, crates/frink-core/src/matmul.rs:634-650,
// in front of the down projection's own quantization, ffn_batch.rs:405-415): one launch for the two.
template <bool GLU>
__global__ __launch_bounds__(256) void quantize_q8_k_kernel(const float *__restrict__ x, const float *__restrict__ up, size_t n_blocks,
                                                            int8_t *__restrict__ q, float *__restrict__ d,
                                                            int16_t *__restrict__ bsums) {
    const int lane = threadIdx.x & 63;
    const size_t b = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= n_blocks) return;
    float4 v = reinterpret_cast<const float4 *>(x + b * QK_K)[lane];
    if (GLU) {
        const float4 u = reinterpret_cast<const float4 *>(up + b * QK_K)[lane];
        v = make_float4(silu_as_host(v.x) * u.x, silu_as_host(v.y) * u.y, silu_as_host(v.z) * u.z, silu_as_host(v.w) * u.w);
    }
    // f32::max ignores a NaN operand, as fmaxf does; max is exact, so the fold order is free
    float amax = fmaxf(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))), 0.0f);
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    int q0 = 0, q1 = 0, q2 = 0, q3 = 0;
    float dd = 0.0f;
    if (amax != 0.0f) {
        const float iscale = __fdiv_rn(127.0f, amax);
        auto quant = [&](float e) {
            const float r = rintf(iscale * e);  // round half to even
            // (f32::clamp keeps a NaN, which `as i8` turns into 0; fmaxf would turn it into -127)
            return (r != r) ? 0 : (int)fminf(fmaxf(r, -127.0f), 127.0f);
        };
        q0 = quant(v.x);
        q1 = quant(v.y);
        q2 = quant(v.z);
        q3 = quant(v.w);
        dd = __fdiv_rn(1.0f, iscale);
    }
    const uint32_t packed = (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) |
                            ((uint32_t)(q3 & 0xff) << 24);
    reinterpret_cast<uint32_t *>(q + b * QK_K)[lane] = packed;
    int s = q0 + q1 + q2 + q3;  // four lanes make one 16-wide group
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    if ((lane & 3) == 0) bsums[b * 16 + (lane >> 2)] = (int16_t)s;
    if (lane == 0) d[b] = dd;
}

// ---- quantize_activations_q8, Avx form (crates/frink-quant/src/act_quant.rs:157-189) ----
// Eight lanes per 32-value block.
template <bool GLU>
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float *__restrict__ x, const float *__restrict__ up, size_t n_blocks,
                                                            int8_t *__restrict__ q, float *__restrict__ d) {
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
    if ((t & 7) == 0) d[b] = f16_bits_to_f32(f32_to_f16_bits(scale));  // d is what an f16 field holds
}

// ---- row permutation into the resident layout ----
__global__ __launch_bounds__(256) void repack_kernel(int kind, const uint8_t *__restrict__ src,
                                                     uint8_t *__restrict__ dst, size_t rows, size_t src_row_bytes,
                                                     Layout l) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * src_row_bytes) return;
    const size_t r = i / src_row_bytes, o = i % src_row_bytes;
    size_t to;
    if (kind == FRK_KIND_Q6_K) {
        const size_t blk = o / Q6_K_BYTES, w = o % Q6_K_BYTES;
        if (w < 128) to = blk * 128 + w;
        else if (w < 192) to = l.off_a + blk * 64 + (w - 128);
        else if (w < 208) to = l.off_b + blk * 16 + (w - 192);
        else to = l.off_c + blk * 2 + (w - 208);
    } else if (kind == FRK_KIND_Q8_0) {
        const size_t blk = o / Q8_0_BYTES, w = o % Q8_0_BYTES;
        to = w < 2 ? l.off_a + blk * 2 + w : blk * 32 + (w - 2);
    } else if (kind == FRK_KIND_Q4_0) {
        const size_t blk = o / Q4_0_BYTES, w = o % Q4_0_BYTES;
        to = w < 2 ? l.off_a + blk * 2 + w : blk * 16 + (w - 2);
    } else {
        to = o;
    }
    dst[r * l.row_stride + to] = src[i];
}

// ---- dequantizers, one thread per element, reading the resident layout ----
// With a list of row numbers they are the embedding gather (get_rows, crates/frink-cuda/src/get_rows.rs:
// output row r is the dequantized row ids[r], bit for bit what the dequantizer gives); a number outside
// the table reads its nearest row instead of faulting (the host-side entry point refuses such lists).
__device__ __forceinline__ size_t source_row(size_t r, const int32_t *ids, size_t table_rows) {
    if (!ids) return r;
    const int32_t id = ids[r];
    return id < 0 ? 0 : (size_t)id >= table_rows ? table_rows - 1 : (size_t)id;
}
// dequant_q4_k (crates/frink-quant/src/lib.rs:334-364)
__global__ __launch_bounds__(256) void dequant_q4_k_kernel(const uint8_t *__restrict__ w, size_t rows, size_t cols,
                                                           size_t row_stride, const int32_t *__restrict__ ids, size_t table_rows,
                                                           float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * cols) return;
    const size_t r = source_row(i / cols, ids, table_rows), c = i % cols;
    const uint8_t *blk = w + r * row_stride + (c / QK_K) * Q4_K_BYTES;
    const int e = (int)(c % QK_K), sub = e >> 5, within = e & 31;
    const uint8_t *s = blk + 4;
    int sc, m;
    if (sub < 4) {
        sc = s[sub] & 63;
        m = s[sub + 4] & 63;
    } else {
        sc = (s[sub + 4] & 0x0F) | ((s[sub - 4] >> 6) << 4);
        m = (s[sub + 4] >> 4) | ((s[sub] >> 6) << 4);
    }
    const float d = f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    const float dmin = f16_bits_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
    const uint8_t byte = blk[16 + (sub >> 1) * 32 + within];
    const int nib = (sub & 1) ? (byte >> 4) : (byte & 15);
    const float d1 = d * (float)sc;
    const float min1 = dmin * (float)m;
    out[i] = d1 * (float)nib - min1;
}

// dequant_q5_k (crates/frink-quant/src/lib.rs:424-459): Q4_K's arithmetic on a five-bit code, whose
// top bit is bit `sub` of qh[within] (the 32 bytes behind the header)
__global__ __launch_bounds__(256) void dequant_q5_k_kernel(const uint8_t *__restrict__ w, size_t rows, size_t cols,
                                                           size_t row_stride, const int32_t *__restrict__ ids, size_t table_rows,
                                                           float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * cols) return;
    const size_t r = source_row(i / cols, ids, table_rows), c = i % cols;
    const uint8_t *blk = w + r * row_stride + (c / QK_K) * Q5_K_BYTES;
    const int e = (int)(c % QK_K), sub = e >> 5, within = e & 31;
    const uint8_t *s = blk + 4;
    int sc, m;
    if (sub < 4) {
        sc = s[sub] & 63;
        m = s[sub + 4] & 63;
    } else {
        sc = (s[sub + 4] & 0x0F) | ((s[sub - 4] >> 6) << 4);
        m = (s[sub + 4] >> 4) | ((s[sub] >> 6) << 4);
    }
    const float d = f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    const float dmin = f16_bits_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
    const uint8_t byte = blk[48 + (sub >> 1) * 32 + within];
    const int code = ((sub & 1) ? (byte >> 4) : (byte & 15)) + 16 * ((blk[16 + within] >> sub) & 1);
    const float d1 = d * (float)sc;
    const float min1 = dmin * (float)m;
    out[i] = d1 * (float)code - min1;
}

// dequant_q6_k (crates/frink-quant/src/lib.rs:519-552)
__global__ __launch_bounds__(256) void dequant_q6_k_kernel(const uint8_t *__restrict__ w, size_t rows, size_t cols,
                                                           Layout l, const int32_t *__restrict__ ids, size_t table_rows,
                                                           float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * cols) return;
    const size_t r = source_row(i / cols, ids, table_rows), c = i % cols, b = c / QK_K;
    const uint8_t *row = w + r * l.row_stride;
    const int e = (int)(c % QK_K), half = e >> 7, rem = e & 127, quarter = rem >> 5, ll = rem & 31;
    const int qlb = row[b * 128 + half * 64 + (quarter & 1) * 32 + ll];
    const int lo = (quarter & 2) ? (qlb >> 4) : (qlb & 15);
    const int hi = (row[l.off_a + b * 64 + half * 32 + ll] >> (2 * quarter)) & 3;
    const int qv = (lo | (hi << 4)) - 32;
    const int sc = (int8_t)row[l.off_b + b * 16 + (e >> 4)];
    const uint8_t *dp = row + l.off_c + b * 2;
    const float d = f16_bits_to_f32((uint16_t)(dp[0] | (dp[1] << 8)));
    out[i] = d * (float)sc * (float)qv;
}

// dequant_q8_0 (crates/frink-quant/src/lib.rs:271-286)
__global__ __launch_bounds__(256) void dequant_q8_0_kernel(const uint8_t *__restrict__ w, size_t rows, size_t cols,
                                                           Layout l, const int32_t *__restrict__ ids, size_t table_rows,
                                                           float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * cols) return;
    const size_t r = source_row(i / cols, ids, table_rows), c = i % cols, b = c / Q8_0_ELEMS;
    const uint8_t *row = w + r * l.row_stride;
    const uint8_t *dp = row + l.off_a + b * 2;
    const float scale = f16_bits_to_f32((uint16_t)(dp[0] | (dp[1] << 8)));
    out[i] = (float)(int8_t)row[c] * scale;
}

// dequant_q4_0 (crates/frink-quant/src/lib.rs:291-310): byte i of a block holds element i in its low
// nibble and element i + 16 in its high one
__global__ __launch_bounds__(256) void dequant_q4_0_kernel(const uint8_t *__restrict__ w, size_t rows, size_t cols,
                                                           Layout l, const int32_t *__restrict__ ids, size_t table_rows,
                                                           float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * cols) return;
    const size_t r = source_row(i / cols, ids, table_rows), c = i % cols, b = c / Q8_0_ELEMS;
    const int e = (int)(c % Q8_0_ELEMS);
    const uint8_t *row = w + r * l.row_stride;
    const uint8_t *dp = row + l.off_a + b * 2;
    const float scale = f16_bits_to_f32((uint16_t)(dp[0] | (dp[1] << 8)));
    const uint8_t byte = row[b * 16 + (e & 15)];
    const int nib = e < 16 ? (byte & 15) : (byte >> 4);
    out[i] = (float)(nib - 8) * scale;
}

// ---- bandwidth calibration kernels ----
__global__ __launch_bounds__(256) void copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// (Two 16-byte loads a thread and round, up to 8192 workgroups: the fastest of the shapes tried for
// 8 .. 280 MB -- four loads a thread over 2048 workgroups took 5 % longer at 33 MB.)
__global__ __launch_bounds__(256) void read_kernel(const uint4 *__restrict__ src, size_t n, uint32_t *__restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * 512;
    uint32_t acc = 0;
    size_t base = (size_t)blockIdx.x * 512;
    for (; base + 512 <= n; base += stride) {
        const uint4 *p = src + base + threadIdx.x;
        // (non-temporal loads: 0.4 us of 6.4 at 33 MB)
        typedef uint32_t nt4_t __attribute__((ext_vector_type(4)));
        const nt4_t a = __builtin_nontemporal_load(reinterpret_cast<const nt4_t *>(p));
        const nt4_t b = __builtin_nontemporal_load(reinterpret_cast<const nt4_t *>(p + 256));
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w;
    }
    if (base < n) {  // at most one workgroup holds the ragged tail
        for (size_t i = base + threadIdx.x; i < n; i += 256) {
            const uint4 a = src[i];
            acc ^= a.x ^ a.y ^ a.z ^ a.w;
        }
    }
    // (The loads must be used, not more: a reduction over the wavefront and a store at the end of every wavefront
    // made this kernel 0.6 us longer at 33 MB -- 7.46 against 6.88 -- than the same loads without them.  A word
    // that never takes this value in the buffers measured keeps the compiler from dropping the loads.)
    if (acc == 0x9e3779b9u) sink[(blockIdx.x * 256 + threadIdx.x) & 16383] = acc;
}

static inline unsigned blocks_for(size_t n, size_t per) { return (unsigned)((n + per - 1) / per); }

#define FRK_LAUNCH_CHECK(what)                                                                   \
    do {                                                                                         \
        hipError_t e_ = hipGetLastError();                                                       \
        if (e_ != hipSuccess) return set_error(FRK_ERR_HIP, what " launch: %s", hipGetErrorString(e_)); \
    } while (0)

int launch_quantize_q8_k(const float *x, size_t n, int8_t *q, float *d, int16_t *bsums, hipStream_t s) {
    const size_t nb = n / QK_K;
    hipLaunchKernelGGL(quantize_q8_k_kernel<false>, dim3(blocks_for(nb, 4)), dim3(256), 0, s, x, (const float *)nullptr, nb, q, d, bsums);
    FRK_LAUNCH_CHECK("quantize_q8_k");
    return FRK_OK;
}

int launch_quantize_q8_0(const float *x, size_t n, int8_t *q, float *d, hipStream_t s) {
    const size_t nb = n / Q8_0_ELEMS;
    hipLaunchKernelGGL(quantize_q8_0_kernel<false>, dim3(blocks_for(nb * 8, 256)), dim3(256), 0, s, x, (const float *)nullptr, nb, q, d);
    FRK_LAUNCH_CHECK("quantize_q8_0");
    return FRK_OK;
}

// silu(gate) * up quantized in the same launch (n a multiple of the block)
int launch_swiglu_quantize_q8_k(const float *gate, const float *up, size_t n, int8_t *q, float *d, int16_t *bsums, hipStream_t s) {
    const size_t nb = n / QK_K;
    hipLaunchKernelGGL(quantize_q8_k_kernel<true>, dim3(blocks_for(nb, 4)), dim3(256), 0, s, gate, up, nb, q, d, bsums);
    FRK_LAUNCH_CHECK("swiglu_quantize_q8_k");
    return FRK_OK;
}
int launch_swiglu_quantize_q8_0(const float *gate, const float *up, size_t n, int8_t *q, float *d, hipStream_t s) {
    const size_t nb = n / Q8_0_ELEMS;
    hipLaunchKernelGGL(quantize_q8_0_kernel<true>, dim3(blocks_for(nb * 8, 256)), dim3(256), 0, s, gate, up, nb, q, d);
    FRK_LAUNCH_CHECK("swiglu_quantize_q8_0");
    return FRK_OK;
}

int launch_repack(int kind, const uint8_t *src, uint8_t *dst, size_t rows, size_t cols, const Layout &l,
                  hipStream_t s) {
    const size_t src_row_bytes = cols / (size_t)block_elems(kind) * (size_t)block_bytes(kind);
    if (kind == FRK_KIND_Q4_K || kind == FRK_KIND_Q5_K) {
        hipError_t e = hipMemcpyAsync(dst, src, rows * src_row_bytes, hipMemcpyDeviceToDevice, s);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipMemcpyAsync(weights): %s", hipGetErrorString(e));
        return FRK_OK;
    }
    if (l.row_stride != src_row_bytes) {
        hipError_t e = hipMemsetAsync(dst, 0, rows * l.row_stride, s);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipMemsetAsync: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(repack_kernel, dim3(blocks_for(rows * src_row_bytes, 256)), dim3(256), 0, s, kind, src, dst,
                       rows, src_row_bytes, l);
    FRK_LAUNCH_CHECK("repack");
    return FRK_OK;
}

// out[n_out][cols]: every row of the matrix (ids == nullptr, n_out == rows) or the rows ids[0..n_out)
int launch_dequant_rows(const frk_weights *w, const int32_t *ids, size_t n_out, float *out, hipStream_t s) {
    if (n_out == 0) return FRK_OK;
    if (is_unit_kind(w->kind)) return launch_dequant_units(w, ids, n_out, out, s);
    const unsigned g = blocks_for(n_out * w->cols, 256);
    switch (w->kind) {
    case FRK_KIND_Q4_K:
        hipLaunchKernelGGL(dequant_q4_k_kernel, dim3(g), dim3(256), 0, s, w->dev, n_out, w->cols, w->layout.row_stride, ids,
                           w->rows, out);
        break;
    case FRK_KIND_Q5_K:
        hipLaunchKernelGGL(dequant_q5_k_kernel, dim3(g), dim3(256), 0, s, w->dev, n_out, w->cols, w->layout.row_stride, ids,
                           w->rows, out);
        break;
    case FRK_KIND_Q6_K:
        hipLaunchKernelGGL(dequant_q6_k_kernel, dim3(g), dim3(256), 0, s, w->dev, n_out, w->cols, w->layout, ids, w->rows, out);
        break;
    case FRK_KIND_Q8_0:
        hipLaunchKernelGGL(dequant_q8_0_kernel, dim3(g), dim3(256), 0, s, w->dev, n_out, w->cols, w->layout, ids, w->rows, out);
        break;
    case FRK_KIND_Q4_0:
        hipLaunchKernelGGL(dequant_q4_0_kernel, dim3(g), dim3(256), 0, s, w->dev, n_out, w->cols, w->layout, ids, w->rows, out);
        break;
    default:
        return set_error(FRK_ERR_UNSUPPORTED, "no dequantizer for quant kind %d", w->kind);
    }
    FRK_LAUNCH_CHECK("dequant");
    return FRK_OK;
}

int launch_dequant(const frk_weights *w, float *out, hipStream_t s) { return launch_dequant_rows(w, nullptr, w->rows, out, s); }

int launch_copy(const void *src, void *dst, size_t bytes, hipStream_t s) {
    const size_t n = bytes / 16;
    if (n == 0) return FRK_OK;
    const unsigned g = (unsigned)std::min<size_t>(blocks_for(n, 256), 256 * 16);
    hipLaunchKernelGGL(copy_kernel, dim3(g), dim3(256), 0, s, (const uint4 *)src, (uint4 *)dst, n);
    FRK_LAUNCH_CHECK("copy");
    return FRK_OK;
}

int launch_read(const void *src, size_t bytes, void *sink, hipStream_t s) {
    const size_t n = bytes / 16;
    if (n == 0) return FRK_OK;
    const unsigned g = (unsigned)std::min<size_t>(blocks_for(n, 512), 8192);
    hipLaunchKernelGGL(read_kernel, dim3(g), dim3(256), 0, s, (const uint4 *)src, n, (uint32_t *)sink);
    FRK_LAUNCH_CHECK("read");
    return FRK_OK;
}

}  // namespace frk
