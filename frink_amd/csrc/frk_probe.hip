// Calibration kernels for the matrix-core GEMMs (not on any product path): how much vector-ALU issue time a
// v_mfma_i32_32x32x32_i8 takes away from the SIMD that runs it, and what the shader clock is while the matrix
// cores are busy.  The GEMM kernels' tile budgets are priced with these two figures.
//
// issue_probe_kernel<N>: every wavefront runs one chain of dependent MFMAs with N independent vector
// instructions behind each (v_and_b32, the cheapest kind), two wavefronts per SIMD as in the GEMM kernels.  The
// matrix core alone needs 32 clocks per MFMA; what the loop needs beyond that is issue time.  The first
// wavefront also reads the shader's cycle counter (s_memtime) and the constant 100 MHz counter (s_memrealtime)
// around its loop: their ratio is the shader clock under this load.
#include "frk_device.hpp"

namespace frk {

typedef int v4i_p __attribute__((ext_vector_type(4)));
typedef int v16i_p __attribute__((ext_vector_type(16)));

template <int N>
__global__ __launch_bounds__(512) void issue_probe_kernel(int iters, unsigned long long *clocks, int *sink) {
    v4i_p a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, 6, (int)blockIdx.x};
    v16i_p acc = {0};
    int x[8];
#pragma unroll
    for (int j = 0; j < 8; j++) x[j] = (int)threadIdx.x + j;
    const int m = (int)blockIdx.x | 1;
    unsigned long long c0, c1, r0, r1;
    asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(c0), "=s"(r0));
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
#pragma unroll
            for (int j = 0; j < N; j++) asm volatile("v_and_b32 %0, %0, %1" : "+v"(x[(j + u * N) & 7]) : "v"(m));
        }
    }
    asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(c1), "=s"(r1));
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clocks[0] = c1 - c0;
        clocks[1] = r1 - r0;
    }
    int s = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) s += x[j];
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[r];
    if (s == 0x7fffffff) sink[0] = s;  // (keeps the loop alive)
}

// One launch per N in {0, 4, 8, 12}: out[4 * k + 0] = shader cycles per MFMA and SIMD (the launch's duration at the
// clock measured in it), [1] = shader clock in MHz during the loop, [2] = microseconds of the launch (HIP events),
// [3] = the share of the launch the first wavefront's own loop took (the older wavefront of a SIMD is served first: at
// N = 0 it finishes in half the time, and its partner runs alone afterwards).  One workgroup of eight wavefronts per
// compute unit.
int launch_issue_probe(float *out, hipStream_t s) {
    int dev = 0, cus = 0;
    FRK_HIP_TRY(hipGetDevice(&dev));
    FRK_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    unsigned long long *clocks = nullptr;
    int *sink = nullptr;
    FRK_HIP_TRY(hipMalloc(&clocks, 16));
    FRK_HIP_TRY(hipMalloc(&sink, 64));
    hipEvent_t e0, e1;
    FRK_HIP_TRY(hipEventCreate(&e0));
    FRK_HIP_TRY(hipEventCreate(&e1));
    const int iters = 4000;
    int rc = FRK_OK;
    for (int k = 0; k < 4 && rc == FRK_OK; k++) {
        auto launch = [&]() {
            if (k == 0) hipLaunchKernelGGL(issue_probe_kernel<0>, dim3((unsigned)cus), dim3(512), 0, s, iters, clocks, sink);
            if (k == 1) hipLaunchKernelGGL(issue_probe_kernel<4>, dim3((unsigned)cus), dim3(512), 0, s, iters, clocks, sink);
            if (k == 2) hipLaunchKernelGGL(issue_probe_kernel<8>, dim3((unsigned)cus), dim3(512), 0, s, iters, clocks, sink);
            if (k == 3) hipLaunchKernelGGL(issue_probe_kernel<12>, dim3((unsigned)cus), dim3(512), 0, s, iters, clocks, sink);
        };
        launch();  // (warm: the clocks settle)
        launch();
        hipError_t e = hipEventRecord(e0, s);
        launch();
        if (e == hipSuccess) e = hipEventRecord(e1, s);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        float ms = 0.f;
        unsigned long long h[2] = {0, 0};
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e == hipSuccess) e = hipMemcpy(h, clocks, 16, hipMemcpyDeviceToHost);
        if (e != hipSuccess) {
            rc = set_error(FRK_ERR_HIP, "issue probe: %s", hipGetErrorString(e));
            break;
        }
        const double mfmas_per_simd = (double)iters * 8 * 2;  // two wavefronts per SIMD
        const double mhz = h[1] ? (double)h[0] / ((double)h[1] / 100.0) : 0.0;
        out[4 * k + 0] = (float)((double)ms * 1e3 * mhz / mfmas_per_simd);
        out[4 * k + 1] = (float)mhz;
        out[4 * k + 2] = ms * 1e3f;
        out[4 * k + 3] = ms > 0.f && mhz > 0. ? (float)((double)h[0] / mhz / ((double)ms * 1e3)) : 0.f;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(clocks);
    (void)hipFree(sink);
    return rc;
}

// read_shape_kernel: the bare fetch of a buffer in the shape the decode kernels use -- every wavefront owns one
// contiguous span of SPAN KB and issues all of its 16-byte loads before it waits for the first -- so that the
// shape's parameters can be priced one at a time: the span, the wavefronts per workgroup, whether the data lands
// in registers or is copied straight into LDS, and the cache policy bits of the load (POLICY 0 none, 1 nt,
// 2 sc1, 3 sc0 sc1).  Nothing is done with the data beyond what keeps the loads alive.
template <int POLICY>
__device__ __forceinline__ v4i_p load16_policy(const uint4 *p) {
    v4i_p v;
    if (POLICY == 0) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    if (POLICY == 1) asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(v) : "v"(p) : "memory");
    if (POLICY == 2) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    if (POLICY == 3) asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int POLICY>
__device__ __forceinline__ void dma16_policy(uint32_t lds_uniform, const uint4 *p) {
    const uint32_t m = __builtin_amdgcn_readfirstlane(lds_uniform);
    if (POLICY == 0) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m), "v"(p) : "memory");
    if (POLICY == 1) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" : : "s"(m), "v"(p) : "memory");
    if (POLICY == 2) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off sc1" : : "s"(m), "v"(p) : "memory");
    if (POLICY == 3) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off sc0 sc1" : : "s"(m), "v"(p) : "memory");
}

template <int SPAN, int POLICY, bool TO_LDS>
__global__ __launch_bounds__(1024) void read_shape_kernel(const uint4 *__restrict__ src, size_t spans, uint32_t *__restrict__ sink) {
    extern __shared__ uint4 landing[];  // TO_LDS: min(SPAN, 8) KB per wavefront
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const size_t span = (size_t)blockIdx.x * (blockDim.x >> 6) + wave;
    if (span >= spans) return;
    const uint4 *p = src + span * (SPAN * 64) + lane;
    uint32_t acc = 0;
    if (TO_LDS) {
        constexpr int ROOM = SPAN < 8 ? SPAN : 8;
        const uint32_t base = lds_address(landing) + wave * (ROOM * 1024);
#pragma unroll
        for (int i = 0; i < SPAN; i++) dma16_policy<POLICY>(base + (i % ROOM) * 1024, p + i * 64);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
        v4i_p v[SPAN];
#pragma unroll
        for (int i = 0; i < SPAN; i++) v[i] = load16_policy<POLICY>(p + i * 64);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < SPAN; i++) {
            asm volatile("" : "+v"(v[i]));  // (the values exist only after the wait above)
            acc ^= (uint32_t)(v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3]);
        }
        if (acc == 0x9e3779b9u) sink[(blockIdx.x * 64 + lane) & 16383] = acc;
    }
}

template <int SPAN, int POLICY>
static int launch_read_shape_sp(const void *src, size_t spans, void *sink, int waves, bool to_lds, hipStream_t s) {
    const unsigned grid = (unsigned)((spans + waves - 1) / waves);
    if (to_lds) {
        const size_t room = (size_t)waves * (SPAN < 8 ? SPAN : 8) * 1024;
        auto k = read_shape_kernel<SPAN, POLICY, true>;
        FRK_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)room));
        hipLaunchKernelGGL(k, dim3(grid), dim3(waves * 64), room, s, (const uint4 *)src, spans, (uint32_t *)sink);
    } else {
        hipLaunchKernelGGL((read_shape_kernel<SPAN, POLICY, false>), dim3(grid), dim3(waves * 64), 0, s, (const uint4 *)src, spans,
                           (uint32_t *)sink);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(FRK_ERR_HIP, "read shape launch: %s", hipGetErrorString(e));
    return FRK_OK;
}
template <int SPAN>
static int launch_read_shape_s(const void *src, size_t spans, void *sink, int waves, bool to_lds, int policy, hipStream_t s) {
    switch (policy) {
        case 0: return launch_read_shape_sp<SPAN, 0>(src, spans, sink, waves, to_lds, s);
        case 1: return launch_read_shape_sp<SPAN, 1>(src, spans, sink, waves, to_lds, s);
        case 2: return launch_read_shape_sp<SPAN, 2>(src, spans, sink, waves, to_lds, s);
        case 3: return launch_read_shape_sp<SPAN, 3>(src, spans, sink, waves, to_lds, s);
    }
    return set_error(FRK_ERR_ARG, "read shape: policy %d is not one of 0..3", policy);
}

// Reads floor(bytes / (span_kb KB)) spans of the buffer; span_kb in {2, 4, 9, 18}, waves (per workgroup) in 1..16.
int launch_read_shape(const void *src, size_t bytes, void *sink, int span_kb, int waves, int to_lds, int policy, hipStream_t s) {
    if (waves < 1 || waves > 16) return set_error(FRK_ERR_ARG, "read shape: %d wavefronts per workgroup", waves);
    const size_t spans = bytes / ((size_t)span_kb * 1024);
    if (spans == 0 || spans / waves >= 0x7fffffffu) return set_error(FRK_ERR_ARG, "read shape: %zu bytes", bytes);
    if (to_lds && (size_t)waves * (span_kb < 8 ? span_kb : 8) * 1024 > 160 * 1024)
        return set_error(FRK_ERR_ARG, "read shape: %d wavefronts of %d KB do not fit the LDS", waves, span_kb);
    switch (span_kb) {
        case 2: return launch_read_shape_s<2>(src, spans, sink, waves, to_lds != 0, policy, s);
        case 4: return launch_read_shape_s<4>(src, spans, sink, waves, to_lds != 0, policy, s);
        case 9: return launch_read_shape_s<9>(src, spans, sink, waves, to_lds != 0, policy, s);
        case 18: return launch_read_shape_s<18>(src, spans, sink, waves, to_lds != 0, policy, s);
    }
    return set_error(FRK_ERR_ARG, "read shape: span of %d KB is not one of 2, 4, 9, 18", span_kb);
}


}  // namespace frk
