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

}  // namespace frk
