// mg_probe_mfma: what the matrix cores of this chip sustain with no memory traffic at all.
//
// The MFMA rate of MI355X under load is set by the power-managed clock, and the clock by the
// operand bits: the same register-only loop runs near the 2.4 GHz boost clock on all-zero
// operands and several hundred MHz lower on random ones.  GEMM throughput on real data has to
// be read against the second figure, so the library can measure it: every SIMD of every CU runs
// two wavefronts of back-to-back v_mfma_f32_32x32x16 on eight independent accumulators, from
// registers only; device time comes from HIP events, the clock from the shader clock counter
// against the constant 100 MHz counter.  (The reference's counterpart is the hand-written peak
// probe it prices its kernels against, bench/RESULTS.md:113-119.)
#include <hip/hip_runtime.h>

#include "ew_common.h"
#include "gemm_kernel.h"

namespace mg {

template <int DT>
__global__ void __launch_bounds__(512) k_probe_mfma(int iters, uint32_t seed, int random_operands,
                                                   unsigned long long *clocks, float *sink) {
    const int lane = threadIdx.x & 63;
    u32x4 a[4], b[2];
    uint32_t x = seed ^ (blockIdx.x * 2654435761u) ^ (threadIdx.x * 40503u);
    auto next = [&]() {
        x = x * 1664525u + 1013904223u;
        // two 16-bit values in (-2, 2): sign, exponent 126 / 127 (f16: 14 / 15), random mantissa
        const uint32_t hi = DT == D_F16 ? (0x3800u | (x >> 18 & 0x87ffu)) : (0x3f00u | (x >> 17 & 0x80ffu));
        const uint32_t lo = DT == D_F16 ? (0x3800u | (x >> 2 & 0x87ffu)) : (0x3f00u | (x >> 1 & 0x80ffu));
        return random_operands ? (hi << 16 | lo) : 0u;
    };
#pragma unroll
    for (int i = 0; i < 4; i++) a[i] = u32x4{next(), next(), next(), next()};
#pragma unroll
    for (int j = 0; j < 2; j++) b[j] = u32x4{next(), next(), next(), next()};
    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    const unsigned long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = mfma32<DT>(a[i], b[j], acc[i][j]);
    }
    const unsigned long long c1 = clock64(), w1 = wall_clock64();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) s += acc[i][j][lane & 15];
    if (s == 12345.678f) sink[0] = s;   // keeps the loop alive
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clocks[0] = c1 - c0;
        clocks[1] = w1 - w0;
    }
}

// mg_probe_stream: what a launch shaped like the skinny-M stream can read from, or write to, HBM
// when it does nothing else - four wavefronts to a workgroup, every wavefront one contiguous
// 24 KB span (16 rows of 768 16-bit elements) with all 24 loads (or stores) of a lane issued
// before anything is used.  The floor under the 1 x N x 768 forward GEMM.
__global__ void __launch_bounds__(256) k_probe_read(const uint4 *src, int64_t n16, unsigned *sink) {
    const int lane = threadIdx.x & 63;
    const int64_t span = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 1536;   // 16-byte pieces per wavefront
    uint4 v[24];
#pragma unroll
    for (int i = 0; i < 24; i++) {
        const int64_t at = span + i * 64 + lane;
        v[i] = at < n16 ? src[at] : uint4{0u, 0u, 0u, 0u};
    }
    unsigned acc = 0;
#pragma unroll
    for (int i = 0; i < 24; i++) acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    if (acc == 0x9e3779b9u) *sink = acc;   // never true for the fill pattern: keeps the loads alive
}
__global__ void __launch_bounds__(256) k_probe_fill(uint4 *dst, int64_t n16, unsigned value) {
    const int lane = threadIdx.x & 63;
    const int64_t span = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 1536;
#pragma unroll
    for (int i = 0; i < 24; i++) {
        const int64_t at = span + i * 64 + lane;
        if (at < n16) dst[at] = uint4{value, value + 1, value + 2, value + 3};
    }
}

}  // namespace mg

using namespace mg;

extern "C" int mg_probe_stream(mg_ctx *ctx, int64_t nbytes, int nsets, int repeat, double *read_us, double *fill_us) {
    EW_PRECHECK("mg_probe_stream", nbytes >= 16 && nbytes <= ((int64_t)1 << 32) && nsets >= 1 && nsets <= 64 &&
                                       repeat >= 1 && repeat <= 100000 && read_us && fill_us);
    hipStream_t stream = ctx_stream(ctx);
    const int64_t n16 = nbytes / 16;
    const unsigned wgs = (unsigned)((n16 + 4 * 1536 - 1) / (4 * 1536));
    uint4 *buf[64] = {nullptr};
    unsigned *sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipMalloc((void **)&sink, 64);
    for (int i = 0; i < nsets && e == hipSuccess; i++) e = hipMalloc((void **)&buf[i], (size_t)n16 * 16);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    float ms_read = 0.f, ms_fill = 0.f;
    if (e == hipSuccess) {
        // enough rotating buffers make every launch find its bytes in HBM, not in the last-level cache
        for (int i = 0; i < nsets; i++) hipLaunchKernelGGL(k_probe_fill, dim3(wgs), dim3(256), 0, stream, buf[i], n16, 7u * i);
        e = hipEventRecord(e0, stream);
        for (int r = 0; r < repeat; r++)
            hipLaunchKernelGGL(k_probe_read, dim3(wgs), dim3(256), 0, stream, buf[r % nsets], n16, sink);
        if (e == hipSuccess) e = hipEventRecord(e1, stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms_read, e0, e1);
        if (e == hipSuccess) e = hipEventRecord(e0, stream);
        for (int r = 0; r < repeat; r++)
            hipLaunchKernelGGL(k_probe_fill, dim3(wgs), dim3(256), 0, stream, buf[r % nsets], n16, (unsigned)r);
        if (e == hipSuccess) e = hipEventRecord(e1, stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms_fill, e0, e1);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    for (int i = 0; i < nsets; i++)
        if (buf[i]) (void)hipFree(buf[i]);
    if (sink) (void)hipFree(sink);
    if (e != hipSuccess) return ctx_hip_fail(e, "mg_probe_stream");
    *read_us = (double)ms_read * 1e3 / repeat;
    *fill_us = (double)ms_fill * 1e3 / repeat;
    return MG_OK;
}

extern "C" int mg_probe_mfma(mg_ctx *ctx, int dtype, int random_operands, int iters, int workgroups, double *tflops,
                             double *ghz) {
    EW_PRECHECK("mg_probe_mfma", dtype_ok(dtype) && iters > 0 && iters <= (1 << 24) && workgroups >= 0 && tflops && ghz);
    hipStream_t stream = ctx_stream(ctx);
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    unsigned long long *clocks = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (e == hipSuccess) e = hipMalloc((void **)&clocks, 64);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    float ms = 0.f;
    unsigned long long h[2] = {0, 0};
    if (e == hipSuccess) {
        auto kern = dtype == MG_F16 ? k_probe_mfma<D_F16> : k_probe_mfma<D_BF16>;
        float *sink = reinterpret_cast<float *>(clocks + 4);
        // one workgroup of eight wavefronts per CU (two per SIMD), on all CUs or on the first
        // `workgroups` the dispatcher picks; a short untimed launch first
        if (workgroups > 0 && workgroups < cus) cus = workgroups;
        hipLaunchKernelGGL(kern, dim3(cus), dim3(512), 0, stream, iters / 8 + 1, 1u, random_operands, clocks, sink);
        e = hipEventRecord(e0, stream);
        hipLaunchKernelGGL(kern, dim3(cus), dim3(512), 0, stream, iters, 2u, random_operands, clocks, sink);
        if (e == hipSuccess) e = hipEventRecord(e1, stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e == hipSuccess) e = hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (clocks) (void)hipFree(clocks);
    if (e != hipSuccess) return ctx_hip_fail(e, "mg_probe_mfma");
    const double flop = (double)cus * 8.0 * (double)iters * 8.0 * 32768.0;   // wavefronts x iterations x MFMAs x FLOP
    *tflops = flop / ((double)ms * 1e-3) / 1e12;
    *ghz = h[1] ? (double)h[0] / ((double)h[1] * 10.0) : 0.0;               // shader clocks per 10 ns tick
    return MG_OK;
}
