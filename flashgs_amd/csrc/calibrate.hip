// Microbenchmarks that measure what this GPU attains on the three resources the rasterizer's
// rooflines are priced against: streaming memory traffic, fp32 FMA issue and exp2 issue.  Built
// into its own small library (libflashgs_calibrate.so): measurement aid, not part of the
// rasterizer.  Every function runs on `stream`, times its kernel with HIP events and returns the
// result through `out`; return value 0 or a hipError_t code.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, size_t n)
{
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (; i < n; i += stride) dst[i] = src[i];
}

__global__ __launch_bounds__(kThreads) void read_kernel(const float4* __restrict__ src, float* __restrict__ sink, size_t n)
{
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * kThreads;
    float acc = 0.f;
    for (; i < n; i += stride) {
        const float4 v = src[i];
        acc += v.x + v.y + v.z + v.w;
    }
    if (acc == 12345.678f) *sink = acc;      // never true for the fill value; keeps the loads alive
}

// kChains independent dependency chains per lane, each `iters` long.
// kExpEvery = 0: FMA only; k > 0: one exp2 after every k FMAs of a chain.
template <int kExpEvery>
__global__ __launch_bounds__(kThreads) void alu_kernel(float* __restrict__ sink, int iters, float a, float b)
{
    constexpr int kChains = 8;
    float x[kChains];
#pragma unroll
    for (int c = 0; c < kChains; c++) x[c] = (float)threadIdx.x * 1e-3f + (float)c;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int c = 0; c < kChains; c++) {
            if (kExpEvery < 0) {
                x[c] = __builtin_amdgcn_exp2f(x[c]) - 1.0f;          // exp2 only (the subtraction keeps it bounded)
            } else {
#pragma unroll
                for (int k = 0; k < (kExpEvery > 0 ? kExpEvery : 4); k++) x[c] = __builtin_fmaf(x[c], a, b);
                if (kExpEvery > 0) x[c] = __builtin_amdgcn_exp2f(x[c]);
            }
        }
    }
    float r = 0.f;
#pragma unroll
    for (int c = 0; c < kChains; c++) r += x[c];
    if (r == 12345.678f) *sink = r;
}

template <typename Launch>
int timed(hipStream_t st, int reps, double* ms, Launch launch)
{
    hipEvent_t e0, e1;
    hipError_t rc = hipEventCreate(&e0);
    if (rc != hipSuccess) return (int)rc;
    rc = hipEventCreate(&e1);
    if (rc != hipSuccess) return (int)rc;
    launch();                                   // warm-up
    (void)hipEventRecord(e0, st);
    for (int r = 0; r < reps; r++) launch();
    (void)hipEventRecord(e1, st);
    rc = hipEventSynchronize(e1);
    float t = 0.f;
    if (rc == hipSuccess) rc = hipEventElapsedTime(&t, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc == hipSuccess) rc = hipGetLastError();
    *ms = (double)t / reps;
    return (int)rc;
}

} // namespace

// Bytes per second moved by a device-to-device copy of `bytes` bytes (read + write counted).
extern "C" int fgs_cal_copy(const void* src, void* dst, size_t bytes, double* bytes_per_s, void* stream)
{
    hipStream_t st = (hipStream_t)stream;
    const size_t n = bytes / sizeof(float4);
    double ms = 0;
    const int rc = timed(st, 10, &ms, [&] {
        hipLaunchKernelGGL(copy_kernel, dim3(256 * 32), dim3(kThreads), 0, st, (const float4*)src, (float4*)dst, n);
    });
    *bytes_per_s = 2.0 * (double)(n * sizeof(float4)) / (ms * 1e-3);
    return rc;
}

// Bytes per second read by a streaming reduction over `bytes` bytes.
extern "C" int fgs_cal_read(const void* src, float* sink, size_t bytes, double* bytes_per_s, void* stream)
{
    hipStream_t st = (hipStream_t)stream;
    const size_t n = bytes / sizeof(float4);
    double ms = 0;
    const int rc = timed(st, 10, &ms, [&] {
        hipLaunchKernelGGL(read_kernel, dim3(256 * 32), dim3(kThreads), 0, st, (const float4*)src, sink, n);
    });
    *bytes_per_s = (double)(n * sizeof(float4)) / (ms * 1e-3);
    return rc;
}

// Wave64 instructions per second, summed over the chip: mode 0 = v_fma_f32 only, mode 1 = one
// v_exp_f32 after every four FMAs (reports FMA + exp instructions), mode 2 = the same after every
// eight, mode 3 = v_exp_f32 + one subtraction only (reports exp instructions only).
extern "C" int fgs_cal_alu(int mode, float* sink, double* lane_ops_per_s, void* stream)
{
    hipStream_t st = (hipStream_t)stream;
    const int iters = 2048, blocks = 256 * 8 * 4;          // 8 waves per SIMD on 256 CUs, 4 rounds
    double ms = 0;
    int rc;
    double per_chain_iter;
    if (mode == 0) {
        rc = timed(st, 3, &ms, [&] { hipLaunchKernelGGL(alu_kernel<0>, dim3(blocks), dim3(kThreads), 0, st, sink, iters, 0.999f, 0.001f); });
        per_chain_iter = 4;
    } else if (mode == 1) {
        rc = timed(st, 3, &ms, [&] { hipLaunchKernelGGL(alu_kernel<4>, dim3(blocks), dim3(kThreads), 0, st, sink, iters, 0.5f, -1.0f); });
        per_chain_iter = 5;
    } else if (mode == 2) {
        rc = timed(st, 3, &ms, [&] { hipLaunchKernelGGL(alu_kernel<8>, dim3(blocks), dim3(kThreads), 0, st, sink, iters, 0.5f, -1.0f); });
        per_chain_iter = 9;
    } else {
        rc = timed(st, 3, &ms, [&] { hipLaunchKernelGGL(alu_kernel<-1>, dim3(blocks), dim3(kThreads), 0, st, sink, iters, 0.f, 0.f); });
        per_chain_iter = 1;
    }
    const double lane_ops = (double)blocks * kThreads * 8.0 * iters * per_chain_iter;
    *lane_ops_per_s = lane_ops / (ms * 1e-3);
    return rc;
}
