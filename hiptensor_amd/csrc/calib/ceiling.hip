// Bench-only calibration library (libhiptk_calib.so, not part of the product library):
// the rate a loop of nothing but MFMA instructions sustains on every CU,
// with constant operands and with pseudo-random operands in [-1, 1).  Under a full MFMA load
// the clock this part holds depends on how much the operand bits toggle, so this is the
// practical ceiling the contraction kernels are measured against (next to the nominal peak).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <chrono>

#include "hiptk_calib.h"
#include "hiptk_kernels.h"

namespace
{
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    typedef float    f32x16_t __attribute__((ext_vector_type(16)));
    typedef double   f64x4_t __attribute__((ext_vector_type(4)));
    typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
    typedef __bf16   bf16x8_t __attribute__((ext_vector_type(8)));

    __device__ inline uint32_t hash32(uint32_t x)
    {
        uint32_t s = x * 747796405u + 2891336453u;
        uint32_t w = ((s >> ((s >> 28u) + 4u)) ^ s) * 277803737u;
        return (w >> 22u) ^ w;
    }
    __device__ inline float unit(uint32_t seed)
    {
        return ((float)hash32(seed) / 4294967296.0f - 0.5f) * 2.f;
    }

    // 16 independent 32x32 accumulators per wave, 8 operand sets cycled through
    template <int BF16>
    __global__ void __launch_bounds__(256) ceiling_h(float* sink, int iters, int random)
    {
        const uint32_t tid = threadIdx.x + blockIdx.x * 256u;
        f32x16_t       acc[16];
        for(int i = 0; i < 16; i++)
            for(int r = 0; r < 16; r++)
                acc[i][r] = 0.f;
        u32x4_t xf[8][4], yf[8][4];
        for(int s = 0; s < 8; s++)
            for(int i = 0; i < 4; i++)
                for(int e = 0; e < 4; e++)
                {
                    float v[4] = {1.f, 1.f, 1.f, 1.f};
                    if(random)
                        for(int q = 0; q < 4; q++)
                            v[q] = unit(tid * 1315423911u + (uint32_t)(((s * 4 + i) * 4 + e) * 4 + q));
                    uint16_t h[4];
                    for(int q = 0; q < 4; q++)
                        h[q] = BF16 ? (uint16_t)(__float_as_uint(v[q]) >> 16) : __builtin_bit_cast(uint16_t, (_Float16)v[q]);
                    xf[s][i][e] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
                    yf[s][i][e] = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
                }
        for(int it = 0; it < iters; it++)
#pragma unroll
            for(int s = 0; s < 8; s++)
#pragma unroll
                for(int i = 0; i < 4; i++)
#pragma unroll
                    for(int j = 0; j < 4; j++)
                    {
                        if(BF16)
                            acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                __builtin_bit_cast(bf16x8_t, xf[s][i]), __builtin_bit_cast(bf16x8_t, yf[s][j]), acc[i * 4 + j], 0, 0, 0);
                        else
                            acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                                __builtin_bit_cast(half8_t, xf[s][i]), __builtin_bit_cast(half8_t, yf[s][j]), acc[i * 4 + j], 0, 0, 0);
                    }
        float sum = 0;
        for(int i = 0; i < 16; i++)
            for(int r = 0; r < 16; r++)
                sum += acc[i][r];
        if(sum == 1.2345f)
            sink[threadIdx.x] = sum;
    }

    __global__ void __launch_bounds__(256) ceiling_f32(float* sink, int iters, int random)
    {
        const uint32_t tid = threadIdx.x + blockIdx.x * 256u;
        f32x16_t       acc[8];
        for(int i = 0; i < 8; i++)
            for(int r = 0; r < 16; r++)
                acc[i][r] = 0.f;
        float x[8], y[8];
        for(int s = 0; s < 8; s++)
        {
            x[s] = random ? unit(tid * 1315423911u + s) : 1.f;
            y[s] = random ? unit(tid * 2654435761u + s + 64) : 1.f;
        }
        for(int it = 0; it < iters; it++)
#pragma unroll
            for(int s = 0; s < 8; s++)
#pragma unroll
                for(int i = 0; i < 8; i++)
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(x[(s + i) & 7], y[s], acc[i], 0, 0, 0);
        float sum = 0;
        for(int i = 0; i < 8; i++)
            for(int r = 0; r < 16; r++)
                sum += acc[i][r];
        if(sum == 1.2345f)
            sink[threadIdx.x] = sum;
    }

    __global__ void __launch_bounds__(256) ceiling_f64(float* sink, int iters, int random)
    {
        const uint32_t tid = threadIdx.x + blockIdx.x * 256u;
        f64x4_t        acc[16];
        for(int i = 0; i < 16; i++)
            for(int r = 0; r < 4; r++)
                acc[i][r] = 0.0;
        double x[8], y[8];
        for(int s = 0; s < 8; s++)
        {
            x[s] = random ? (double)unit(tid * 1315423911u + s) + 1e-9 * unit(tid + 7u * s) : 1.0;
            y[s] = random ? (double)unit(tid * 2654435761u + s + 64) + 1e-9 * unit(tid + 11u * s) : 1.0;
        }
        for(int it = 0; it < iters; it++)
#pragma unroll
            for(int s = 0; s < 8; s++)
#pragma unroll
                for(int i = 0; i < 16; i++)
                    acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(x[(s + i) & 7], y[s], acc[i], 0, 0, 0);
        double sum = 0;
        for(int i = 0; i < 16; i++)
            for(int r = 0; r < 4; r++)
                sum += acc[i][r];
        if(sum == 1.2345)
            sink[threadIdx.x] = (float)sum;
    }
}

extern "C" int hiptk_mfma_ceiling(int cls, int random_operands, double* tflops)
{
    if(!tflops)
        return HIPTK_ERR_ARG;
    int             dev = 0;
    hipDeviceProp_t prop;
    if(hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
        return HIPTK_ERR_LAUNCH;
    const int grid = prop.multiProcessorCount; // one workgroup of 4 waves per CU
    float*    sink = nullptr;
    if(hipMalloc(&sink, 4096) != hipSuccess)
        return HIPTK_ERR_LAUNCH;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    double flops_per_iter = 0;
    int    iters          = 0;
    auto   launch         = [&]() {
        switch(cls)
        {
        case HIPTK_F16:
            iters          = 400;
            flops_per_iter = 128.0 * 32768;
            hipLaunchKernelGGL(ceiling_h<0>, dim3(grid), dim3(256), 0, 0, sink, iters, random_operands);
            break;
        case HIPTK_BF16:
            iters          = 400;
            flops_per_iter = 128.0 * 32768;
            hipLaunchKernelGGL(ceiling_h<1>, dim3(grid), dim3(256), 0, 0, sink, iters, random_operands);
            break;
        case HIPTK_F32:
        case HIPTK_C32:
            iters          = 800;
            flops_per_iter = 64.0 * 4096;
            hipLaunchKernelGGL(ceiling_f32, dim3(grid), dim3(256), 0, 0, sink, iters, random_operands);
            break;
        case HIPTK_F64:
        case HIPTK_C64:
            iters          = 300;
            flops_per_iter = 128.0 * 2048;
            hipLaunchKernelGGL(ceiling_f64, dim3(grid), dim3(256), 0, 0, sink, iters, random_operands);
            break;
        default: break;
        }
    };
    launch(); // sets iters
    if(iters == 0)
    {
        (void)hipFree(sink);
        return HIPTK_ERR_ARG;
    }
    (void)hipDeviceSynchronize();
    // the clock governor takes tens of milliseconds of load to settle: run untimed for ~150 ms
    const auto t0 = std::chrono::steady_clock::now();
    while(std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < 0.15)
    {
        for(int r = 0; r < 10; r++)
            launch();
        (void)hipDeviceSynchronize();
    }
    const int reps = 20;
    (void)hipEventRecord(e0, 0);
    for(int r = 0; r < reps; r++)
        launch();
    (void)hipEventRecord(e1, 0);
    (void)hipEventSynchronize(e1);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if(hipGetLastError() != hipSuccess || ms <= 0.f)
        return HIPTK_ERR_LAUNCH;
    *tflops = flops_per_iter * iters * 4.0 * grid * reps / (ms * 1e-3) / 1e12;
    return HIPTK_OK;
}
