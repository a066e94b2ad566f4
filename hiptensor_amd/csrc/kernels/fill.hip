// Fills device memory with finite pseudo-random elements of a kernel class's storage type.
// The measured kernel selection (DEFAULT_PATIENT) times its candidates on such data: the clock
// this device sustains under a matrix-core load depends on the operand values, so timing on
// zeros would rank the wrong kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "hiptk_kernels.h"

namespace
{
    __device__ inline uint32_t hash32(uint32_t x)
    {
        uint32_t s = x * 747796405u + 2891336453u;
        uint32_t w = ((s >> ((s >> 28u) + 4u)) ^ s) * 277803737u;
        return (w >> 22u) ^ w;
    }
}

namespace
{
    // Pseudo-random finite values of magnitude [0.5, 1) with random signs, written as 32-bit
    // words laid out for the class's element type.
    __global__ void __launch_bounds__(256) fill_pattern(uint32_t* out, size_t words, int cls)
    {
        const size_t stride = (size_t)gridDim.x * 256;
        for(size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += stride)
        {
            const uint32_t r = hash32((uint32_t)i * 2654435761u + (uint32_t)(i >> 32));
            uint32_t       w;
            switch(cls)
            {
            case HIPTK_F16: w = 0x38003800u | (r & 0x83FF83FFu); break;
            case HIPTK_BF16: w = 0x3F003F00u | (r & 0x807F807Fu); break;
            case HIPTK_F64:
            case HIPTK_C64:
            case HIPTK_F64_AS_F32: w = (i & 1) ? (0x3FE00000u | (r & 0x800FFFFFu)) : r; break;
            default: w = 0x3F000000u | (r & 0x807FFFFFu); break;
            }
            out[i] = w;
        }
    }
}

extern "C" int hiptk_fill_pattern(void* dst, uint64_t bytes, int cls, void* stream)
{
    if(!dst || (bytes & 3))
        return HIPTK_ERR_ARG;
    const size_t words = (size_t)(bytes / 4);
    if(words == 0)
        return HIPTK_OK;
    const unsigned blocks = (unsigned)std::min<size_t>((words + 255) / 256, 4096);
    hipLaunchKernelGGL(fill_pattern, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t*)dst, words, cls);
    return hipGetLastError() == hipSuccess ? HIPTK_OK : HIPTK_ERR_LAUNCH;
}
