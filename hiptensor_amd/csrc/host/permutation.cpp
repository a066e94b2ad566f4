// hiptensorPermutation: B[perm(index)] = opB(alpha * opA(A[index])).
//
// Argument checks, their order, status codes and messages follow the reference,
// library/src/permutation/hiptensor_permutation.cpp:44-279.  Below the checks the reference
// walks a registry of Composable Kernel element-wise instances until one accepts the problem;
// here the problem is fused and mapped to one of four memory-bound kernels
// (permute_plan.cpp) and launched once on the caller's stream.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include <hip/hip_runtime_api.h>

#include <hiptensor/hiptensor.hpp>

#include "handle.hpp"
#include "logger.hpp"
#include "permute_plan.hpp"

using hipta::Handle;
using hipta::Logger;

namespace
{
    float halfToFloat(uint16_t h)
    {
        const int   sign = (h >> 15) & 1, exp = (h >> 10) & 0x1F, man = h & 0x3FF;
        float       v;
        if(exp == 0)
            v = std::ldexp((float)man, -24);
        else if(exp == 31)
            v = man ? std::nanf("") : INFINITY;
        else
            v = std::ldexp((float)(man | 0x400), exp - 25);
        return sign ? -v : v;
    }

    // HIPTENSOR_AMD_PERMUTE="kernel[,tile[,maxvec[,group]]]": kernel is auto | gather | tiled |
    // rows | strip | grouped (tiled and rows name the same preference: whichever of the two the
    // layout admits; strip and grouped - which includes the shared-fastest-mode tiles - are
    // taken wherever the layout admits them),
    // tile is 0..2 or -1, maxvec caps the vector width, group sets the band width of the
    // workgroup order.  For tests and experiments.
    hipta::PermuteTuning tuningFromEnv()
    {
        hipta::PermuteTuning t;
        const char*          e = std::getenv("HIPTENSOR_AMD_PERMUTE");
        if(!e || !*e)
            return t;
        char buf[64];
        std::snprintf(buf, sizeof(buf), "%s", e);
        char* save = nullptr;
        char* tok  = strtok_r(buf, ",", &save);
        if(tok)
        {
            if(!std::strcmp(tok, "gather"))
                t.kernel = HIPTK_PERM_GATHER;
            else if(!std::strcmp(tok, "tiled") || !std::strcmp(tok, "rows"))
                t.kernel = HIPTK_PERM_TILED;
            else if(!std::strcmp(tok, "strip"))
                t.kernel = HIPTK_PERM_STRIP;
            else if(!std::strcmp(tok, "grouped"))
                t.kernel = HIPTK_PERM_GROUPED;
            tok = strtok_r(nullptr, ",", &save);
        }
        if(tok)
        {
            t.tile = std::atoi(tok);
            tok    = strtok_r(nullptr, ",", &save);
        }
        if(tok)
        {
            t.max_vec = std::atoi(tok);
            tok       = strtok_r(nullptr, ",", &save);
        }
        if(tok)
            t.group = std::atoi(tok);
        return t;
    }
}

namespace hipta
{
    // What hiptensorPermutation would launch for these descriptors and addresses; no device
    // needed.  Returns the status the call itself would return before launching.
    hiptensorStatus_t planPermutation(const hiptensorTensorDescriptor_t* descA,
                                      const int32_t                      modeA[],
                                      const hiptensorTensorDescriptor_t* descB,
                                      const int32_t                      modeB[],
                                      const void*                        A,
                                      const void*                        B,
                                      hiptk_permute_t&                   out,
                                      bool&                              empty)
    {
        empty          = false;
        const int rank = (int)descA->mLengths.size();
        PermuteIn in;
        in.elem_bytes = descA->mType == HIP_R_16F ? 2 : 4;
        in.lenA.assign(descA->mLengths.begin(), descA->mLengths.end());
        in.lenB.assign(descB->mLengths.begin(), descB->mLengths.end());
        in.modeA.assign(modeA, modeA + rank);
        in.modeB.assign(modeB, modeB + descB->mLengths.size());
        in.A = A;
        in.B = B;
        switch(plan_permutation(in, tuningFromEnv(), out))
        {
        case PermuteStatus::OK: break;
        case PermuteStatus::EMPTY: empty = true; break;
        case PermuteStatus::TOO_LARGE: return HIPTENSOR_STATUS_NOT_SUPPORTED;
        default: return HIPTENSOR_STATUS_INVALID_VALUE;
        }
        out.op_a = descA->mUnaryOp == HIPTENSOR_OP_SQRT ? 1 : 0;
        out.op_b = descB->mUnaryOp == HIPTENSOR_OP_SQRT ? 1 : 0;
        return HIPTENSOR_STATUS_SUCCESS;
    }
}

hiptensorStatus_t hiptensorPermutation(const hiptensorHandle_t*           handle,
                                       const void*                        alpha,
                                       const void*                        A,
                                       const hiptensorTensorDescriptor_t* descA,
                                       const int32_t                      modeA[],
                                       void*                              B,
                                       const hiptensorTensorDescriptor_t* descB,
                                       const int32_t                      modeB[],
                                       const hipDataType                  typeScalar,
                                       const hipStream_t                  stream)
{
    Logger&     log = Logger::get();
    const char* fn  = "hiptensorPermutation";
    log.apif(fn,
             "handle=%p, alpha=%p, A=%p, descA=%p, modeA=%p, B=%p, descB=%p, modeB=%p, "
             "typeScalar=0x%02X, stream=%p",
             (const void*)handle,
             alpha,
             A,
             (const void*)descA,
             (const void*)modeA,
             B,
             (const void*)descB,
             (const void*)modeB,
             (unsigned)typeScalar,
             (void*)stream);

    if(!handle || !alpha || !A || !descA || !modeA || !B || !descB || !modeB)
    {
        const struct
        {
            const void* p;
            const char* name;
        } params[] = {{handle, "handle"}, {alpha, "alpha"}, {A, "A"}, {descA, "descA"}, {modeA, "modeA"}, {B, "B"}, {descB, "descB"}, {modeB, "modeB"}};
        for(const auto& q : params)
            if(!q.p)
                log.errorf(fn, "Initialization Error : %s = nullptr (%s)", q.name, hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    if(descA->mType != HIP_R_16F && descA->mType != HIP_R_32F)
    {
        log.errorf(fn,
                   "Unsupported Data Type Error : The supported data types of A and B are HIP_R_16F and HIP_R_32F (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_SUPPORTED));
        return HIPTENSOR_STATUS_NOT_SUPPORTED;
    }
    if(descA->mType != descB->mType)
    {
        log.errorf(fn,
                   "Mismatched Data Type Error : Data types of A and B are not the same. (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    if(typeScalar != HIP_R_16F && typeScalar != HIP_R_32F)
    {
        log.errorf(fn,
                   "Unsupported Data Type Error : The supported data types of alpha are HIP_R_16F and HIP_R_32F (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_SUPPORTED));
        return HIPTENSOR_STATUS_NOT_SUPPORTED;
    }
    // The reference registers instances for ranks 2..6 only and reports any other rank as
    // "No Kernels Found" (hiptensor_permutation.cpp:173-189,
    // permutation_solution_rank2..6_instances.cpp).
    const size_t rank = descA->mLengths.size();
    if(rank < 2 || rank > 6)
    {
        log.errorf(fn, "Internal Error : No Kernels Found (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
    Handle* h = Handle::from(handle->fields);
    if(!h)
        return HIPTENSOR_STATUS_NOT_INITIALIZED;

    hiptk_permute_t prob;
    bool            empty = false;
    if(auto st = hipta::planPermutation(descA, modeA, descB, modeB, A, B, prob, empty); st != HIPTENSOR_STATUS_SUCCESS)
    {
        if(st == HIPTENSOR_STATUS_NOT_SUPPORTED)
            log.errorf(fn, "Tensors of 2^31 elements or more are not supported (%s)", hiptensorGetErrorString(st));
        else
            log.errorf(fn,
                       "Input Parameter Error : modeB is not a reordering of modeA, or the lengths of A and B disagree (%s)",
                       hiptensorGetErrorString(st));
        return st;
    }
    if(h->hostOnly())
    {
        log.errorf(fn, "This handle has no device; it cannot execute (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_ARCH_MISMATCH));
        return HIPTENSOR_STATUS_ARCH_MISMATCH;
    }
    int cur = -1;
    if(hipGetDevice(&cur) != hipSuccess || cur != h->device())
    {
        log.errorf(fn,
                   "Device mismatch error: current device id: %d, handle device id: %d (%s)",
                   cur,
                   h->device(),
                   hiptensorGetErrorString(HIPTENSOR_STATUS_ARCH_MISMATCH));
        return HIPTENSOR_STATUS_ARCH_MISMATCH;
    }
    if(empty)
        return HIPTENSOR_STATUS_SUCCESS;

    // alpha is read as typeScalar and widened to float (permutation_solution_impl.hpp:108-113)
    prob.alpha = typeScalar == HIP_R_16F ? halfToFloat(*(const uint16_t*)alpha) : *(const float*)alpha;

    bool       timed = (log.mask() & HIPTENSOR_LOG_LEVEL_PERF_TRACE) != 0;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if(timed)
    {
        // timing synchronises with the stream, which would invalidate a capture in progress: the
        // call is then enqueued untimed (no PERF_TRACE line)
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if(hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone)
            timed = false;
    }
    if(timed)
    {
        if(hipEventCreate(&e0) != hipSuccess)
            return HIPTENSOR_STATUS_HIP_ERROR;
        if(hipEventCreate(&e1) != hipSuccess)
        {
            (void)hipEventDestroy(e0);
            return HIPTENSOR_STATUS_HIP_ERROR;
        }
        (void)hipEventRecord(e0, stream);
    }
    int hipErr = 0;
    int rc     = hiptk_permute(&prob, A, B, (void*)stream, &hipErr);
    if(timed)
    {
        (void)hipEventRecord(e1, stream);
        (void)hipEventSynchronize(e1);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, e0, e1);
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        if(rc == HIPTK_OK)
        {
            // Same line as the reference (hiptensor_permutation.cpp:243-251).  Its figures are
            // derived from the rank (flops = 2 * rank, bytes = rank * element sizes); here they
            // describe the work: one multiply per element, every element read and written once.
            double n = 1.0;
            for(size_t i = 0; i < rank; ++i)
                n *= (double)descA->mLengths[i];
            const char* name = hiptk_permute_kernel_name(&prob);
            uint64_t    uid  = 1469598103934665603ull;
            for(const char* c = name; *c; ++c)
                uid = (uid ^ (unsigned char)*c) * 1099511628211ull;
            char msg[512];
            snprintf(msg,
                     sizeof(msg),
                     "KernelId: %lu KernelName: %s, %0.3f ms, %0.3f TFlops, %0.3f GB/s",
                     (unsigned long)uid,
                     name,
                     ms,
                     n / 1e9 / ms,
                     2.0 * n * prob.elem_bytes / 1e6 / ms);
            log.perf(fn, msg);
        }
    }
    switch(rc)
    {
    case HIPTK_OK: return HIPTENSOR_STATUS_SUCCESS;
    case HIPTK_ERR_LAUNCH:
        log.errorf(fn, "Kernel launch failed: %s (%s)", hipGetErrorString((hipError_t)hipErr), hiptensorGetErrorString(HIPTENSOR_STATUS_EXECUTION_FAILED));
        return HIPTENSOR_STATUS_EXECUTION_FAILED;
    default:
        log.errorf(fn, "Selected kernel is unable to solve the problem (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
}
