// Public hipTensor-compatible entry points of the contraction path.
//
// Argument checks, their order and the status codes follow the reference:
//   library/src/hiptensor.cpp:35-321 (create / destroy / tensor descriptor / error
//   string / alignment) and library/src/contraction/hiptensor_contraction.cpp:71-855
//   (contraction descriptor, find, workspace size, plan, execute).
// What differs is below the checks: planning folds the problem once and caches
// everything the execute call needs, and execution is a single kernel launch (plus
// one reduction launch under split-K) on the caller's stream.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <sstream>

#include <hip/hip_runtime_api.h>
#include <hip/hip_version.h>

#include <hiptensor/hiptensor.hpp>

#include "handle.hpp"
#include "logger.hpp"
#include "planner.hpp"
#include "solution.hpp"

using hipta::Handle;
using hipta::Logger;
using hipta::PlanState;

namespace
{
    constexpr hipDataType NONE_TYPE = (hipDataType)31; // placeholder type of the absent C tensor

    enum OpId : int32_t
    {
        OP_SCALE            = 0,
        OP_BILINEAR         = 1,
        OP_SCALE_COMPLEX    = 2,
        OP_BILINEAR_COMPLEX = 3
    };

    uint32_t elemSize(hipDataType t)
    {
        switch(t)
        {
        case HIP_R_16F:
        case HIP_R_16BF: return 2;
        case HIP_R_32F: return 4;
        case HIP_R_64F:
        case HIP_C_32F: return 8;
        case HIP_C_64F: return 16;
        default: return 0;
        }
    }

    float halfBitsToFloat(uint16_t h)
    {
        const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
        uint32_t       exp  = (h >> 10) & 0x1Fu;
        uint32_t       man  = h & 0x3FFu;
        uint32_t       bits;
        if(exp == 0)
        {
            if(man == 0)
                bits = sign;
            else
            {
                int e = -1;
                do
                {
                    man <<= 1;
                    e++;
                } while(!(man & 0x400u));
                bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
            }
        }
        else if(exp == 31)
            bits = sign | 0x7F800000u | (man << 13);
        else
            bits = sign | ((exp + 112u) << 23) | (man << 13);
        float f;
        std::memcpy(&f, &bits, 4);
        return f;
    }

    // Reads alpha / beta as the plan's compute type (reference: readVal<ScalarData>,
    // library/src/data_types.cpp:153-204) into (re, im) doubles.
    bool readScalar(const void* p, int compute, double out[2])
    {
        out[0] = out[1] = 0.0;
        if(!p)
            return false;
        switch(compute)
        {
        case HIPTENSOR_COMPUTE_16F: out[0] = halfBitsToFloat(*(const uint16_t*)p); return true;
        case HIPTENSOR_COMPUTE_16BF:
        {
            uint32_t b = (uint32_t)(*(const uint16_t*)p) << 16;
            float    f;
            std::memcpy(&f, &b, 4);
            out[0] = f;
            return true;
        }
        case HIPTENSOR_COMPUTE_32F: out[0] = *(const float*)p; return true;
        case HIPTENSOR_COMPUTE_64F: out[0] = *(const double*)p; return true;
        case HIPTENSOR_COMPUTE_C32F:
            out[0] = ((const float*)p)[0];
            out[1] = ((const float*)p)[1];
            return true;
        case HIPTENSOR_COMPUTE_C64F:
            out[0] = ((const double*)p)[0];
            out[1] = ((const double*)p)[1];
            return true;
        default: return false;
        }
    }

    // Packs (re, im) into the scalar layout the kernel layer expects for a class.
    void packScalar(int cls, const double v[2], unsigned char out[16])
    {
        switch(cls)
        {
        case HIPTK_C32:
        {
            float f[2] = {(float)v[0], (float)v[1]};
            std::memcpy(out, f, 8);
            break;
        }
        case HIPTK_C64: std::memcpy(out, v, 16); break;
        case HIPTK_F64:
        case HIPTK_F64_AS_F32: std::memcpy(out, v, 8); break;
        default:
        {
            float f = (float)v[0];
            std::memcpy(out, &f, 4);
            break;
        }
        }
    }

    hipta::ProblemIn problemFromDesc(const hiptensorContractionDescriptor_t& d)
    {
        hipta::ProblemIn in;
        in.bilinear = d.mContractionOpId == OP_BILINEAR || d.mContractionOpId == OP_BILINEAR_COMPLEX;
        in.compute  = (int)d.mComputeType;
        auto fill   = [](hipta::TensorIn& t, const hiptensorTensorDescriptor_t& td, const std::vector<int32_t>& modes, uint32_t align) {
            t.dtype = (int)td.mType;
            t.len.assign(td.mLengths.begin(), td.mLengths.end());
            t.stride.assign(td.mStrides.begin(), td.mStrides.end());
            t.mode  = modes;
            t.align = align;
        };
        // The mode list at index 2 serves both C and D (the reference passes
        // mTensorMode[2] for both, hiptensor_contraction.cpp:397, 545, 772).
        fill(in.A, d.mTensorDesc[0], d.mTensorMode[0], d.mAlignmentReq[0]);
        fill(in.B, d.mTensorDesc[1], d.mTensorMode[1], d.mAlignmentReq[1]);
        fill(in.D, d.mTensorDesc[3], d.mTensorMode[2], d.mAlignmentReq[3]);
        if(in.bilinear)
            fill(in.C, d.mTensorDesc[2], d.mTensorMode[2], d.mAlignmentReq[2]);
        else
            in.C.dtype = -1;
        return in;
    }

    bool descWellFormed(const hiptensorContractionDescriptor_t* d)
    {
        return d->mTensorDesc.size() == 4 && d->mAlignmentReq.size() == 4 && d->mTensorMode.size() >= 3;
    }

    // Key of a planning request.  `ws` is the workspace size as it bounds the plan: sizes beyond
    // what planning can ever use are one request.
    std::string planKey(const hipta::ProblemIn& in, int algo, uint64_t ws)
    {
        std::ostringstream os;
        os << in.bilinear << '|' << in.compute << '|' << algo << '|' << ws;
        for(const hipta::TensorIn* t : {&in.A, &in.B, &in.C, &in.D})
        {
            os << "|t" << t->dtype << ',' << t->align;
            for(size_t i = 0; i < t->len.size(); i++)
                os << ';' << t->len[i] << ',' << t->stride[i] << ',' << t->mode[i];
        }
        return os.str();
    }

    hiptensorStatus_t checkDevice(const Handle* h, const char* func)
    {
        if(h->hostOnly())
            return HIPTENSOR_STATUS_SUCCESS;
        int cur = -1;
        if(hipGetDevice(&cur) != hipSuccess || cur != h->device())
        {
            Logger::get().errorf(func,
                                 "Device mismatch error: current device id: %d, handle device id: %d (%s)",
                                 cur,
                                 h->device(),
                                 hiptensorGetErrorString(HIPTENSOR_STATUS_ARCH_MISMATCH));
            return HIPTENSOR_STATUS_ARCH_MISMATCH;
        }
        return HIPTENSOR_STATUS_SUCCESS;
    }

    constexpr uint64_t WS_CAP = 512ull << 20; // most workspace split-K is ever allowed to ask for
    constexpr uint64_t PACK_CAP = 8ull << 30; // most workspace packed copies of A and B may take

    // Uploads the eight offset tables as one device block and points prob at them.
    hiptensorStatus_t uploadTables(PlanState& st)
    {
        const hipta::GemmView& v = st.view;
        const std::vector<int32_t>* tabs[8] = {&v.xp, &v.xk, &v.yq, &v.yk, &v.cp, &v.cq, &v.dp, &v.dq};
        size_t total = 0, offs[8];
        for(int i = 0; i < 8; i++)
        {
            offs[i] = total;
            total += (tabs[i]->size() + 63) / 64 * 64; // keep every table 256-byte aligned
        }
        std::vector<int32_t> host(total, 0);
        for(int i = 0; i < 8; i++)
            std::copy(tabs[i]->begin(), tabs[i]->end(), host.begin() + (long)offs[i]);
        void* dev = nullptr;
        if(hipMalloc(&dev, total * sizeof(int32_t)) != hipSuccess)
            return HIPTENSOR_STATUS_ALLOC_FAILED;
        if(hipMemcpy(dev, host.data(), total * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess)
        {
            (void)hipFree(dev);
            return HIPTENSOR_STATUS_HIP_ERROR;
        }
        st.dev_block       = dev;
        const int32_t* base = (const int32_t*)dev;
        st.prob.xp          = base + offs[0];
        st.prob.xk          = base + offs[1];
        st.prob.yq          = base + offs[2];
        st.prob.yk          = base + offs[3];
        st.prob.cp          = v.bilinear ? base + offs[4] : nullptr;
        st.prob.cq          = v.bilinear ? base + offs[5] : nullptr;
        st.prob.dp          = base + offs[6];
        st.prob.dq          = base + offs[7];
        return HIPTENSOR_STATUS_SUCCESS;
    }
}

// Exposed to the flat C ABI (c_api.cpp) only.
namespace hipta
{
    hiptensorStatus_t createHostOnlyHandle(hiptensorHandle_t** handle)
    {
        if(!handle)
            return HIPTENSOR_STATUS_NOT_INITIALIZED;
        *handle = new(std::nothrow) hiptensorHandle_t;
        if(!*handle)
            return HIPTENSOR_STATUS_ALLOC_FAILED;
        std::memset((*handle)->fields, 0, sizeof((*handle)->fields));
        Handle::create((*handle)->fields, -1, "host-only", 256, 2.4);
        return HIPTENSOR_STATUS_SUCCESS;
    }

    const PlanState* planState(const hiptensorContractionPlan_t* plan)
    {
        if(!plan || !plan->mSolution)
            return nullptr;
        const PlanState* st = (const PlanState*)plan->mSolution;
        return st->magic == PlanState::MAGIC ? st : nullptr;
    }
}

hiptensorStatus_t hiptensorCreate(hiptensorHandle_t** handle)
{
    Logger& log = Logger::get();
    log.apif("hiptensorCreate", "handle=0x%0*llX", 2 * (int)sizeof(void*), (unsigned long long)handle);
    if(!handle)
    {
        log.errorf("hiptensorCreate",
                   "Initialization Error : handle = nullptr (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    *handle = new(std::nothrow) hiptensorHandle_t;
    if(!*handle)
    {
        log.errorf("hiptensorCreate",
                   "Initialization Error : handle = nullptr (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_ALLOC_FAILED));
        return HIPTENSOR_STATUS_ALLOC_FAILED;
    }
    std::memset((*handle)->fields, 0, sizeof((*handle)->fields));

    auto fail = [&](hiptensorStatus_t st, const char* what) {
        log.errorf("hiptensorCreate", "Initialization error: %s (%s)", what, hiptensorGetErrorString(st));
        delete *handle;
        *handle = nullptr;
        return st;
    };
    hipError_t e = hipInit(0);
    if(e == hipErrorInvalidDevice)
        return fail(HIPTENSOR_STATUS_HIP_ERROR, "invalid device");
    if(e == hipErrorInvalidValue)
        return fail(HIPTENSOR_STATUS_INVALID_VALUE, "invalid value");
    if(e != hipSuccess)
        return fail(HIPTENSOR_STATUS_ARCH_MISMATCH, "no usable HIP device");
    int             dev = -1;
    hipDeviceProp_t prop;
    if(hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
        return fail(HIPTENSOR_STATUS_ARCH_MISMATCH, "no usable HIP device");
    const std::string arch(prop.gcnArchName);
    if(arch.compare(0, 6, "gfx950") != 0)
        return fail(HIPTENSOR_STATUS_ARCH_MISMATCH, "this library runs on gfx950 only");
    Handle::create((*handle)->fields, dev, arch, prop.multiProcessorCount, prop.clockRate * 1e-6);
    // look up, once per device, the address of the workspace the library itself holds (used by
    // hiptensorAmdContractionNoAlloc); a failure here is reported when that entry point is called
    void*    ws       = nullptr;
    uint64_t ws_bytes = 0;
    (void)hiptk_static_workspace(&ws, &ws_bytes, nullptr);
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorDestroy(hiptensorHandle_t* handle)
{
    Logger::get().apif("hiptensorDestroy", "handle=0x%0*llX", 2 * (int)sizeof(void*), (unsigned long long)handle);
    if(!handle)
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    Handle::destroy(handle->fields);
    delete handle;
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorInitTensorDescriptor(const hiptensorHandle_t*     handle,
                                                hiptensorTensorDescriptor_t* desc,
                                                const uint32_t               numModes,
                                                const int64_t                lens[],
                                                const int64_t                strides[],
                                                hipDataType                  dataType,
                                                hiptensorOperator_t          unaryOp)
{
    Logger&     log = Logger::get();
    const char* fn  = "hiptensorInitTensorDescriptor";
    log.apif(fn,
             "handle=0x%0*llX, desc=0x%llX, numModes=0x%02X, lens=0x%llX, strides=0x%llX,"
             "dataType=0x%02X, unaryOp=0x%02X",
             2 * (int)sizeof(void*),
             (unsigned long long)handle,
             (unsigned long long)desc,
             (unsigned)numModes,
             (unsigned long long)lens,
             (unsigned long long)strides,
             (unsigned)dataType,
             (unsigned)unaryOp);
    if(!handle || !desc)
    {
        log.errorf(fn,
                   "Initialization Error : %s = nullptr (%s)",
                   !handle ? "handle" : "contraction descriptor",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    const bool badPtrs = (lens == nullptr && strides != nullptr) || (lens == nullptr && numModes > 0);
    const bool badOp   = unaryOp != HIPTENSOR_OP_IDENTITY && unaryOp != HIPTENSOR_OP_SQRT;
    const bool badType = elemSize(dataType) == 0;
    if(badPtrs || badOp || badType)
    {
        const char* what = badPtrs ? "lens = nullptr and strides != nullptr"
                           : badOp ? "op != identity / op != unarysquare"
                                   : "datatype should be float or double";
        log.errorf(fn, "Tensor Initialization Error : %s (%s)", what, hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    // (the reference rejects f64 on devices without f64 MFMA here; gfx950 has it)

    desc->mType    = dataType;
    desc->mUnaryOp = unaryOp;
    desc->mLengths.assign(lens, lens + numModes);
    if(strides)
        desc->mStrides.assign(strides, strides + numModes);
    else
    {
        // packed, last mode fastest (what the reference's stridesFromLengths default does,
        // library/src/include/util.hpp:45-60)
        desc->mStrides.assign(numModes, 1);
        for(int i = (int)numModes - 2; i >= 0; i--)
            desc->mStrides[(size_t)i] = desc->mStrides[(size_t)i + 1] * desc->mLengths[(size_t)i + 1];
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

const char* hiptensorGetErrorString(const hiptensorStatus_t error)
{
    switch(error)
    {
    case HIPTENSOR_STATUS_SUCCESS: return "HIPTENSOR_STATUS_SUCCESS";
    case HIPTENSOR_STATUS_NOT_INITIALIZED: return "HIPTENSOR_STATUS_NOT_INITIALIZED";
    case HIPTENSOR_STATUS_ALLOC_FAILED: return "HIPTENSOR_STATUS_ALLOC_FAILED";
    case HIPTENSOR_STATUS_INVALID_VALUE: return "HIPTENSOR_STATUS_INVALID_VALUE";
    case HIPTENSOR_STATUS_ARCH_MISMATCH: return "HIPTENSOR_STATUS_ARCH_MISMATCH";
    case HIPTENSOR_STATUS_EXECUTION_FAILED: return "HIPTENSOR_STATUS_EXECUTION_FAILED";
    case HIPTENSOR_STATUS_INTERNAL_ERROR: return "HIPTENSOR_STATUS_INTERNAL_ERROR";
    case HIPTENSOR_STATUS_NOT_SUPPORTED: return "HIPTENSOR_STATUS_NOT_SUPPORTED";
    case HIPTENSOR_STATUS_CK_ERROR: return "HIPTENSOR_STATUS_CK_ERROR";
    case HIPTENSOR_STATUS_HIP_ERROR: return "HIPTENSOR_STATUS_HIP_ERROR";
    case HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE: return "HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE";
    case HIPTENSOR_STATUS_INSUFFICIENT_DRIVER: return "HIPTENSOR_STATUS_INSUFFICIENT_DRIVER";
    case HIPTENSOR_STATUS_IO_ERROR: return "HIPTENSOR_STATUS_IO_ERROR";
    }
    return "HIPTENSOR_STATUS_UNKNOWN";
}

hiptensorStatus_t hiptensorGetAlignmentRequirement(const hiptensorHandle_t*           handle,
                                                   const void*                        ptr,
                                                   const hiptensorTensorDescriptor_t* desc,
                                                   uint32_t*                          alignmentRequirement)
{
    Logger&     log = Logger::get();
    const char* fn  = "hiptensorGetAlignmentRequirement";
    log.apif(fn,
             "handle=0x%0*llX, ptr=0x%llX, desc=0x%llX, alignmentRequirement=0x%llX",
             2 * (int)sizeof(void*),
             (unsigned long long)handle,
             (unsigned long long)ptr,
             (unsigned long long)desc,
             (unsigned long long)alignmentRequirement);
    if(!handle || !desc || !alignmentRequirement)
    {
        log.errorf(fn,
                   "Error : %s = nullptr (%s)",
                   !handle ? "handle" : !desc ? "contraction descriptor" : "alignmentRequirement",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    *alignmentRequirement = 0u;
    const uint32_t es     = elemSize(desc->mType);
    for(uint32_t a = es; a != 0 && a <= 16u; a *= 2)
        if((std::size_t)ptr % a == 0)
            *alignmentRequirement = a;
    if(*alignmentRequirement == 0)
    {
        log.errorf(fn, "Error : alignment requirement is 0 (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorInitContractionDescriptor(const hiptensorHandle_t*           handle,
                                                     hiptensorContractionDescriptor_t*  desc,
                                                     const hiptensorTensorDescriptor_t* descA,
                                                     const int32_t                      modeA[],
                                                     const uint32_t                     alignmentRequirementA,
                                                     const hiptensorTensorDescriptor_t* descB,
                                                     const int32_t                      modeB[],
                                                     const uint32_t                     alignmentRequirementB,
                                                     const hiptensorTensorDescriptor_t* descC,
                                                     const int32_t                      modeC[],
                                                     const uint32_t                     alignmentRequirementC,
                                                     const hiptensorTensorDescriptor_t* descD,
                                                     const int32_t                      modeD[],
                                                     const uint32_t                     alignmentRequirementD,
                                                     hiptensorComputeType_t             typeCompute)
{
    Logger&     log = Logger::get();
    const char* fn  = "hiptensorInitContractionDescriptor";
    log.apif(fn,
             "handle=0x%0*llX, desc=0x%llX, descA=0x%llX, modeA=0x%llX, alignmentRequirementA=0x%02X, "
             "descB=0x%llX, modeB=0x%llX, alignmentRequirementB=0x%02X, descC=0x%llX, modeC=0x%llX, "
             "alignmentRequirementC=0x%02X, descD=0x%llX, modeD=0x%llX, alignmentRequirementD=0x%02X, "
             "typeCompute=0x%02X",
             2 * (int)sizeof(void*),
             (unsigned long long)handle,
             (unsigned long long)desc,
             (unsigned long long)descA,
             (unsigned long long)modeA,
             (unsigned)alignmentRequirementA,
             (unsigned long long)descB,
             (unsigned long long)modeB,
             (unsigned)alignmentRequirementB,
             (unsigned long long)descC,
             (unsigned long long)modeC,
             (unsigned)alignmentRequirementC,
             (unsigned long long)descD,
             (unsigned long long)modeD,
             (unsigned)alignmentRequirementD,
             (unsigned)typeCompute);
    if(!handle || !desc || !descA || !descB || !descD)
    {
        log.errorf(fn,
                   "Initialization Error : %s = nullptr (%s)",
                   !handle ? "handle" : !desc ? "contraction descriptor" : "Tensor descriptors",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    if(descA->mUnaryOp != HIPTENSOR_OP_IDENTITY || descB->mUnaryOp != HIPTENSOR_OP_IDENTITY
       || descD->mUnaryOp != HIPTENSOR_OP_IDENTITY || (descC && descC->mUnaryOp != HIPTENSOR_OP_IDENTITY))
    {
        log.errorf(fn,
                   "Unsupported Operator Type Error : The supported Operator is HIPTENSOR_OP_IDENTITY (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_SUPPORTED));
        return HIPTENSOR_STATUS_NOT_SUPPORTED;
    }
    if((!modeA && !descA->mLengths.empty()) || (!modeB && !descB->mLengths.empty())
       || (!modeD && !descD->mLengths.empty()))
    {
        log.errorf(fn, "Input Parameter Error : mode list = nullptr (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    const bool complexOp = typeCompute == HIPTENSOR_COMPUTE_C32F || typeCompute == HIPTENSOR_COMPUTE_C64F;
    auto       modes     = [](const int32_t* m, const hiptensorTensorDescriptor_t* d) {
        return std::vector<int32_t>(m, m + d->mLengths.size());
    };
    desc->mComputeType = typeCompute;
    if(!descC || !modeC)
    {
        // scale: C is a typeless placeholder shaped like D
        hiptensorTensorDescriptor_t none;
        none.mType    = NONE_TYPE;
        none.mUnaryOp = HIPTENSOR_OP_IDENTITY;
        none.mLengths.assign(descD->mLengths.size(), 0);
        none.mStrides.assign(descD->mStrides.size(), 0);
        desc->mContractionOpId = complexOp ? OP_SCALE_COMPLEX : OP_SCALE;
        desc->mTensorDesc      = {*descA, *descB, none, *descD};
        desc->mAlignmentReq    = {alignmentRequirementA, alignmentRequirementB, 0u, alignmentRequirementD};
        desc->mTensorMode      = {modes(modeA, descA), modes(modeB, descB), modes(modeD, descD)};
    }
    else
    {
        desc->mContractionOpId = complexOp ? OP_BILINEAR_COMPLEX : OP_BILINEAR;
        desc->mTensorDesc      = {*descA, *descB, *descC, *descD};
        desc->mAlignmentReq
            = {alignmentRequirementA, alignmentRequirementB, alignmentRequirementC, alignmentRequirementD};
        desc->mTensorMode = {modes(modeA, descA), modes(modeB, descB), modes(modeC, descC), modes(modeD, descD)};
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorInitContractionFind(const hiptensorHandle_t*    handle,
                                               hiptensorContractionFind_t* find,
                                               const hiptensorAlgo_t       algo)
{
    Logger&     log = Logger::get();
    const char* fn  = "hiptensorInitContractionFind";
    log.apif(fn,
             "handle=0x%0*llX, find=0x%llX, algo=0x%02X",
             2 * (int)sizeof(void*),
             (unsigned long long)handle,
             (unsigned long long)find,
             (int)algo);
    if(!handle || !find)
    {
        log.errorf(fn,
                   "Initialization Error : %s = nullptr (%s)",
                   !handle ? "handle" : "contraction find",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    Handle* h = Handle::from(handle->fields);
    if(!h)
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    if(auto st = checkDevice(h, fn); st != HIPTENSOR_STATUS_SUCCESS)
        return st;
    if(algo != HIPTENSOR_ALGO_DEFAULT && algo != HIPTENSOR_ALGO_DEFAULT_PATIENT && algo != HIPTENSOR_ALGO_ACTOR_CRITIC)
    {
        log.errorf(fn, "Invalid selection algorithm %d (%s)", (int)algo, hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    const auto& all = hipta::SolutionRegistry::get().all();
    if(all.empty())
    {
        log.errorf(fn, "Internal Error : No Kernels Found (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
    find->mSelectionAlgorithm = algo;
    find->mCandidates.clear();
    for(const hipta::Solution& s : all)
        find->mCandidates.push_back((void*)&s);
    return HIPTENSOR_STATUS_SUCCESS;
}

namespace
{
    std::vector<const hipta::Solution*> candidatesOf(const hiptensorContractionFind_t* find)
    {
        std::vector<const hipta::Solution*> out;
        for(void* p : find->mCandidates)
            out.push_back((const hipta::Solution*)p);
        return out;
    }
}

hiptensorStatus_t hiptensorContractionGetWorkspaceSize(const hiptensorHandle_t*                handle,
                                                       const hiptensorContractionDescriptor_t* desc,
                                                       const hiptensorContractionFind_t*       find,
                                                       const hiptensorWorksizePreference_t     pref,
                                                       uint64_t*                               workspaceSize)
{
    Logger&     log = Logger::get();
    const char* fn  = "hiptensorContractionGetWorkspaceSize";
    log.apif(fn,
             "handle=0x%0*llX, desc=0x%llX, find=0x%llX, pref=0x%02X, workspaceSize=0x%llX",
             2 * (int)sizeof(void*),
             (unsigned long long)handle,
             (unsigned long long)desc,
             (unsigned long long)find,
             (unsigned)pref,
             (unsigned long long)workspaceSize);
    if(!handle || !desc || !find || !workspaceSize)
    {
        log.errorf(fn,
                   "Initialization Error : %s = nullptr (%s)",
                   !handle ? "handle" : !desc ? "contraction descriptor" : !find ? "contraction find" : "workspace size",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    *workspaceSize = 0;
    Handle* h      = Handle::from(handle->fields);
    if(!h || !descWellFormed(desc))
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    if(pref == HIPTENSOR_WORKSPACE_MIN)
        return HIPTENSOR_STATUS_SUCCESS; // the single-pass kernels need none
    // the most a plan can use: packed copies of both operands plus split-K partials
    hipta::ContractionPlanChoice pc;
    std::string                  why;
    const hipta::ProblemIn       in = problemFromDesc(*desc);
    if(hipta::plan_contraction(in, candidatesOf(find), PACK_CAP + WS_CAP, WS_CAP, h->model(), hipta::repack_mode_from_env(), pc, why)
       != hipta::PlanStatus::OK)
        return HIPTENSOR_STATUS_SUCCESS; // nothing can run it: 0 bytes, like the reference
    if(pc.ranked.empty())
        return HIPTENSOR_STATUS_SUCCESS;
    if(pref == HIPTENSOR_WORKSPACE_RECOMMENDED)
    {
        // RECOMMENDED never asks for more than the problem's own tensors occupy (at least 64 MiB,
        // at most 1 GiB): a caller that allocates what is recommended at most doubles its footprint.
        // Plans that want more (packed copies of large operands) are left to MAX.
        const hipta::GemmView& v         = pc.view;
        const uint64_t         footprint = (uint64_t)(v.spanA + v.spanB + v.spanC + v.spanD) * (uint64_t)v.elem_bytes;
        const uint64_t         budget    = std::min<uint64_t>(1ull << 30, std::max<uint64_t>(64ull << 20, footprint));
        uint64_t               need      = pc.pack_bytes + pc.ranked.front().ws_bytes;
        if(need > budget)
        {
            hipta::ContractionPlanChoice bounded;
            if(hipta::plan_contraction(in, candidatesOf(find), budget, std::min<uint64_t>(WS_CAP, budget), h->model(), hipta::repack_mode_from_env(), bounded, why)
                   == hipta::PlanStatus::OK
               && !bounded.ranked.empty())
                need = bounded.pack_bytes + bounded.ranked.front().ws_bytes;
            else
                need = 0;
        }
        *workspaceSize = need;
    }
    else
    {
        for(const hipta::Choice& c : pc.ranked)
            *workspaceSize = std::max<uint64_t>(*workspaceSize, pc.pack_bytes + c.ws_bytes);
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

namespace hipta
{
    // defined in autotune.cpp: times the leading choices on the device, returns the index
    // of the fastest (0 when timing is not possible)
    size_t time_choices(const Handle& h, const GemmView& view, const std::vector<Choice>& ranked, size_t top, std::string& trace);
}

hiptensorStatus_t hiptensorInitContractionPlan(const hiptensorHandle_t*                handle,
                                               hiptensorContractionPlan_t*             plan,
                                               const hiptensorContractionDescriptor_t* desc,
                                               const hiptensorContractionFind_t*       find,
                                               const uint64_t                          workspaceSize)
{
    Logger&     log = Logger::get();
    const char* fn  = "hiptensorInitContractionPlan";
    log.apif(fn,
             "handle=0x%0*llX, plan=0x%llX, desc=0x%llX, find=0x%llX, workspaceSize=0x%04lX",
             2 * (int)sizeof(void*),
             (unsigned long long)handle,
             (unsigned long long)plan,
             (unsigned long long)desc,
             (unsigned long long)find,
             (unsigned long)workspaceSize);
    if(!handle || !plan || !desc || !find)
    {
        log.errorf(fn,
                   "Initialization Error : %s = nullptr (%s)",
                   !handle ? "handle" : !plan ? "plan" : !desc ? "contraction descriptor" : "contraction find",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    Handle* h = Handle::from(handle->fields);
    if(!h || !descWellFormed(desc))
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    if(auto st = checkDevice(h, fn); st != HIPTENSOR_STATUS_SUCCESS)
        return st;

    const auto             t0 = std::chrono::steady_clock::now();
    const hipta::ProblemIn in = problemFromDesc(*desc);
    // HIPTENSOR_AMD_FORCE_KERNEL="tile[,splitK]" pins the kernel choice (testing / tuning aid)
    const char*            force = std::getenv("HIPTENSOR_AMD_FORCE_KERNEL");
    const hipta::RepackMode repack = hipta::repack_mode_from_env();
    const uint64_t          ws_eff = std::min<uint64_t>(workspaceSize, PACK_CAP + WS_CAP);
    const std::string       problem = planKey(in, (int)find->mSelectionAlgorithm, 0) + (force ? std::string("|force=") + force : std::string())
                                + "|repack=" + std::to_string((int)repack);
    const std::string       key = problem + "|ws=" + std::to_string(ws_eff);
    PlanState*             st  = h->lookup(key);
    if(!st)
    {
        auto                         fresh = std::make_unique<PlanState>();
        std::string                  why;
        hipta::ContractionPlanChoice pc;
        switch(hipta::plan_contraction(in, candidatesOf(find), ws_eff, WS_CAP, h->model(), repack, pc, why))
        {
        case hipta::PlanStatus::OK: break;
        case hipta::PlanStatus::INVALID:
            log.errorf(fn, "Invalid contraction: %s (%s)", why.c_str(), hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
            return HIPTENSOR_STATUS_INVALID_VALUE;
        case hipta::PlanStatus::UNSUPPORTED_SHAPE:
            log.errorf(fn, "Unsupported contraction: %s (%s)", why.c_str(), hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_SUPPORTED));
            return HIPTENSOR_STATUS_NOT_SUPPORTED;
        case hipta::PlanStatus::UNSUPPORTED_TYPES:
            // the reference ends up here with an empty candidate set
            // (contraction_selection.cpp:187-190)
            log.errorf(fn, "Init contraction plan not successful: %s (%s)", why.c_str(), hiptensorGetErrorString(HIPTENSOR_STATUS_EXECUTION_FAILED));
            return HIPTENSOR_STATUS_EXECUTION_FAILED;
        }
        fresh->view                        = std::move(pc.view);
        fresh->pack_a                      = pc.a;
        fresh->pack_b                      = pc.b;
        fresh->pack_bytes                  = pc.pack_bytes;
        const hipta::GemmView&     v      = fresh->view;
        std::vector<hipta::Choice> ranked = std::move(pc.ranked);
        if(ranked.empty())
        {
            log.errorf(fn, "Init contraction plan not successful: no kernel candidate (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_EXECUTION_FAILED));
            return HIPTENSOR_STATUS_EXECUTION_FAILED;
        }
        if((log.mask() & HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE) && (pc.a.on || pc.b.on))
        {
            char msg[256];
            snprintf(msg,
                     sizeof(msg),
                     "packed copies: A %s (%s, %0.1f us), B %s (%s, %0.1f us), %lu bytes of workspace",
                     pc.a.on ? "yes" : "no",
                     pc.a.on ? hiptk_permute_kernel_name(&pc.a.perm) : "-",
                     pc.a.est_us,
                     pc.b.on ? "yes" : "no",
                     pc.b.on ? hiptk_permute_kernel_name(&pc.b.perm) : "-",
                     pc.b.est_us,
                     (unsigned long)pc.pack_bytes);
            log.heuristics(fn, msg);
        }
        if(log.mask() & HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE)
        {
            for(size_t i = 0; i < ranked.size() && i < 8; i++)
            {
                char msg[256];
                snprintf(msg,
                         sizeof(msg),
                         "candidate %zu: KernelId: %lu, KernelName: %s, splitK: %d, estimate: %0.3f us",
                         i,
                         (unsigned long)ranked[i].sol->uid,
                         ranked[i].sol->name.c_str(),
                         ranked[i].split_k,
                         ranked[i].est_us);
                log.heuristics(fn, msg);
            }
        }
        size_t pick = 0;
        if(find->mSelectionAlgorithm == HIPTENSOR_ALGO_DEFAULT_PATIENT && !h->hostOnly())
        {
            // HIPTENSOR_AMD_PATIENT_TOP widens (or narrows) the measured set
            size_t      top = 4;
            if(const char* e = std::getenv("HIPTENSOR_AMD_PATIENT_TOP"))
                top = (size_t)std::max(1, std::atoi(e));
            std::string trace;
            pick = hipta::time_choices(*h, v, ranked, top, trace);
            // one log line per timed candidate
            for(size_t b = 0; b < trace.size();)
            {
                size_t e = trace.find("; ", b);
                if(e == std::string::npos)
                    e = trace.size();
                log.heuristics(fn, trace.substr(b, e - b).c_str());
                b = e + 2;
            }
        }
        if(force)
        {
            int       tile = -1, split = 0;
            const int got = std::sscanf(force, "%d,%d", &tile, &split);
            size_t    hit = ranked.size();
            for(size_t i = 0; i < ranked.size() && hit == ranked.size(); i++)
                if(got >= 1 && ranked[i].sol->tile_id == tile && (got < 2 || ranked[i].split_k == split))
                    hit = i;
            if(hit == ranked.size())
            {
                log.errorf(fn, "HIPTENSOR_AMD_FORCE_KERNEL=%s matches no candidate (%s)", force, hiptensorGetErrorString(HIPTENSOR_STATUS_EXECUTION_FAILED));
                return HIPTENSOR_STATUS_EXECUTION_FAILED;
            }
            pick = hit;
        }
        const hipta::Choice& c = ranked[pick];
        // what planning decided: requests that differ only in a workspace size that did not change
        // the decision share one state (and one set of device tables)
        const std::string decision = problem + "|tile=" + std::to_string(c.sol->tile_id) + ",split=" + std::to_string(c.split_k) + ",pack="
                                     + std::to_string((int)pc.a.on) + std::to_string((int)pc.b.on) + "," + std::to_string((unsigned long long)pc.pack_bytes);
        if(PlanState* known = h->findDecision(key, decision))
        {
            st = known;
            goto planned;
        }
        fresh->magic           = PlanState::MAGIC;
        fresh->sol             = c.sol;
        fresh->ws_bytes        = fresh->pack_bytes + c.ws_bytes;
        fresh->est_us          = c.est_us;
        fresh->device          = h->device();
        fresh->compute         = (int)desc->mComputeType;
        hiptk_problem_t& p     = fresh->prob;
        p.cls                  = v.cls;
        p.op                   = v.bilinear ? HIPTK_OP_BILINEAR : HIPTK_OP_SCALE;
        p.tile_id              = c.sol->tile_id;
        p.split_k              = c.split_k;
        p.P                    = v.P;
        p.Q                    = v.Q;
        p.K                    = v.K;
        p.x_kfast              = v.x_kfast;
        p.y_kfast              = v.y_kfast;
        p.x_vec                = v.x_vec;
        p.y_vec                = v.y_vec;
        p.cd_vec               = v.cd_vec;
        p.k_affine             = v.k_affine;
        p.cd_affine = v.cd_affine;
        p.dp_stride = (int32_t)v.dp_stride;
        p.dq_stride = (int32_t)v.dq_stride;
        p.cp_stride = (int32_t)v.cp_stride;
        p.cq_stride = (int32_t)v.cq_stride;
        p.xp_stride = (int32_t)v.xp_stride;
        p.yq_stride = (int32_t)v.yq_stride;
        p.shift_p   = v.shift_p;
        p.shift_q   = v.shift_q;
        p.xy_aligned = v.xy_aligned;
        p.x_max_off = (int32_t)v.x_max_off;
        p.y_max_off = (int32_t)v.y_max_off;
        p.x_rows_adjacent = v.x_rows_adjacent;
        p.y_rows_adjacent = v.y_rows_adjacent;
        p.xk_stride            = (int32_t)v.xk_stride;
        p.yk_stride            = (int32_t)v.yk_stride;
        (void)hiptk_resolve(&p); // the registry is searched here, once, not at every launch
        fresh->kernel_name     = hiptk_kernel_name(&p);
        if(!h->hostOnly())
            if(auto e = uploadTables(*fresh); e != HIPTENSOR_STATUS_SUCCESS)
            {
                log.errorf(fn, "Could not place the offset tables on the device (%s)", hiptensorGetErrorString(e));
                return e;
            }
        st = h->intern(key, decision, std::move(fresh));
    }
planned:
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    if(log.mask() & HIPTENSOR_LOG_LEVEL_PERF_TRACE)
    {
        char msg[512];
        snprintf(msg,
                 sizeof(msg),
                 "Algo: %d, KernelId: %lu, KernelName: %s, SelectionTime: %0.3f ms",
                 (int)find->mSelectionAlgorithm,
                 (unsigned long)st->sol->uid,
                 st->kernel_name.c_str(),
                 ms);
        log.perf(fn, msg);
    }
    plan->mContractionDesc = *desc;
    plan->mSolution        = st;
    return HIPTENSOR_STATUS_SUCCESS;
}

namespace
{
    // hiptensorContraction, and its variant that takes the workspace from the library's own device
    // array instead of the caller (static_ws: `workspace` / `workspaceSize` are ignored, nothing is
    // allocated and no event is created, so PERF_TRACE timing is left out).
    hiptensorStatus_t contractionImpl(const char*                       fn,
                                      bool                              static_ws,
                                      const hiptensorHandle_t*          handle,
                                      const hiptensorContractionPlan_t* plan,
                                      const void*                       alpha,
                                      const void*                       A,
                                      const void*                       B,
                                      const void*                       beta,
                                      const void*                       C,
                                      void*                             D,
                                      void*                             workspace,
                                      uint64_t                          workspaceSize,
                                      hipStream_t                       stream);
}

hiptensorStatus_t hiptensorContraction(const hiptensorHandle_t*          handle,
                                       const hiptensorContractionPlan_t* plan,
                                       const void*                       alpha,
                                       const void*                       A,
                                       const void*                       B,
                                       const void*                       beta,
                                       const void*                       C,
                                       void*                             D,
                                       void*                             workspace,
                                       uint64_t                          workspaceSize,
                                       hipStream_t                       stream)
{
    return contractionImpl("hiptensorContraction", false, handle, plan, alpha, A, B, beta, C, D, workspace, workspaceSize, stream);
}

namespace hipta
{
    hiptensorStatus_t contractionNoAlloc(const hiptensorHandle_t*          handle,
                                         const hiptensorContractionPlan_t* plan,
                                         const void*                       alpha,
                                         const void*                       A,
                                         const void*                       B,
                                         const void*                       beta,
                                         const void*                       C,
                                         void*                             D,
                                         hipStream_t                       stream)
    {
        return contractionImpl("hiptensorAmdContractionNoAlloc", true, handle, plan, alpha, A, B, beta, C, D, nullptr, 0, stream);
    }
}

namespace
{
hiptensorStatus_t contractionImpl(const char*                       fn,
                                  bool                              static_ws,
                                  const hiptensorHandle_t*          handle,
                                  const hiptensorContractionPlan_t* plan,
                                  const void*                       alpha,
                                  const void*                       A,
                                  const void*                       B,
                                  const void*                       beta,
                                  const void*                       C,
                                  void*                             D,
                                  void*                             workspace,
                                  uint64_t                          workspaceSize,
                                  hipStream_t                       stream)
{
    Logger&     log = Logger::get();
    if(log.mask() & HIPTENSOR_LOG_LEVEL_API_TRACE)
    {
        char   am[64] = "alpha=NULL", bm[64] = "beta=NULL";
        double v[2];
        if(plan && alpha && readScalar(alpha, (int)plan->mContractionDesc.mComputeType, v))
            snprintf(am, sizeof(am), "alpha=%.6lf", v[0]);
        if(plan && beta && readScalar(beta, (int)plan->mContractionDesc.mComputeType, v))
            snprintf(bm, sizeof(bm), "beta=%.6lf", v[0]);
        log.apif(fn,
                 "handle=0x%0*llX, plan=0x%llX, %s, A=0x%llX, B=0x%llX, %s, "
                 "C=0x%llX, D=0x%llX, workspace=0x%llX, workspaceSize=0x%04lX, stream=0x%llX",
                 2 * (int)sizeof(void*),
                 (unsigned long long)handle,
                 (unsigned long long)plan,
                 am,
                 (unsigned long long)A,
                 (unsigned long long)B,
                 bm,
                 (unsigned long long)C,
                 (unsigned long long)D,
                 (unsigned long long)workspace,
                 (unsigned long)workspaceSize,
                 (unsigned long long)stream);
    }
    if(!handle || !plan)
    {
        log.errorf(fn,
                   "Initialization Error : %s = nullptr (%s)",
                   !handle ? "handle" : "plan",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_NOT_INITIALIZED));
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    }
    if(!alpha || !A || !B || !D)
    {
        log.errorf(fn,
                   "Input Parameter Error : %s = nullptr (%s)",
                   !alpha ? "alpha" : "A/B/D",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    if(!plan->mSolution)
    {
        log.errorf(fn, "Internal Error : solution = nullptr (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
    Handle* h = Handle::from(handle->fields);
    if(!h)
        return HIPTENSOR_STATUS_NOT_INITIALIZED;
    if(h->hostOnly())
    {
        log.errorf(fn, "This handle has no device; it can plan but not execute (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_ARCH_MISMATCH));
        return HIPTENSOR_STATUS_ARCH_MISMATCH;
    }
    if(auto st = checkDevice(h, fn); st != HIPTENSOR_STATUS_SUCCESS)
        return st;
    if(plan->mSolution && ((const PlanState*)plan->mSolution)->magic == PlanState::RETIRED)
    {
        // (retired states stay allocated for the life of the process, so this read is safe)
        log.errorf(fn,
                   "This plan is no longer valid: its handle was destroyed, or the handle's plan cache retired it "
                   "before it was ever executed; create the plan again (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
    const PlanState* st = hipta::planState(plan);
    // from its first execution on a state is never retired by the cache (the device may hold its
    // table addresses beyond this call); a state the cache retired a moment ago is refused here
    if(st && !Handle::pin(st))
    {
        log.errorf(fn,
                   "This plan is no longer valid: the handle's plan cache retired it before it was ever executed; "
                   "create the plan again (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
    if(st)
        st->last_use.store(hipta::next_use_tick(), std::memory_order_relaxed);
    if(!st || st->device != h->device() || !st->dev_block)
    {
        log.errorf(fn, "Selected kernel is unable to solve the problem (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
    const bool bilinear = st->view.bilinear;
    if(bilinear && (!C || !beta))
    {
        log.errorf(fn, "Input Parameter Error : beta/C = nullptr (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    if(static_ws)
    {
        // the workspace is the library's own device array: a fixed size, shared by every call on
        // this device
        workspace     = nullptr;
        workspaceSize = 0;
        if(st->ws_bytes > 0)
        {
            int hipErr = 0;
            if(hiptk_static_workspace(&workspace, &workspaceSize, &hipErr) != HIPTK_OK)
            {
                log.errorf(fn, "The library's workspace is not available on this device: hip error %d (%s)", hipErr, hiptensorGetErrorString(HIPTENSOR_STATUS_HIP_ERROR));
                return HIPTENSOR_STATUS_HIP_ERROR;
            }
            if(st->ws_bytes > workspaceSize)
            {
                log.errorf(fn,
                           "This plan needs %lu bytes of workspace; the library's own holds %lu: plan with a smaller workspaceSize, "
                           "or call hiptensorContraction with a workspace of the caller's (%s)",
                           (unsigned long)st->ws_bytes,
                           (unsigned long)workspaceSize,
                           hiptensorGetErrorString(HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE));
                return HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE;
            }
        }
    }
    if(st->ws_bytes > 0 && (!workspace || workspaceSize < st->ws_bytes))
    {
        log.errorf(fn,
                   "Insufficient workspace: req: %lu alloc: %lu (%s)",
                   (unsigned long)st->ws_bytes,
                   (unsigned long)workspaceSize,
                   hiptensorGetErrorString(HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE));
        return HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE;
    }

    double av[2], bv[2] = {0, 0};
    readScalar(alpha, st->compute, av);
    if(beta)
        readScalar(beta, st->compute, bv);
    alignas(16) unsigned char ab[16], bb[16];
    packScalar(st->prob.cls, av, ab);
    packScalar(st->prob.cls, bv, bb);

    bool timed = !static_ws && (log.mask() & HIPTENSOR_LOG_LEVEL_PERF_TRACE) != 0;
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
    int  hipErr     = 0;
    int  rc         = HIPTK_OK;
    bool misaligned = false;
    if(st->pack_bytes)
    {
        // the copies start at the first 256-byte boundary of the workspace; what follows them is
        // left to the kernel (split-K partials)
        const uintptr_t base = (reinterpret_cast<uintptr_t>(workspace) + hipta::PACK_ALIGN - 1) / hipta::PACK_ALIGN * hipta::PACK_ALIGN;
        const uint64_t  lead = (uint64_t)(base - reinterpret_cast<uintptr_t>(workspace));
        char*           wsb  = reinterpret_cast<char*>(base);
        if(st->pack_a.on && rc == HIPTK_OK)
        {
            rc = hiptk_permute(&st->pack_a.perm, A, wsb + st->pack_a.offset, (void*)stream, &hipErr);
            A  = wsb + st->pack_a.offset;
        }
        if(st->pack_b.on && rc == HIPTK_OK)
        {
            rc = hiptk_permute(&st->pack_b.perm, B, wsb + st->pack_b.offset, (void*)stream, &hipErr);
            B  = wsb + st->pack_b.offset;
        }
        misaligned = rc == HIPTK_ERR_ARG; // the only argument a plan's own move can get wrong
        const uint64_t used = st->pack_bytes - hipta::PACK_ALIGN + lead;
        workspace           = wsb + (st->pack_bytes - hipta::PACK_ALIGN);
        workspaceSize       = workspaceSize - used;
    }
    const void* X = st->view.swapped ? B : A;
    const void* Y = st->view.swapped ? A : B;
    if(rc == HIPTK_OK)
        rc = hiptk_contract(&st->prob, ab, bilinear ? bb : nullptr, X, Y, bilinear ? C : nullptr, D, workspace, workspaceSize, (void*)stream, &hipErr);
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
            // same formulas as the reference (hiptensor_contraction.cpp:785-796):
            // flops = 2 M N K, TFlops = flops / 1e9 / ms, GB/s = bytes / 1e6 / ms
            const hipta::GemmView& v     = st->view;
            const double           flops = 2.0 * (double)v.P * (double)v.Q * (double)v.K;
            const double           bytes = ((double)v.P * v.K + (double)v.Q * v.K + (double)v.P * v.Q * (bilinear ? 2 : 1)) * v.elem_bytes;
            char                   msg[512];
            snprintf(msg,
                     sizeof(msg),
                     "KernelId: %lu KernelName: %s, %0.3f ms, %0.3f TFlops, %0.3f GB/s%s",
                     (unsigned long)st->sol->uid,
                     // (the kernel that ran: the plan's, or its register-staged stand-in for operands
                     // that are not 16-byte aligned)
                     hiptk_kernel_name_at(&st->prob, X, Y),
                     ms,
                     flops / 1e9 / ms,
                     bytes / 1e6 / ms,
                     // (the time then covers the moves into the packed copies as well)
                     st->pack_a.on && st->pack_b.on ? ", A and B from packed copies"
                     : st->pack_a.on               ? ", A from a packed copy"
                     : st->pack_b.on               ? ", B from a packed copy"
                                                   : "");
            log.perf(fn, msg);
        }
    }
    if(misaligned)
    {
        log.errorf(fn,
                   "An operand is not aligned as its contraction descriptor declared (%s)",
                   hiptensorGetErrorString(HIPTENSOR_STATUS_INVALID_VALUE));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    switch(rc)
    {
    case HIPTK_OK: return HIPTENSOR_STATUS_SUCCESS;
    case HIPTK_ERR_WORKSPACE:
        log.errorf(fn,
                   "Insufficient workspace: req: %lu alloc: %lu (%s)",
                   (unsigned long)st->ws_bytes,
                   (unsigned long)workspaceSize,
                   hiptensorGetErrorString(HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE));
        return HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE;
    case HIPTK_ERR_LAUNCH:
        log.errorf(fn, "Kernel launch failed: %s (%s)", hipGetErrorString((hipError_t)hipErr), hiptensorGetErrorString(HIPTENSOR_STATUS_EXECUTION_FAILED));
        return HIPTENSOR_STATUS_EXECUTION_FAILED;
    default:
        log.errorf(fn, "Selected kernel is unable to solve the problem (%s)", hiptensorGetErrorString(HIPTENSOR_STATUS_INTERNAL_ERROR));
        return HIPTENSOR_STATUS_INTERNAL_ERROR;
    }
}
} // namespace

// ---- logger control (reference: library/src/hiptensor.cpp:323-458) ----

hiptensorStatus_t hiptensorLoggerSetCallback(hiptensorLoggerCallback_t callback)
{
    Logger& log = Logger::get();
    log.apif("hiptensorLoggerSetCallback", "callback=0x%0*llX", 2 * (int)sizeof(void*), (unsigned long long)callback);
    auto r = log.setCallback(callback);
    if(r != Logger::Result::OK)
    {
        log.errorf("hiptensorLoggerSetCallback", "Error : logger set callback not successful (%s)", Logger::resultName(r));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorLoggerSetFile(FILE* file)
{
    Logger& log = Logger::get();
    log.apif("hiptensorLoggerSetFile", "file=0x%0*llX", 2 * (int)sizeof(void*), (unsigned long long)file);
    auto r = log.setStream(file);
    if(r != Logger::Result::OK)
    {
        log.errorf("hiptensorLoggerSetFile", "Error : logger set file not successful (%s)", Logger::resultName(r));
        return HIPTENSOR_STATUS_IO_ERROR;
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorLoggerOpenFile(const char* logFile)
{
    Logger& log = Logger::get();
    log.apif("hiptensorLoggerOpenFile", "logFile=%s", logFile ? logFile : "(null)");
    auto r = log.openFile(logFile);
    if(r != Logger::Result::OK)
    {
        log.errorf("hiptensorLoggerOpenFile", "fileName=%s (%s)", logFile ? logFile : "(null)", Logger::resultName(r));
        return HIPTENSOR_STATUS_IO_ERROR;
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorLoggerSetLevel(hiptensorLogLevel_t level)
{
    Logger& log = Logger::get();
    log.apif("hiptensorLoggerSetLevel", "log level=0x%02X", (unsigned)level);
    auto r = log.setLevel((int)level);
    if(r != Logger::Result::OK)
    {
        log.errorf("hiptensorLoggerSetLevel", "level=0x%02X (%s)", (unsigned)level, Logger::resultName(r));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorLoggerSetMask(int32_t mask)
{
    Logger& log = Logger::get();
    log.apif("hiptensorLoggerSetMask", "mask=0x%02X", (unsigned)mask);
    auto r = log.setMask(mask);
    if(r != Logger::Result::OK)
    {
        log.errorf("hiptensorLoggerSetMask", "mask=0x%02X (%s)", (unsigned)mask, Logger::resultName(r));
        return HIPTENSOR_STATUS_INVALID_VALUE;
    }
    return HIPTENSOR_STATUS_SUCCESS;
}

hiptensorStatus_t hiptensorLoggerForceDisable()
{
    Logger& log = Logger::get();
    log.api("hiptensorLoggerForceDisable", "Logging Disabled");
    log.setEnabled(false);
    return HIPTENSOR_STATUS_SUCCESS;
}

int hiptensorGetHiprtVersion()
{
    Logger::get().api("hiptensorGetHiprtVersion", "");
    int version = 0;
    if(hipRuntimeGetVersion(&version) != hipSuccess)
    {
        Logger::get().errorf("hiptensorGetHiprtVersion", "Error : hipRuntimeGetVersion failed");
        return -1;
    }
    return version;
}
