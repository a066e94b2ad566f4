// Public types of the contraction path.
//
// Source- and layout-compatible with the types that hipTensor 1.4 declares in
// library/include/hiptensor/hiptensor_types.hpp:42-238 (same enumerator names
// and values, same struct members in the same order), so that programs written
// against that header build and link against this library unchanged.
#ifndef HIPTENSOR_TYPES_HPP
#define HIPTENSOR_TYPES_HPP

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <vector>

#include <hip/hip_common.h>
#include <hip/library_types.h>

// ---------------------------------------------------------------------------
// Status codes returned by every entry point (hiptensor_types.hpp:42-71).
// ---------------------------------------------------------------------------
typedef enum
{
    HIPTENSOR_STATUS_SUCCESS                = 0, // call completed
    HIPTENSOR_STATUS_NOT_INITIALIZED        = 1, // a handle / descriptor / plan pointer was null
    HIPTENSOR_STATUS_ALLOC_FAILED           = 3, // host or device allocation failed
    HIPTENSOR_STATUS_INVALID_VALUE          = 7, // an argument is out of its domain
    HIPTENSOR_STATUS_ARCH_MISMATCH          = 8, // device is not gfx950, or not the handle's device
    HIPTENSOR_STATUS_EXECUTION_FAILED       = 13, // a kernel launch failed / no kernel for the types
    HIPTENSOR_STATUS_INTERNAL_ERROR         = 14, // plan holds no solution, or it cannot run the problem
    HIPTENSOR_STATUS_NOT_SUPPORTED          = 15, // operation outside what this path implements
    HIPTENSOR_STATUS_CK_ERROR               = 17, // kept for compatibility; never returned here
    HIPTENSOR_STATUS_HIP_ERROR              = 18, // a HIP runtime call failed
    HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE = 19, // workspace smaller than the plan needs
    HIPTENSOR_STATUS_INSUFFICIENT_DRIVER    = 20,
    HIPTENSOR_STATUS_IO_ERROR               = 21,
} hiptensorStatus_t;

// ---------------------------------------------------------------------------
// Arithmetic type used inside the contraction; also the type alpha / beta are
// read as (hiptensor_types.hpp:74-99).
// ---------------------------------------------------------------------------
typedef enum
{
    HIPTENSOR_COMPUTE_NONE = 0,
    HIPTENSOR_COMPUTE_16F  = (1U << 0U),
    HIPTENSOR_COMPUTE_32F  = (1U << 2U),
    HIPTENSOR_COMPUTE_64F  = (1U << 4U),
    HIPTENSOR_COMPUTE_8U   = (1U << 6U), // reserved
    HIPTENSOR_COMPUTE_32U  = (1U << 7U), // reserved
    HIPTENSOR_COMPUTE_8I   = (1U << 8U), // reserved
    HIPTENSOR_COMPUTE_32I  = (1U << 9U), // reserved
    HIPTENSOR_COMPUTE_16BF = (1U << 10U),
    HIPTENSOR_COMPUTE_C32F = (1U << 11U),
    HIPTENSOR_COMPUTE_C64F = (1U << 12U),
} hiptensorComputeType_t;

// Element-wise operators attached to tensor descriptors (hiptensor_types.hpp:102-121).
// Contraction accepts HIPTENSOR_OP_IDENTITY only.
typedef enum
{
    HIPTENSOR_OP_IDENTITY = 1,
    HIPTENSOR_OP_SQRT     = 2,
    HIPTENSOR_OP_ADD      = 3,
    HIPTENSOR_OP_MUL      = 5,
    HIPTENSOR_OP_MAX      = 6,
    HIPTENSOR_OP_MIN      = 7,
    HIPTENSOR_OP_UNKNOWN  = 126,
} hiptensorOperator_t;

// Kernel selection policy (hiptensor_types.hpp:124-133).  All three values are
// accepted.  DEFAULT and ACTOR_CRITIC use the analytic tile heuristic;
// DEFAULT_PATIENT additionally times the heuristic's top candidates on the device.
typedef enum
{
    HIPTENSOR_ALGO_ACTOR_CRITIC    = -8,
    HIPTENSOR_ALGO_DEFAULT_PATIENT = -6,
    HIPTENSOR_ALGO_DEFAULT         = -1,
} hiptensorAlgo_t;

// Workspace policy (hiptensor_types.hpp:136-145).  MIN is always 0 bytes (the
// single-pass kernels need none); RECOMMENDED / MAX return what split-K needs.
typedef enum
{
    HIPTENSOR_WORKSPACE_MIN         = 1,
    HIPTENSOR_WORKSPACE_RECOMMENDED = 2,
    HIPTENSOR_WORKSPACE_MAX         = 3,
} hiptensorWorksizePreference_t;

// Logger mask bits (hiptensor_types.hpp:149-164).
typedef enum
{
    HIPTENSOR_LOG_LEVEL_OFF              = 0,
    HIPTENSOR_LOG_LEVEL_ERROR            = 1,
    HIPTENSOR_LOG_LEVEL_PERF_TRACE       = 2,
    HIPTENSOR_LOG_LEVEL_PERF_HINT        = 4,
    HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE = 8,
    HIPTENSOR_LOG_LEVEL_API_TRACE        = 16,
} hiptensorLogLevel_t;

// Opaque library context: 4 KiB the library places its own state in
// (hiptensor_types.hpp:167-170).
struct hiptensorHandle_t
{
    int64_t fields[512];
};

// Element type, extents, strides (in elements) and unary operator of one tensor
// (hiptensor_types.hpp:177-187).
struct hiptensorTensorDescriptor_t
{
    hipDataType              mType;
    std::vector<std::size_t> mLengths;
    std::vector<std::size_t> mStrides;
    hiptensorOperator_t      mUnaryOp;
};

// One contraction problem: op id (scale / bilinear, real / complex), compute type,
// the four tensor descriptors {A, B, C, D}, their alignments in bytes and the mode
// lists {A, B, D} (scale) or {A, B, C, D} (bilinear) (hiptensor_types.hpp:196-208).
struct hiptensorContractionDescriptor_t
{
    int32_t                                  mContractionOpId;
    hiptensorComputeType_t                   mComputeType;
    std::vector<hiptensorTensorDescriptor_t> mTensorDesc;
    std::vector<uint32_t>                    mAlignmentReq;
    std::vector<std::vector<int32_t>>        mTensorMode;
};

// Selection policy plus the candidate kernel families it may pick from
// (hiptensor_types.hpp:211-217).  The candidates are non-owning pointers into the
// library's registry.
struct hiptensorContractionFind_t
{
    hiptensorAlgo_t    mSelectionAlgorithm;
    std::vector<void*> mCandidates;
};

// A planned contraction (hiptensor_types.hpp:221-227).  mSolution is a non-owning
// pointer to immutable plan state owned by the handle that created it.
struct hiptensorContractionPlan_t
{
    void*                            mSolution;
    hiptensorContractionDescriptor_t mContractionDesc;
};

// Log sink: (context bit, function name, message) (hiptensor_types.hpp:234-236).
typedef void (*hiptensorLoggerCallback_t)(int32_t logContext, const char* funcName, const char* msg);

#endif // HIPTENSOR_TYPES_HPP
