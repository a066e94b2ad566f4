// Public entry points of the contraction path and of the tensor permutation beside it.
//
// Declarations are source-compatible with hipTensor 1.4's
// library/include/hiptensor/hiptensor.hpp (line numbers cited per function), so a
// program written against that header compiles and links against this library
// unchanged.  Functions have C++ linkage because the descriptor structs carry
// std::vector members, exactly as in the reference; a flat extern "C" flavour of
// the same calls lives in <hiptensor_amd.h>.
//
// hiptensorReduction (hiptensor.hpp:230-300) is not part of this path and is not provided.
#ifndef HIPTENSOR_API_HPP
#define HIPTENSOR_API_HPP

#include "hiptensor_types.hpp"
#include "internal/hiptensor_utility.hpp"

// Allocates a handle bound to the current HIP device, which must be a gfx950 GPU
// (HIPTENSOR_STATUS_ARCH_MISMATCH otherwise).                     [hiptensor.hpp:41]
hiptensorStatus_t hiptensorCreate(hiptensorHandle_t** handle);

// Releases the handle and every plan state / device table it owns. [hiptensor.hpp:46]
hiptensorStatus_t hiptensorDestroy(hiptensorHandle_t* handle);

// Fills a tensor descriptor.  `strides == nullptr` means packed with the LAST mode
// fastest (row-major), which is what the reference does despite its comment.
//                                                              [hiptensor.hpp:60-66]
hiptensorStatus_t hiptensorInitTensorDescriptor(const hiptensorHandle_t*     handle,
                                                hiptensorTensorDescriptor_t* desc,
                                                const uint32_t               numModes,
                                                const int64_t                lens[],
                                                const int64_t                strides[],
                                                hipDataType                  dataType,
                                                hiptensorOperator_t          unaryOp);

// Name of a status code.                                           [hiptensor.hpp:71]
const char* hiptensorGetErrorString(const hiptensorStatus_t error);

// B[perm(index)] = opB(alpha * opA(A[index])) for f16 or f32 tensors of 2 to 6 modes; modeB is
// a reordering of modeA.  As in the reference, both tensors are taken as packed with their
// FIRST listed mode fastest, whatever strides the descriptors hold, and the unary operator
// HIPTENSOR_OP_SQRT squares its argument.  alpha is a host pointer to one scalar of
// typeScalar (HIP_R_16F or HIP_R_32F).  Enqueued on `stream`, returns without synchronising.
//                                                              [hiptensor.hpp:89-98]
hiptensorStatus_t hiptensorPermutation(const hiptensorHandle_t*           handle,
                                       const void*                        alpha,
                                       const void*                        A,
                                       const hiptensorTensorDescriptor_t* descA,
                                       const int32_t                      modeA[],
                                       void*                              B,
                                       const hiptensorTensorDescriptor_t* descB,
                                       const int32_t                      modeB[],
                                       const hipDataType                  typeScalar,
                                       const hipStream_t                  stream);

// Largest power-of-two alignment (element size .. 16 bytes) of `ptr`.
//                                                            [hiptensor.hpp:108-111]
hiptensorStatus_t hiptensorGetAlignmentRequirement(const hiptensorHandle_t*           handle,
                                                   const void*                        ptr,
                                                   const hiptensorTensorDescriptor_t* desc,
                                                   uint32_t* alignmentRequirement);

// Describes D = alpha * A * B + beta * C (descC / modeC non-null) or
// D = alpha * A * B (descC or modeC null).                    [hiptensor.hpp:131-145]
hiptensorStatus_t hiptensorInitContractionDescriptor(const hiptensorHandle_t*           handle,
                                                     hiptensorContractionDescriptor_t*  desc,
                                                     const hiptensorTensorDescriptor_t* descA,
                                                     const int32_t                      modeA[],
                                                     const uint32_t alignmentRequirementA,
                                                     const hiptensorTensorDescriptor_t* descB,
                                                     const int32_t                      modeB[],
                                                     const uint32_t alignmentRequirementB,
                                                     const hiptensorTensorDescriptor_t* descC,
                                                     const int32_t                      modeC[],
                                                     const uint32_t alignmentRequirementC,
                                                     const hiptensorTensorDescriptor_t* descD,
                                                     const int32_t                      modeD[],
                                                     const uint32_t         alignmentRequirementD,
                                                     hiptensorComputeType_t typeCompute);

// Chooses the selection policy and lists the candidate kernel families.
//                                                            [hiptensor.hpp:157-159]
hiptensorStatus_t hiptensorInitContractionFind(const hiptensorHandle_t*    handle,
                                               hiptensorContractionFind_t* find,
                                               const hiptensorAlgo_t       algo);

// Workspace in bytes: 0 for MIN; what the heuristic's split-K choice needs for
// RECOMMENDED; the largest any candidate could use for MAX.   [hiptensor.hpp:170-174]
hiptensorStatus_t hiptensorContractionGetWorkspaceSize(const hiptensorHandle_t* handle,
                                                       const hiptensorContractionDescriptor_t* desc,
                                                       const hiptensorContractionFind_t*       find,
                                                       const hiptensorWorksizePreference_t     pref,
                                                       uint64_t* workspaceSize);

// Folds the problem into a GEMM view, picks a kernel and uploads the offset tables.
// Everything the execute call needs is computed here, once.    [hiptensor.hpp:191-195]
hiptensorStatus_t hiptensorInitContractionPlan(const hiptensorHandle_t*                handle,
                                               hiptensorContractionPlan_t*             plan,
                                               const hiptensorContractionDescriptor_t* desc,
                                               const hiptensorContractionFind_t*       find,
                                               const uint64_t workspaceSize);

// Enqueues the contraction on `stream` and returns without synchronising.  alpha and
// beta are host pointers to one scalar of the compute type.  D may alias C.
//                                                            [hiptensor.hpp:218-228]
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
                                       hipStream_t                       stream);

// Logger control.                                             [hiptensor.hpp:308-338]
hiptensorStatus_t hiptensorLoggerSetCallback(hiptensorLoggerCallback_t callback);
hiptensorStatus_t hiptensorLoggerSetFile(FILE* file);
hiptensorStatus_t hiptensorLoggerOpenFile(const char* logFile);
hiptensorStatus_t hiptensorLoggerSetLevel(hiptensorLogLevel_t level);
hiptensorStatus_t hiptensorLoggerSetMask(int32_t mask);
hiptensorStatus_t hiptensorLoggerForceDisable();

// HIP runtime version the library was built against.               [hiptensor.hpp:343]
int hiptensorGetHiprtVersion();

#endif // HIPTENSOR_API_HPP
