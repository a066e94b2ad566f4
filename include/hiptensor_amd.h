/*
 * Flat C ABI of the contraction path and of the tensor permutation (extern "C", plain
 * pointers and sizes).
 *
 * The reference's public functions take C++ structs with std::vector members
 * (library/include/hiptensor/hiptensor_types.hpp:177-227), so they cannot be bound
 * from C, ctypes, cgo or JNI.  Each function below is the same call with those
 * structs held behind opaque pointers that the library allocates; argument meaning,
 * check order and status codes are those of the function cited beside it, because
 * each one forwards to that function's implementation in this library.
 *
 * Status codes are hiptensorStatus_t values (0 = success).  Data types are
 * hipDataType values (0 f32, 1 f64, 2 f16, 4 c32, 5 c64, 14 bf16), compute types
 * hiptensorComputeType_t values (1 f16, 4 f32, 16 f64, 1024 bf16, 2048 c32, 4096 c64).
 */
#ifndef HIPTENSOR_AMD_H
#define HIPTENSOR_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hiptensorCreate / hiptensorDestroy            (library/include/hiptensor/hiptensor.hpp:41,46) */
int hiptensorAmdCreate(void** handle);
int hiptensorAmdDestroy(void* handle);
/* A handle without a device: descriptors, workspace queries and planning work (for
 * inspection and host-side tests); hiptensorAmdContraction refuses it with
 * HIPTENSOR_STATUS_ARCH_MISMATCH.  No counterpart in the reference. */
int hiptensorAmdCreateHostOnly(void** handle);

/* hiptensorInitTensorDescriptor                                        (hiptensor.hpp:60-66) */
int hiptensorAmdInitTensorDescriptor(const void*    handle,
                                     void**         desc,
                                     uint32_t       numModes,
                                     const int64_t* lens,
                                     const int64_t* strides,
                                     int            dataType,
                                     int            unaryOp);
int hiptensorAmdDestroyTensorDescriptor(void* desc);

/* hiptensorGetErrorString                                                 (hiptensor.hpp:71) */
const char* hiptensorAmdGetErrorString(int status);

/* hiptensorGetAlignmentRequirement                                   (hiptensor.hpp:108-111) */
int hiptensorAmdGetAlignmentRequirement(const void* handle,
                                        const void* ptr,
                                        const void* desc,
                                        uint32_t*   alignmentRequirement);

/* hiptensorInitContractionDescriptor                                 (hiptensor.hpp:131-145) */
int hiptensorAmdInitContractionDescriptor(const void*    handle,
                                          void**         desc,
                                          const void*    descA,
                                          const int32_t* modeA,
                                          uint32_t       alignmentRequirementA,
                                          const void*    descB,
                                          const int32_t* modeB,
                                          uint32_t       alignmentRequirementB,
                                          const void*    descC,
                                          const int32_t* modeC,
                                          uint32_t       alignmentRequirementC,
                                          const void*    descD,
                                          const int32_t* modeD,
                                          uint32_t       alignmentRequirementD,
                                          int            typeCompute);
int hiptensorAmdDestroyContractionDescriptor(void* desc);

/* hiptensorInitContractionFind                                       (hiptensor.hpp:157-159) */
int hiptensorAmdInitContractionFind(const void* handle, void** find, int algo);
int hiptensorAmdDestroyContractionFind(void* find);

/* hiptensorContractionGetWorkspaceSize                               (hiptensor.hpp:170-174) */
int hiptensorAmdContractionGetWorkspaceSize(
    const void* handle, const void* desc, const void* find, int pref, uint64_t* workspaceSize);

/* hiptensorInitContractionPlan                                       (hiptensor.hpp:191-195) */
int hiptensorAmdInitContractionPlan(
    const void* handle, void** plan, const void* desc, const void* find, uint64_t workspaceSize);
int hiptensorAmdDestroyContractionPlan(void* plan);

/* hiptensorContraction; stream is a hipStream_t                      (hiptensor.hpp:218-228) */
int hiptensorAmdContraction(const void* handle,
                            const void* plan,
                            const void* alpha,
                            const void* A,
                            const void* B,
                            const void* beta,
                            const void* C,
                            void*       D,
                            void*       workspace,
                            uint64_t    workspaceSize,
                            void*       stream);

/* hiptensorAmdContraction for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results as hiptensorAmdContraction, minus the workspace: whatever
 * workspace the plan needs (split-K partials, packed operand copies) is taken from a device array
 * of HIPTK_STATIC_WORKSPACE_BYTES (32 MiB) that the library itself holds on every device until the
 * process ends.  The call allocates nothing and frees nothing (and skips the PERF_TRACE timing,
 * which would create events).  A plan that needs more than the array holds is refused with
 * HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE: plan with a smaller workspaceSize.  Every call on one
 * device uses the same array: calls that overlap in time on one device (different streams, or
 * threads) race on it and must be serialised by the caller; calls in one stream are safe. */
int hiptensorAmdContractionNoAlloc(const void* handle,
                                   const void* plan,
                                   const void* alpha,
                                   const void* A,
                                   const void* B,
                                   const void* beta,
                                   const void* C,
                                   void*       D,
                                   void*       stream);

/* hiptensorPermutation; typeScalar is a hipDataType, stream a hipStream_t  (hiptensor.hpp:89-98) */
int hiptensorAmdPermutation(const void*    handle,
                            const void*    alpha,
                            const void*    A,
                            const void*    descA,
                            const int32_t* modeA,
                            void*          B,
                            const void*    descB,
                            const int32_t* modeB,
                            int            typeScalar,
                            void*          stream);

/* What hiptensorAmdPermutation would launch for these descriptors, mode lists and addresses
 * (only the alignment of A and B is looked at; nothing is read or launched, no device is
 * needed).  Returns the status the call would return before launching.  No counterpart in
 * the reference. */
typedef struct hiptensorAmdPermutationInfo
{
    int32_t fused_rank;   /* modes left after extent-1 modes are dropped and neighbours fused */
    int32_t extent[6];    /* fused extents in A's order, fastest first                        */
    int32_t a_stride[6], b_stride[6];
    int32_t kernel;       /* HIPTK_PERM_COPY / TILED / ROWS / GATHER / STRIP / GROUPED / SHARED */
    int32_t mode_i, mode_j, tile, vec_r, vec_w;
    int32_t empty;        /* 1: an extent is zero, nothing would be launched                  */
    char    kernel_name[96];
} hiptensorAmdPermutationInfo_t;
int hiptensorAmdPermutationInfo(const void*                    descA,
                                const int32_t*                 modeA,
                                const void*                    descB,
                                const int32_t*                 modeB,
                                const void*                    A,
                                const void*                    B,
                                hiptensorAmdPermutationInfo_t* out);

/* logger control                                                     (hiptensor.hpp:308-343) */
typedef void (*hiptensorAmdLoggerCallback_t)(int32_t logContext, const char* funcName, const char* msg);
int hiptensorAmdLoggerSetCallback(hiptensorAmdLoggerCallback_t callback);
int hiptensorAmdLoggerOpenFile(const char* logFile);
int hiptensorAmdLoggerSetLevel(int level);
int hiptensorAmdLoggerSetMask(int32_t mask);
int hiptensorAmdLoggerForceDisable(void);
int hiptensorAmdGetHiprtVersion(void);

/* What a plan decided; for tests, benchmarks and logs.  No counterpart in the reference
 * (its plan exposes only a kernel pointer). */
typedef struct hiptensorAmdPlanInfo
{
    int64_t  P, Q, K;        /* folded GEMM view: rows, columns, reduction            */
    int32_t  swapped;        /* 1: rows come from B and columns from A                */
    int32_t  kernel_class;   /* HIPTK_* element class                                 */
    int32_t  tile_p, tile_q, tile_k, threads, lds_bytes;
    int32_t  split_k;
    int32_t  x_kfast, y_kfast, x_vec, y_vec, cd_vec;
    int32_t  n_pdims, n_qdims, n_kdims; /* dims left after fusion                     */
    uint64_t workspace_bytes;
    uint64_t kernel_uid;
    double   estimate_us;
    char     kernel_name[96];
    /* operands the plan first moves into a packed copy in the workspace (interleaved layouts
     * that would otherwise be gathered element by element); the view above is that of the copies */
    int32_t  pack_a, pack_b;
    uint64_t pack_bytes;     /* leading part of workspace_bytes that holds the copies  */
    char     pack_a_kernel[96], pack_b_kernel[96];
} hiptensorAmdPlanInfo_t;
int hiptensorAmdPlanInfo(const void* plan, hiptensorAmdPlanInfo_t* out);
/* Size of a handle's plan cache: `states` = plan states it holds (each owns its offset tables on the
 * device; one per distinct planning decision; beyond 4096 the least recently planned one that was never
 * executed is retired), `requests` = distinct planning requests (problem x workspace size ...) that map onto them.
 * No counterpart in the reference, whose plans point into process-wide singletons. */
int hiptensorAmdPlanCacheInfo(const void* handle, int64_t* states, int64_t* requests);
/* Keeps the plan's state (and its offset tables on the device) until hiptensorDestroy: the cache never
 * retires it.  The first execution of a plan does the same by itself, since from then on a captured
 * graph or a launch in another thread may read the tables; this call is for a caller that holds a
 * plan for later without having executed it.  Returns HIPTENSOR_STATUS_INTERNAL_ERROR for a plan whose
 * state was retired already.  No counterpart in the reference (its plans never expire). */
int hiptensorAmdPlanRetain(const void* plan);

/* Copies offset table `which` (0 xp, 1 xk, 2 yq, 3 yk, 4 cp, 5 cq, 6 dp, 7 dq; logical
 * length only, without padding) into out[0..cap); returns the logical length. */
int64_t hiptensorAmdPlanTable(const void* plan, int which, int32_t* out, int64_t cap);

#ifdef __cplusplus
}
#endif
#endif /* HIPTENSOR_AMD_H */
