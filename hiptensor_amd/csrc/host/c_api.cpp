// Flat C ABI: each function forwards to the C++ entry point of the same name.
#include <cstring>
#include <new>

#include <hiptensor/hiptensor.hpp>
#include <hiptensor_amd.h>

#include "handle.hpp"

namespace hipta
{
    hiptensorStatus_t createHostOnlyHandle(hiptensorHandle_t** handle);
    const PlanState*  planState(const hiptensorContractionPlan_t* plan);
    hiptensorStatus_t contractionNoAlloc(const hiptensorHandle_t*          handle,
                                         const hiptensorContractionPlan_t* plan,
                                         const void*                       alpha,
                                         const void*                       A,
                                         const void*                       B,
                                         const void*                       beta,
                                         const void*                       C,
                                         void*                             D,
                                         hipStream_t                       stream);
    hiptensorStatus_t planPermutation(const hiptensorTensorDescriptor_t* descA,
                                      const int32_t                      modeA[],
                                      const hiptensorTensorDescriptor_t* descB,
                                      const int32_t                      modeB[],
                                      const void*                        A,
                                      const void*                        B,
                                      hiptk_permute_t&                   out,
                                      bool&                              empty);
}

namespace
{
    template <typename T>
    T* fresh(void** slot)
    {
        if(!slot)
            return nullptr;
        T* p  = new(std::nothrow) T();
        *slot = p;
        return p;
    }

    template <typename T>
    int finish(hiptensorStatus_t st, void** slot, T* obj)
    {
        if(st != HIPTENSOR_STATUS_SUCCESS && slot && obj)
        {
            delete obj;
            *slot = nullptr;
        }
        return (int)st;
    }
}

extern "C" int hiptensorAmdCreate(void** handle)
{
    return (int)hiptensorCreate((hiptensorHandle_t**)handle);
}

extern "C" int hiptensorAmdCreateHostOnly(void** handle)
{
    return (int)hipta::createHostOnlyHandle((hiptensorHandle_t**)handle);
}

extern "C" int hiptensorAmdDestroy(void* handle)
{
    return (int)hiptensorDestroy((hiptensorHandle_t*)handle);
}

extern "C" int hiptensorAmdInitTensorDescriptor(const void*    handle,
                                                void**         desc,
                                                uint32_t       numModes,
                                                const int64_t* lens,
                                                const int64_t* strides,
                                                int            dataType,
                                                int            unaryOp)
{
    auto* d = fresh<hiptensorTensorDescriptor_t>(desc);
    return finish(hiptensorInitTensorDescriptor((const hiptensorHandle_t*)handle,
                                                d,
                                                numModes,
                                                lens,
                                                strides,
                                                (hipDataType)dataType,
                                                (hiptensorOperator_t)unaryOp),
                  desc,
                  d);
}

extern "C" int hiptensorAmdDestroyTensorDescriptor(void* desc)
{
    delete(hiptensorTensorDescriptor_t*)desc;
    return 0;
}

extern "C" const char* hiptensorAmdGetErrorString(int status)
{
    return hiptensorGetErrorString((hiptensorStatus_t)status);
}

extern "C" int hiptensorAmdGetAlignmentRequirement(const void* handle,
                                                   const void* ptr,
                                                   const void* desc,
                                                   uint32_t*   alignmentRequirement)
{
    return (int)hiptensorGetAlignmentRequirement(
        (const hiptensorHandle_t*)handle, ptr, (const hiptensorTensorDescriptor_t*)desc, alignmentRequirement);
}

extern "C" int hiptensorAmdInitContractionDescriptor(const void*    handle,
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
                                                     int            typeCompute)
{
    auto* d = fresh<hiptensorContractionDescriptor_t>(desc);
    return finish(hiptensorInitContractionDescriptor((const hiptensorHandle_t*)handle,
                                                     d,
                                                     (const hiptensorTensorDescriptor_t*)descA,
                                                     modeA,
                                                     alignmentRequirementA,
                                                     (const hiptensorTensorDescriptor_t*)descB,
                                                     modeB,
                                                     alignmentRequirementB,
                                                     (const hiptensorTensorDescriptor_t*)descC,
                                                     modeC,
                                                     alignmentRequirementC,
                                                     (const hiptensorTensorDescriptor_t*)descD,
                                                     modeD,
                                                     alignmentRequirementD,
                                                     (hiptensorComputeType_t)typeCompute),
                  desc,
                  d);
}

extern "C" int hiptensorAmdDestroyContractionDescriptor(void* desc)
{
    delete(hiptensorContractionDescriptor_t*)desc;
    return 0;
}

extern "C" int hiptensorAmdInitContractionFind(const void* handle, void** find, int algo)
{
    auto* f = fresh<hiptensorContractionFind_t>(find);
    return finish(hiptensorInitContractionFind((const hiptensorHandle_t*)handle, f, (hiptensorAlgo_t)algo), find, f);
}

extern "C" int hiptensorAmdDestroyContractionFind(void* find)
{
    delete(hiptensorContractionFind_t*)find;
    return 0;
}

extern "C" int hiptensorAmdContractionGetWorkspaceSize(
    const void* handle, const void* desc, const void* find, int pref, uint64_t* workspaceSize)
{
    return (int)hiptensorContractionGetWorkspaceSize((const hiptensorHandle_t*)handle,
                                                     (const hiptensorContractionDescriptor_t*)desc,
                                                     (const hiptensorContractionFind_t*)find,
                                                     (hiptensorWorksizePreference_t)pref,
                                                     workspaceSize);
}

extern "C" int hiptensorAmdInitContractionPlan(
    const void* handle, void** plan, const void* desc, const void* find, uint64_t workspaceSize)
{
    auto* p = fresh<hiptensorContractionPlan_t>(plan);
    if(p)
        p->mSolution = nullptr;
    return finish(hiptensorInitContractionPlan((const hiptensorHandle_t*)handle,
                                               p,
                                               (const hiptensorContractionDescriptor_t*)desc,
                                               (const hiptensorContractionFind_t*)find,
                                               workspaceSize),
                  plan,
                  p);
}

extern "C" int hiptensorAmdDestroyContractionPlan(void* plan)
{
    delete(hiptensorContractionPlan_t*)plan;
    return 0;
}

extern "C" int hiptensorAmdContraction(const void* handle,
                                       const void* plan,
                                       const void* alpha,
                                       const void* A,
                                       const void* B,
                                       const void* beta,
                                       const void* C,
                                       void*       D,
                                       void*       workspace,
                                       uint64_t    workspaceSize,
                                       void*       stream)
{
    return (int)hiptensorContraction((const hiptensorHandle_t*)handle,
                                     (const hiptensorContractionPlan_t*)plan,
                                     alpha,
                                     A,
                                     B,
                                     beta,
                                     C,
                                     D,
                                     workspace,
                                     workspaceSize,
                                     (hipStream_t)stream);
}

extern "C" int hiptensorAmdContractionNoAlloc(const void* handle,
                                              const void* plan,
                                              const void* alpha,
                                              const void* A,
                                              const void* B,
                                              const void* beta,
                                              const void* C,
                                              void*       D,
                                              void*       stream)
{
    return (int)hipta::contractionNoAlloc((const hiptensorHandle_t*)handle,
                                          (const hiptensorContractionPlan_t*)plan,
                                          alpha,
                                          A,
                                          B,
                                          beta,
                                          C,
                                          D,
                                          (hipStream_t)stream);
}

extern "C" int hiptensorAmdPermutation(const void*    handle,
                                       const void*    alpha,
                                       const void*    A,
                                       const void*    descA,
                                       const int32_t* modeA,
                                       void*          B,
                                       const void*    descB,
                                       const int32_t* modeB,
                                       int            typeScalar,
                                       void*          stream)
{
    return (int)hiptensorPermutation((const hiptensorHandle_t*)handle,
                                     alpha,
                                     A,
                                     (const hiptensorTensorDescriptor_t*)descA,
                                     modeA,
                                     B,
                                     (const hiptensorTensorDescriptor_t*)descB,
                                     modeB,
                                     (hipDataType)typeScalar,
                                     (hipStream_t)stream);
}

extern "C" int hiptensorAmdPermutationInfo(const void*                    descA,
                                           const int32_t*                 modeA,
                                           const void*                    descB,
                                           const int32_t*                 modeB,
                                           const void*                    A,
                                           const void*                    B,
                                           hiptensorAmdPermutationInfo_t* out)
{
    if(!descA || !modeA || !descB || !modeB || !out)
        return (int)HIPTENSOR_STATUS_NOT_INITIALIZED;
    const auto* dA = (const hiptensorTensorDescriptor_t*)descA;
    const auto* dB = (const hiptensorTensorDescriptor_t*)descB;
    std::memset(out, 0, sizeof(*out));
    hiptk_permute_t p;
    bool            empty = false;
    auto            st    = hipta::planPermutation(dA, modeA, dB, modeB, A, B, p, empty);
    if(st != HIPTENSOR_STATUS_SUCCESS)
        return (int)st;
    out->fused_rank = p.rank;
    for(int d = 0; d < 6; ++d)
    {
        out->extent[d]   = p.extent[d];
        out->a_stride[d] = p.a_stride[d];
        out->b_stride[d] = p.b_stride[d];
    }
    out->kernel = p.kernel;
    out->mode_i = p.mode_i;
    out->mode_j = p.mode_j;
    out->tile   = p.tile;
    out->vec_r  = p.vec_r;
    out->vec_w  = p.vec_w;
    out->empty  = empty ? 1 : 0;
    if(!empty)
        std::strncpy(out->kernel_name, hiptk_permute_kernel_name(&p), sizeof(out->kernel_name) - 1);
    return 0;
}

extern "C" int hiptensorAmdLoggerSetCallback(hiptensorAmdLoggerCallback_t callback)
{
    return (int)hiptensorLoggerSetCallback((hiptensorLoggerCallback_t)callback);
}
extern "C" int hiptensorAmdLoggerOpenFile(const char* logFile) { return (int)hiptensorLoggerOpenFile(logFile); }
extern "C" int hiptensorAmdLoggerSetLevel(int level) { return (int)hiptensorLoggerSetLevel((hiptensorLogLevel_t)level); }
extern "C" int hiptensorAmdLoggerSetMask(int32_t mask) { return (int)hiptensorLoggerSetMask(mask); }
extern "C" int hiptensorAmdLoggerForceDisable(void) { return (int)hiptensorLoggerForceDisable(); }
extern "C" int hiptensorAmdGetHiprtVersion(void) { return hiptensorGetHiprtVersion(); }

extern "C" int hiptensorAmdPlanInfo(const void* plan, hiptensorAmdPlanInfo_t* out)
{
    const hipta::PlanState* st = hipta::planState((const hiptensorContractionPlan_t*)plan);
    if(!st || !out)
        return (int)HIPTENSOR_STATUS_NOT_INITIALIZED;
    std::memset(out, 0, sizeof(*out));
    const hipta::GemmView& v = st->view;
    out->P                   = v.P;
    out->Q                   = v.Q;
    out->K                   = v.K;
    out->swapped             = v.swapped ? 1 : 0;
    out->kernel_class        = v.cls;
    out->tile_p              = st->sol->bp;
    out->tile_q              = st->sol->bq;
    out->tile_k              = st->sol->bk;
    out->threads             = st->sol->threads;
    out->lds_bytes           = st->sol->lds_bytes;
    out->split_k             = st->prob.split_k;
    out->x_kfast             = v.x_kfast;
    out->y_kfast             = v.y_kfast;
    out->x_vec               = v.x_vec;
    out->y_vec               = v.y_vec;
    out->cd_vec              = v.cd_vec;
    out->n_pdims             = (int32_t)v.pdims.size();
    out->n_qdims             = (int32_t)v.qdims.size();
    out->n_kdims             = (int32_t)v.kdims.size();
    out->workspace_bytes     = st->ws_bytes;
    out->kernel_uid          = st->sol->uid;
    out->estimate_us         = st->est_us;
    std::strncpy(out->kernel_name, st->kernel_name.c_str(), sizeof(out->kernel_name) - 1);
    out->pack_a     = st->pack_a.on ? 1 : 0;
    out->pack_b     = st->pack_b.on ? 1 : 0;
    out->pack_bytes = st->pack_bytes;
    if(st->pack_a.on)
        std::strncpy(out->pack_a_kernel, hiptk_permute_kernel_name(&st->pack_a.perm), sizeof(out->pack_a_kernel) - 1);
    if(st->pack_b.on)
        std::strncpy(out->pack_b_kernel, hiptk_permute_kernel_name(&st->pack_b.perm), sizeof(out->pack_b_kernel) - 1);
    return 0;
}

extern "C" int hiptensorAmdPlanRetain(const void* plan)
{
    if(!plan)
        return (int)HIPTENSOR_STATUS_NOT_INITIALIZED;
    const hipta::PlanState* st = (const hipta::PlanState*)((const hiptensorContractionPlan_t*)plan)->mSolution;
    if(!st)
        return (int)HIPTENSOR_STATUS_NOT_INITIALIZED;
    return hipta::Handle::pin(st) ? 0 : (int)HIPTENSOR_STATUS_INTERNAL_ERROR;
}

extern "C" int hiptensorAmdPlanCacheInfo(const void* handle, int64_t* states, int64_t* requests)
{
    if(!handle)
        return (int)HIPTENSOR_STATUS_NOT_INITIALIZED;
    hipta::Handle* h = hipta::Handle::from(((const hiptensorHandle_t*)handle)->fields);
    if(!h)
        return (int)HIPTENSOR_STATUS_NOT_INITIALIZED;
    if(states)
        *states = (int64_t)h->planCount();
    if(requests)
        *requests = (int64_t)h->aliasCount();
    return 0;
}

extern "C" int64_t hiptensorAmdPlanTable(const void* plan, int which, int32_t* out, int64_t cap)
{
    const hipta::PlanState* st = hipta::planState((const hiptensorContractionPlan_t*)plan);
    if(!st || which < 0 || which > 7)
        return -1;
    const hipta::GemmView&      v       = st->view;
    const std::vector<int32_t>* tabs[8] = {&v.xp, &v.xk, &v.yq, &v.yk, &v.cp, &v.cq, &v.dp, &v.dq};
    const int64_t               lens[8] = {v.P, v.K, v.Q, v.K, v.P, v.Q, v.P, v.Q};
    const int64_t               n       = tabs[which]->empty() ? 0 : lens[which];
    for(int64_t i = 0; i < n && i < cap && out; i++)
        out[i] = (*tabs[which])[(size_t)i];
    return n;
}
