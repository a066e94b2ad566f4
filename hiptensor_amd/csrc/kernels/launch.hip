// Kernel-layer C ABI: kernel registry lookup, argument checks, launch, and the
// split-K reduction kernels.
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

#include "contract_h.hpp"
#include "contract_w.hpp"
#include "dma_lds.hpp"

namespace hiptk
{
    namespace
    {
        struct Registry
        {
            std::vector<KernelEntry> all;
            Registry()
            {
                typedef const KernelEntry* (*src_fn)(int*);
                const src_fn sources[] = {entries_f16_hd,
                                          entries_f16_hd192,
                                          entries_f16_hd192_tab,
                                          entries_bf16_hd,
                                          entries_bf16_hd192,
                                          entries_bf16_hd192_tab,
                                          entries_f16_hk_kx,
                                          entries_f16_hk_rx,
                                          entries_bf16_hk_kx,
                                          entries_bf16_hk_rx,
                                          entries_f16_hr192_kx,
                                          entries_f16_hr192_rx,
                                          entries_bf16_hr192_kx,
                                          entries_bf16_hr192_rx,
                                          entries_f16_aff,
                                          entries_bf16_aff,
                                          entries_f16_vec,
                                          entries_f16_gen,
                                          entries_bf16_vec,
                                          entries_bf16_gen,
                                          entries_f16_v4,
                                          entries_f16_v2,
                                          entries_bf16_v4,
                                          entries_bf16_v2,
                                          entries_f32,
                                          entries_f64,
                                          entries_c32,
                                          entries_c64,
                                          entries_f64_as_f32,
                                          entries_f32_as_f16,
                                          entries_f32_as_bf16};
                for(src_fn f : sources)
                {
                    int                n = 0;
                    const KernelEntry* e = f(&n);
                    all.insert(all.end(), e, e + n);
                }
            }
        };

        const Registry& registry()
        {
            static const Registry r;
            return r;
        }

        int acc_bytes(int cls)
        {
            switch(cls)
            {
            case HIPTK_F64: return 8;
            case HIPTK_C32: return 8;
            case HIPTK_C64: return 16;
            default: return 4;
            }
        }

        // bytes of one operand element in memory
        int operand_bytes(int cls)
        {
            switch(cls)
            {
            case HIPTK_F16:
            case HIPTK_BF16: return 2;
            case HIPTK_F64:
            case HIPTK_F64_AS_F32:
            case HIPTK_C32: return 8;
            case HIPTK_C64: return 16;
            default: return 4;
            }
        }

        // ---- split-K reduction: sum the partials in slice order, apply alpha / beta ----

        struct FinF16
        {
            typedef float    O;
            typedef uint16_t E;
            static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
            {
                float v = (float)al[0] * x;
                if(bil)
                    v += (float)be[0] * TraitsF16::to_f32(*c);
                return TraitsF16::from_f32(v);
            }
            static __device__ inline O add(O a, O b) { return a + b; }
        };

        struct FinBF16
        {
            typedef float    O;
            typedef uint16_t E;
            static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
            {
                float v = (float)al[0] * x;
                if(bil)
                    v += (float)be[0] * TraitsBF16::to_f32(*c);
                return TraitsBF16::from_f32(v);
            }
            static __device__ inline O add(O a, O b) { return a + b; }
        };

        template <typename Tr>
        struct FinWide
        {
            typedef typename Tr::O O;
            typedef typename Tr::E E;
            static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
            {
                return Tr::finish(x, al, be, bil, c);
            }
            static __device__ inline float   add(float a, float b) { return a + b; }
            static __device__ inline double  add(double a, double b) { return a + b; }
            static __device__ inline float2  add(float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); }
            static __device__ inline double2 add(double2 a, double2 b)
            {
                return make_double2(a.x + b.x, a.y + b.y);
            }
        };

        template <typename Fin>
        __global__ void __launch_bounds__(256) splitk_reduce_kernel(const KArgs a)
        {
            typedef typename Fin::O O;
            typedef typename Fin::E E;
            const size_t total = (size_t)a.P * (size_t)a.Q;
            const size_t idx   = (size_t)blockIdx.x * 256 + threadIdx.x;
            if(idx >= total)
                return;
            const int p  = (int)(idx / (size_t)a.Q);
            const int q  = (int)(idx % (size_t)a.Q);
            const O*  ws = (const O*)a.ws;
            O         s  = ws[idx];
            for(int z = 1; z < a.split_k; z++)
                s = Fin::add(s, ws[(size_t)z * total + idx]);
            const bool bil = a.bilinear != 0;
            const E*   c   = bil ? (const E*)a.C + ((uint32_t)a.cp[p] + (uint32_t)a.cq[q]) : nullptr;
            ((E*)a.D)[(uint32_t)a.dp[p] + (uint32_t)a.dq[q]] = Fin::finish(s, a.alpha, a.beta, bil, c);
        }

        template <typename Fin>
        int launch_reduce(const KArgs& a, hipStream_t stream)
        {
            const size_t total  = (size_t)a.P * (size_t)a.Q;
            const size_t blocks = (total + 255) / 256;
            hipLaunchKernelGGL(splitk_reduce_kernel<Fin>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
            return (int)hipGetLastError();
        }

        int reduce_dispatch(int cls, const KArgs& a, hipStream_t stream)
        {
            switch(cls)
            {
            case HIPTK_F16: return launch_reduce<FinF16>(a, stream);
            case HIPTK_BF16: return launch_reduce<FinBF16>(a, stream);
            case HIPTK_F32:
            case HIPTK_F32_AS_F16:
            case HIPTK_F32_AS_BF16: return launch_reduce<FinWide<WTraitsF32>>(a, stream);
            case HIPTK_F64: return launch_reduce<FinWide<WTraitsF64>>(a, stream);
            case HIPTK_C32: return launch_reduce<FinWide<WTraitsC32>>(a, stream);
            case HIPTK_C64: return launch_reduce<FinWide<WTraitsC64>>(a, stream);
            case HIPTK_F64_AS_F32: return launch_reduce<FinWide<WTraitsF64AsF32>>(a, stream);
            default: return (int)hipErrorInvalidValue;
            }
        }

        // The affine-K variant is preferred when the problem allows it; the table variant
        // serves every problem.
        const KernelEntry* find_entry(const hiptk_problem_t* p)
        {
            const KernelEntry* table = nullptr;
            for(const KernelEntry& e : registry().all)
            {
                if(e.cls == p->cls && e.tile_id == p->tile_id && e.x_kfast == (p->x_kfast != 0)
                   && e.y_kfast == (p->y_kfast != 0) && e.x_vec == p->x_vec && e.y_vec == p->y_vec)
                {
                    // a tile can only be moved back to end at P / Q if it fits into P / Q
                    if((p->shift_p && p->P < e.bp) || (p->shift_q && p->Q < e.bq))
                        continue;
                    // the direct-load kernels: a restricted K tail, vectors on 16-byte multiples
                    if(e.k_multiple > 0 && (p->K % e.k_multiple != 0 || p->K < e.bk || !p->xy_aligned))
                        continue;
                    // ... and they address an operand with 32-bit byte offsets
                    if(e.k_multiple > 0)
                    {
                        const uint64_t eb   = (uint64_t)operand_bytes(p->cls);
                        const int32_t  most = p->x_max_off > p->y_max_off ? p->x_max_off : p->y_max_off;
                        // (less the bias some of them keep in a lane's offset so that loads can share a write of M0)
                        if(most < 0 || ((uint64_t)most + 16 / eb) * eb > 0xFFFFFFFFull - (uint64_t)DMA_BIAS)
                            continue;
                    }
                    if(e.k_affine && p->k_affine)
                        return &e;
                    if(!e.k_affine && !table)
                        table = &e;
                }
            }
            return table;
        }

        // The largest register-staged tile of the problem's class and layout: what runs in place of
        // a direct-load kernel when an operand's base address is not 16-byte aligned.
        const KernelEntry* staged_entry(const hiptk_problem_t* p)
        {
            const KernelEntry* best = nullptr;
            hiptk_problem_t    q    = *p;
            for(const KernelEntry& t : registry().all)
            {
                if(t.cls != p->cls || t.k_multiple > 0)
                    continue;
                q.tile_id            = t.tile_id;
                const KernelEntry* e = find_entry(&q);
                if(e && e->k_multiple == 0
                   && (!best || e->bp * e->bq > best->bp * best->bq
                       || (e->bp * e->bq == best->bp * best->bq && e->threads > best->threads)))
                    best = e;
            }
            return best;
        }

        // The entry a launch with these operand addresses runs: the resolved one where the plan
        // resolved it (and the problem still is the one it was resolved for), else a search.
        const KernelEntry* entry_for(const hiptk_problem_t* p, const void* X, const void* Y)
        {
            const KernelEntry* e = (const KernelEntry*)p->kernel;
            const bool         resolved = e && e->cls == p->cls && e->tile_id == p->tile_id && e->x_kfast == (p->x_kfast != 0)
                                  && e->y_kfast == (p->y_kfast != 0) && e->x_vec == p->x_vec && e->y_vec == p->y_vec;
            if(!resolved)
                e = find_entry(p);
            if(e && e->k_multiple > 0 && ((((uintptr_t)X) | ((uintptr_t)Y)) & 15) != 0)
                e = resolved ? (const KernelEntry*)p->kernel_unaligned : staged_entry(p);
            return e;
        }
    }
}

extern "C" int hiptk_resolve(hiptk_problem_t* prob)
{
    if(!prob)
        return HIPTK_ERR_ARG;
    const hiptk::KernelEntry* e = hiptk::find_entry(prob);
    prob->kernel                = e;
    prob->kernel_unaligned      = (e && e->k_multiple > 0) ? hiptk::staged_entry(prob) : e;
    return e ? HIPTK_OK : HIPTK_ERR_NO_KERNEL;
}

extern "C" const char* hiptk_kernel_name_at(const hiptk_problem_t* prob, const void* X, const void* Y)
{
    const hiptk::KernelEntry* e = prob ? hiptk::entry_for(prob, X, Y) : nullptr;
    return e ? e->name : "";
}

extern "C" int hiptk_tile_count(int cls)
{
    int n = 0;
    for(const hiptk::KernelEntry& e : hiptk::registry().all)
        if(e.cls == cls && e.tile_id + 1 > n)
            n = e.tile_id + 1;
    return n;
}

extern "C" int hiptk_tile_info(int cls, int tile_id, hiptk_tile_info_t* out)
{
    if(!out)
        return HIPTK_ERR_ARG;
    for(const hiptk::KernelEntry& e : hiptk::registry().all)
    {
        if(e.cls == cls && e.tile_id == tile_id)
        {
            out->tile_id   = tile_id;
            out->bp        = e.bp;
            out->bq        = e.bq;
            out->bk        = e.bk;
            out->threads   = e.threads;
            out->lds_bytes = e.lds_bytes;
            out->k_multiple = e.k_multiple;
            out->mfma_k     = e.mfma_k;
            std::snprintf(out->name, sizeof(out->name), "cls%d_%dx%dx%d", cls, e.bp, e.bq, e.bk);
            return HIPTK_OK;
        }
    }
    return HIPTK_ERR_NO_KERNEL;
}

extern "C" int hiptk_kernel_available(const hiptk_problem_t* prob)
{
    return (prob && hiptk::find_entry(prob)) ? 1 : 0;
}

extern "C" const char* hiptk_kernel_name(const hiptk_problem_t* prob)
{
    const hiptk::KernelEntry* e = prob ? hiptk::find_entry(prob) : nullptr;
    return e ? e->name : "";
}

extern "C" uint64_t hiptk_workspace_bytes(const hiptk_problem_t* prob)
{
    if(!prob || prob->split_k <= 1)
        return 0;
    return (uint64_t)prob->split_k * (uint64_t)prob->P * (uint64_t)prob->Q
           * (uint64_t)hiptk::acc_bytes(prob->cls);
}

extern "C" int hiptk_contract(const hiptk_problem_t* prob,
                              const void*            alpha,
                              const void*            beta,
                              const void*            X,
                              const void*            Y,
                              const void*            C,
                              void*                  D,
                              void*                  workspace,
                              uint64_t               workspace_bytes,
                              void*                  stream,
                              int*                   hip_error)
{
    using namespace hiptk;
    if(hip_error)
        *hip_error = 0;
    if(!prob || !alpha || !X || !Y || !D)
        return HIPTK_ERR_ARG;
    if(prob->P <= 0 || prob->Q <= 0 || prob->K <= 0 || prob->P > 0x7FFFFF00ll || prob->Q > 0x7FFFFF00ll
       || prob->K > 0x7FFFFF00ll || prob->split_k < 1)
        return HIPTK_ERR_ARG;
    if(!prob->xp || !prob->xk || !prob->yq || !prob->yk || !prob->dp || !prob->dq)
        return HIPTK_ERR_ARG;
    const bool bil = prob->op == HIPTK_OP_BILINEAR;
    if(bil && (!C || !beta || !prob->cp || !prob->cq))
        return HIPTK_ERR_ARG;
    const KernelEntry* e = entry_for(prob, X, Y);
    if(!e)
        return HIPTK_ERR_NO_KERNEL;

    KArgs a;
    std::memset(&a, 0, sizeof(a));
    a.X  = X;
    a.Y  = Y;
    a.C  = C;
    a.D  = D;
    a.ws = workspace;
    a.xp = prob->xp;
    a.xk = prob->xk;
    a.yq = prob->yq;
    a.yk = prob->yk;
    a.cp = prob->cp;
    a.cq = prob->cq;
    a.dp = prob->dp;
    a.dq = prob->dq;
    a.P  = (int32_t)prob->P;
    a.Q  = (int32_t)prob->Q;
    a.K  = (int32_t)prob->K;
    a.bilinear  = bil ? 1 : 0;
    a.cd_affine = prob->cd_affine;
    a.dp_stride = prob->dp_stride;
    a.dq_stride = prob->dq_stride;
    a.cp_stride = prob->cp_stride;
    a.cq_stride = prob->cq_stride;
    a.xp_stride = prob->cd_affine ? prob->xp_stride : 0;
    a.yq_stride = prob->cd_affine ? prob->yq_stride : 0;
    a.xk_stride = prob->xk_stride;
    a.yk_stride = prob->yk_stride;
    a.cd_vec    = prob->cd_vec;
    a.shift_p   = prob->shift_p ? 1 : 0;
    a.shift_q   = prob->shift_q ? 1 : 0;
    {
        // byte offset of the last 16-byte vector of X / Y (the class's own element size)
        const int32_t eb = operand_bytes(prob->cls), back = 16 / eb - 1;
        a.x_last_vec     = prob->x_max_off >= back ? (uint32_t)eb * (uint32_t)(prob->x_max_off - back) : 0u;
        a.y_last_vec     = prob->y_max_off >= back ? (uint32_t)eb * (uint32_t)(prob->y_max_off - back) : 0u;
    }
    a.x_chunked = (prob->x_kfast && prob->x_rows_adjacent) ? 1 : 0;
    a.y_chunked = (prob->y_kfast && prob->y_rows_adjacent) ? 1 : 0;
    // A moved-back tile stores whole 8-element vectors of D that reach into its neighbour's
    // columns (same values).  When D is updated in place (C == D) the neighbour's elements must
    // not be read and written twice, so that case stores element by element.
    if(a.shift_q && bil && C == D && prob->Q % 8 != 0)
        a.cd_vec = 1;
    a.tiles_p  = (int32_t)((prob->P + e->bp - 1) / e->bp);
    a.tiles_q  = (int32_t)((prob->Q + e->bq - 1) / e->bq);
    const int ktiles = (int)((prob->K + e->bk - 1) / e->bk);
    int       split  = prob->split_k;
    if(split > ktiles)
        split = ktiles;
    a.ktiles_per_split = (ktiles + split - 1) / split;
    split              = (ktiles + a.ktiles_per_split - 1) / a.ktiles_per_split; // no empty slice
    a.split_k          = split;
    if((uint64_t)a.tiles_p * (uint64_t)a.tiles_q > 0x7FFFFFFFull || split > 65535)
        return HIPTK_ERR_ARG;

    switch(prob->cls)
    {
    case HIPTK_C32:
        a.alpha[0] = ((const float*)alpha)[0];
        a.alpha[1] = ((const float*)alpha)[1];
        if(beta)
        {
            a.beta[0] = ((const float*)beta)[0];
            a.beta[1] = ((const float*)beta)[1];
        }
        break;
    case HIPTK_C64:
        a.alpha[0] = ((const double*)alpha)[0];
        a.alpha[1] = ((const double*)alpha)[1];
        if(beta)
        {
            a.beta[0] = ((const double*)beta)[0];
            a.beta[1] = ((const double*)beta)[1];
        }
        break;
    case HIPTK_F64:
    case HIPTK_F64_AS_F32:
        a.alpha[0] = *(const double*)alpha;
        if(beta)
            a.beta[0] = *(const double*)beta;
        break;
    default:
        a.alpha[0] = *(const float*)alpha;
        if(beta)
            a.beta[0] = *(const float*)beta;
        break;
    }

    if(split > 1)
    {
        const uint64_t need
            = (uint64_t)split * (uint64_t)prob->P * (uint64_t)prob->Q * (uint64_t)acc_bytes(prob->cls);
        if(!workspace || workspace_bytes < need)
            return HIPTK_ERR_WORKSPACE;
    }

    hipStream_t s  = (hipStream_t)stream;
    int         rc = e->launch(a, s);
    if(rc == 0 && split > 1)
        rc = reduce_dispatch(prob->cls, a, s);
    if(rc != 0)
    {
        if(hip_error)
            *hip_error = rc;
        return HIPTK_ERR_LAUNCH;
    }
    return HIPTK_OK;
}

// ---- a workspace that lives in the library, for callers that cannot allocate ----
//
// Device memory of a fixed, modest size that every device the library runs on holds until the
// process ends.  In host code the array's name is only a stand-in (passing it to a kernel would
// hand the kernel a host-side address); its device address is looked up once per device with
// hipGetSymbolAddress, with that device current, and from then on only that address is used.
static __device__ __align__(256) unsigned char scratch[HIPTK_STATIC_WORKSPACE_BYTES];

namespace
{
    constexpr int MAX_DEVICES = 64;
    std::mutex    g_scratch_lock;
    void*         g_scratch_ptr[MAX_DEVICES] = {};
}

extern "C" int hiptk_static_workspace(void** ptr, uint64_t* bytes, int* hip_error)
{
    if(hip_error)
        *hip_error = 0;
    if(!ptr || !bytes)
        return HIPTK_ERR_ARG;
    *ptr   = nullptr;
    *bytes = 0;
    int        dev = -1;
    hipError_t e   = hipGetDevice(&dev);
    if(e != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
    {
        if(hip_error)
            *hip_error = (int)e;
        return HIPTK_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if(!g_scratch_ptr[dev])
    {
        void* p = nullptr;
        e       = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if(e != hipSuccess || !p)
        {
            if(hip_error)
                *hip_error = (int)e;
            return HIPTK_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = p;
    }
    *ptr   = g_scratch_ptr[dev];
    *bytes = HIPTK_STATIC_WORKSPACE_BYTES;
    return HIPTK_OK;
}
