// 32/64-bit contraction kernels for gfx950: f32, f64, complex f32, complex f64 and
// f64 storage computed in f32.
//
//   acc[p][q] = sum_k X[xp[p] + xk[k]] * Y[yq[q] + yk[k]]
//   D[dp[p] + dq[q]] = alpha * acc (+ beta * C[cp[p] + cq[q]])
//
// These MFMA shapes take one element per lane per operand (v_mfma_f32_32x32x2_f32:
// lane l supplies row l % 32 at k = l / 32; v_mfma_f64_16x16x4_f64: row l % 16 at
// k = l / 16), so both operand tiles live in LDS as tile[k][row + pad] and a lane's
// operand is one ds_read of consecutive rows across lanes: conflict free.
//
// Complex products use the same real MFMA with a lane's (re, im) pair as two operands:
//   RR += xr . yr    II += xi . yi    IM += xr . yi + xi . yr      Re = RR - II, Im = IM
// (the MFMA's k-slots hold consecutive complex k), so a complex tile costs two MFMAs per
// complex k: all four real products of every complex multiply run on the matrix core,
// none is wasted, nothing is selected or negated between the MFMAs, and there is no split
// into separate re/im arrays.
//
// Result layouts (verified on hardware):
//   32x32: lane l, register r -> p = 8 * (r / 4) + 4 * (l / 32) + r % 4, q = l % 32
//   f64 16x16: lane l, register r -> p = 4 * r + l / 16, q = l % 16
#pragma once
#include "kargs.h"

namespace hiptk
{
    typedef float  wf32x16_t __attribute__((ext_vector_type(16)));
    typedef double wf64x4_t __attribute__((ext_vector_type(4)));

    enum
    {
        GATHER_MN_VEC  = 0, // vectors of VMAX along the row index
        GATHER_K_VEC   = 1, // vectors of VMAX along k
        GATHER_SCALAR  = 2,
        GATHER_MN_HALF = 3, // vectors of VMAX / 2 along the row index (8 bytes of f32: runs that are a multiple of 2, not of 4)
        GATHER_K_HALF  = 4 // ... along k
    };

    // ---- per-class traits -------------------------------------------------------

    struct WTraitsF32
    {
        static constexpr int CLS = HIPTK_F32;
        typedef float        E; // storage element
        typedef float        S; // element as staged in LDS
        typedef float        XF;
        typedef float        YF;
        typedef float        O; // accumulator element written to split-K workspace
        static constexpr int TILE = 32, KM = 2, NREG = 16, VMAX = 4;
        struct Acc
        {
            wf32x16_t v;
        };
        static __device__ inline S    stage(E e) { return e; }
        static __device__ inline int  kslot(int lane) { return lane >> 5; }
        static __device__ inline XF   prep_x(S s, int) { return s; }
        static __device__ inline YF   prep_y(S s, int) { return s; }
        static __device__ inline void zero(Acc& a)
        {
#pragma unroll
            for(int r = 0; r < 16; r++)
                a.v[r] = 0.f;
        }
        static __device__ inline void mma(XF x, YF y, Acc& a)
        {
            a.v = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, a.v, 0, 0, 0);
        }
        static __device__ inline int p_of(int r, int lane)
        {
            return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        }
        static __device__ inline int q_of(int lane) { return lane & 31; }
        static __device__ inline O   get(const Acc& a, int r) { return a.v[r]; }
        static __device__ inline void put(Acc& a, int r, O x) { a.v[r] = x; }
        // alpha * x + beta * c with separately rounded products, as the CPU path does.
        static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
        {
            float y = __fmul_rn((float)al[0], x);
            if(bil)
                y = __fadd_rn(y, __fmul_rn((float)be[0], *c));
            return y;
        }
    };

    struct WTraitsF64
    {
        static constexpr int CLS = HIPTK_F64;
        typedef double       E;
        typedef double       S;
        typedef double       XF;
        typedef double       YF;
        typedef double       O;
        static constexpr int TILE = 16, KM = 4, NREG = 4, VMAX = 2;
        struct Acc
        {
            wf64x4_t v;
        };
        static __device__ inline S    stage(E e) { return e; }
        static __device__ inline int  kslot(int lane) { return lane >> 4; }
        static __device__ inline XF   prep_x(S s, int) { return s; }
        static __device__ inline YF   prep_y(S s, int) { return s; }
        static __device__ inline void zero(Acc& a)
        {
#pragma unroll
            for(int r = 0; r < 4; r++)
                a.v[r] = 0.0;
        }
        static __device__ inline void mma(XF x, YF y, Acc& a)
        {
            a.v = __builtin_amdgcn_mfma_f64_16x16x4f64(x, y, a.v, 0, 0, 0);
        }
        static __device__ inline int p_of(int r, int lane) { return 4 * r + (lane >> 4); }
        static __device__ inline int q_of(int lane) { return lane & 15; }
        static __device__ inline O   get(const Acc& a, int r) { return a.v[r]; }
        static __device__ inline void put(Acc& a, int r, O x) { a.v[r] = x; }
        // alpha and beta are narrowed to float first: the reference's Bilinear / Scale
        // functors hold them as float even for f64 data.
        static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
        {
            double y = __dmul_rn((double)(float)al[0], x);
            if(bil)
                y = __dadd_rn(y, __dmul_rn((double)(float)be[0], *c));
            return y;
        }
    };

    // f64 storage, inputs narrowed to f32 when staged, f32 MFMA, f32 accumulate.
    struct WTraitsF64AsF32 : WTraitsF32
    {
        static constexpr int CLS = HIPTK_F64_AS_F32;
        typedef double       E;
        static constexpr int VMAX = 2;
        static __device__ inline S stage(E e) { return (float)e; }
        static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
        {
            double y = __dmul_rn((double)(float)al[0], (double)x);
            if(bil)
                y = __dadd_rn(y, __dmul_rn((double)(float)be[0], *c));
            return y;
        }
    };

    struct WTraitsC32
    {
        static constexpr int CLS = HIPTK_C32;
        typedef float2       E;
        typedef float2       S;
        typedef float2       XF;
        typedef float2       YF;
        typedef float2       O;
        static constexpr int TILE = 32, KM = 2, NREG = 16, VMAX = 2;
        // The two k-slots of the MFMA hold two consecutive complex k, and a lane's (re, im) pair is an
        // operand as it is: Re(x y) accumulates as sum(xr yr) - sum(xi yi) in two chains that are
        // subtracted once at the end, Im(x y) as sum(xr yi + xi yr) in a third.  Four MFMAs per two
        // complex k (8 real flop per complex multiply-add, none wasted) and no selects or negations
        // between them, which at three VALU instructions per two MFMAs of the same wave cost a fifth
        // of the rate (1024 x 1024 x 512: 47.8 -> 39.3 us).
        struct Acc
        {
            wf32x16_t rr, ii, im;
        };
        static __device__ inline S    stage(E e) { return e; }
        static __device__ inline int  kslot(int lane) { return lane >> 5; }
        static __device__ inline XF   prep_x(S s, int) { return s; }
        static __device__ inline YF   prep_y(S s, int) { return s; }
        static __device__ inline void zero(Acc& a)
        {
#pragma unroll
            for(int r = 0; r < 16; r++)
            {
                a.rr[r] = 0.f;
                a.ii[r] = 0.f;
                a.im[r] = 0.f;
            }
        }
        static __device__ inline void mma(XF x, YF y, Acc& a)
        {
            a.rr = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, y.x, a.rr, 0, 0, 0);
            a.im = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, y.y, a.im, 0, 0, 0);
            a.ii = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, y.y, a.ii, 0, 0, 0);
            a.im = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, y.x, a.im, 0, 0, 0);
        }
        static __device__ inline int p_of(int r, int lane)
        {
            return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        }
        static __device__ inline int q_of(int lane) { return lane & 31; }
        static __device__ inline O   get(const Acc& a, int r) { return make_float2(__fsub_rn(a.rr[r], a.ii[r]), a.im[r]); }
        static __device__ inline void put(Acc& a, int r, O x)
        {
            a.rr[r] = x.x;
            a.ii[r] = 0.f;
            a.im[r] = x.y;
        }
        static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
        {
            const float ar = (float)al[0], ai = (float)al[1];
            float       yr = __fsub_rn(__fmul_rn(ar, x.x), __fmul_rn(ai, x.y));
            float       yi = __fadd_rn(__fmul_rn(ai, x.x), __fmul_rn(ar, x.y));
            if(bil)
            {
                const float  br = (float)be[0], bi = (float)be[1];
                const float2 cv = *c;
                yr = __fadd_rn(yr, __fsub_rn(__fmul_rn(br, cv.x), __fmul_rn(bi, cv.y)));
                yi = __fadd_rn(yi, __fadd_rn(__fmul_rn(bi, cv.x), __fmul_rn(br, cv.y)));
            }
            return make_float2(yr, yi);
        }
    };

    struct WTraitsC64
    {
        static constexpr int CLS = HIPTK_C64;
        typedef double2      E;
        typedef double2      S;
        typedef double2      XF;
        typedef double2      YF;
        typedef double2      O;
        static constexpr int TILE = 16, KM = 4, NREG = 4, VMAX = 1;
        // (as complex f32: the four k-slots hold four consecutive complex k, three chains)
        struct Acc
        {
            wf64x4_t rr, ii, im;
        };
        static __device__ inline S    stage(E e) { return e; }
        static __device__ inline int  kslot(int lane) { return lane >> 4; }
        static __device__ inline XF   prep_x(S s, int) { return s; }
        static __device__ inline YF   prep_y(S s, int) { return s; }
        static __device__ inline void zero(Acc& a)
        {
#pragma unroll
            for(int r = 0; r < 4; r++)
            {
                a.rr[r] = 0.0;
                a.ii[r] = 0.0;
                a.im[r] = 0.0;
            }
        }
        static __device__ inline void mma(XF x, YF y, Acc& a)
        {
            a.rr = __builtin_amdgcn_mfma_f64_16x16x4f64(x.x, y.x, a.rr, 0, 0, 0);
            a.im = __builtin_amdgcn_mfma_f64_16x16x4f64(x.x, y.y, a.im, 0, 0, 0);
            a.ii = __builtin_amdgcn_mfma_f64_16x16x4f64(x.y, y.y, a.ii, 0, 0, 0);
            a.im = __builtin_amdgcn_mfma_f64_16x16x4f64(x.y, y.x, a.im, 0, 0, 0);
        }
        static __device__ inline int p_of(int r, int lane) { return 4 * r + (lane >> 4); }
        static __device__ inline int q_of(int lane) { return lane & 15; }
        static __device__ inline O   get(const Acc& a, int r) { return make_double2(__dsub_rn(a.rr[r], a.ii[r]), a.im[r]); }
        static __device__ inline void put(Acc& a, int r, O x)
        {
            a.rr[r] = x.x;
            a.ii[r] = 0.0;
            a.im[r] = x.y;
        }
        static __device__ inline E finish(O x, const double* al, const double* be, bool bil, const E* c)
        {
            const double ar = al[0], ai = al[1];
            double       yr = __dsub_rn(__dmul_rn(ar, x.x), __dmul_rn(ai, x.y));
            double       yi = __dadd_rn(__dmul_rn(ai, x.x), __dmul_rn(ar, x.y));
            if(bil)
            {
                const double  br = be[0], bi = be[1];
                const double2 cv = *c;
                yr = __dadd_rn(yr, __dsub_rn(__dmul_rn(br, cv.x), __dmul_rn(bi, cv.y)));
                yi = __dadd_rn(yi, __dadd_rn(__dmul_rn(bi, cv.x), __dmul_rn(br, cv.y)));
            }
            return make_double2(yr, yi);
        }
    };

    // ---- staging: global -> registers -> LDS tile[k][BR + PAD] ---------------------
    //
    // MODE (compile time) says which way an operand's contiguous vectors run.  Loads are
    // never predicated: beyond K the k offset is 0 (the tables are zero padded), beyond
    // the last row the row offset is that of a valid row, so every address is inside the
    // tensor; values beyond K are replaced by zero after the load (TAIL tiles only).
    // Unconditional loads let all of a tile's loads be in flight together.

    template <typename Tr, int MODE, int BR, int BK, int NT>
    struct WStager
    {
        typedef typename Tr::E E;
        typedef typename Tr::S S;
        static constexpr bool  MN    = MODE == GATHER_MN_VEC || MODE == GATHER_MN_HALF; // vectors along the row index
        static constexpr bool  KV    = MODE == GATHER_K_VEC || MODE == GATHER_K_HALF; // vectors along k
        static constexpr int   V     = MODE == GATHER_SCALAR ? 1 : (MODE == GATHER_MN_HALF || MODE == GATHER_K_HALF) ? Tr::VMAX / 2 : Tr::VMAX;
        static constexpr int   N     = BR * BK / NT; // elements per thread
        static constexpr int   NV    = N / V; // vectors per thread
        static constexpr int   PAD   = (sizeof(S) >= 8 ? 2 : 4);
        static constexpr int   PITCH = BR + PAD;
        static constexpr int   ELEMS = BK * PITCH;
        // threads along the fast direction of the mapping, and rows / k's covered per pass
        static constexpr int PER  = MN ? BR / V : (KV ? BK / V : BK);
        static constexpr int STEP = NT / PER;
        static_assert(BR * BK % NT == 0 && N % V == 0 && NV >= 1 && V >= 1, "tile must split evenly over threads");
        static_assert(NT % PER == 0, "thread mapping");

        struct alignas(sizeof(E) * V) PackE
        {
            E e[V];
        };
        struct alignas(sizeof(S) * V) PackS
        {
            S e[V];
        };

        PackE   data[NV];
        int32_t roff[MN ? 1 : NV]; // row-table offsets (loop invariant)
        int32_t koff[MN ? NV : 1]; // k-table offsets of the tile being fetched
        int     a, b;

        __device__ inline void init(const int32_t* rtab, int r0, int tid)
        {
            a = tid % PER;
            b = tid / PER;
            if constexpr(MN)
                roff[0] = rtab[r0 + a * V];
            else
            {
#pragma unroll
                for(int i = 0; i < NV; i++)
                    roff[i] = rtab[r0 + b + i * STEP];
            }
        }

        __device__ inline void load_koffs(const int32_t* ktab, int k0)
        {
            if constexpr(MN)
            {
#pragma unroll
                for(int i = 0; i < NV; i++)
                    koff[i] = ktab[k0 + b + i * STEP];
            }
            else
                koff[0] = ktab[k0 + a * V];
        }

        template <bool TAIL>
        __device__ inline void fetch(const void* base, int k0, int K)
        {
            const E* bp = (const E*)base;
#pragma unroll
            for(int i = 0; i < NV; i++)
            {
                const int  k  = MN ? k0 + b + i * STEP : k0 + a * V;
                const bool ok = !TAIL || k < K;
                // A k-fast vector that straddles K (K is then one contiguous run, not a multiple
                // of the vector) is loaded V elements back from the end of the run, inside the
                // tensor, and moved down in registers; that also clears the slots from K on.
                const bool partial = KV && TAIL && V > 1 && k < K && k + V > K;
                const uint32_t off = MN ? (uint32_t)roff[0] + (uint32_t)koff[i]
                                                            : (uint32_t)roff[i] + (uint32_t)koff[0] - (partial ? (uint32_t)(k + V - K) : 0u);
                PackE v = *(const PackE*)(bp + off);
                if(TAIL && !ok)
                {
#pragma unroll
                    for(int j = 0; j < V; j++)
                        v.e[j] = E{};
                }
                if constexpr(KV && TAIL && V > 1)
                {
                    const int r = K % V; // uniform; 0 when no vector straddles K
                    if(r != 0)
                    {
                        PackE sh = v;
                        switch(V - r) // uniform: every register index below is static
                        {
                        case 1:
#pragma unroll
                            for(int j = 0; j < V; j++)
                                sh.e[j] = j + 1 < V ? v.e[(j + 1) % V] : E{};
                            break;
                        case 2:
#pragma unroll
                            for(int j = 0; j < V; j++)
                                sh.e[j] = j + 2 < V ? v.e[(j + 2) % V] : E{};
                            break;
                        case 3:
#pragma unroll
                            for(int j = 0; j < V; j++)
                                sh.e[j] = j + 3 < V ? v.e[(j + 3) % V] : E{};
                            break;
                        default: break;
                        }
                        if(partial)
                            v = sh;
                    }
                }
                data[i] = v;
            }
        }

        __device__ inline void commit(S* lds)
        {
#pragma unroll
            for(int i = 0; i < NV; i++)
            {
                if constexpr(MN)
                {
                    PackS s;
#pragma unroll
                    for(int j = 0; j < V; j++)
                        s.e[j] = Tr::stage(data[i].e[j]);
                    *(PackS*)(lds + (b + i * STEP) * PITCH + a * V) = s;
                }
                else
                {
#pragma unroll
                    for(int j = 0; j < V; j++)
                        lds[(a * V + j) * PITCH + b + i * STEP] = Tr::stage(data[i].e[j]);
                }
            }
        }
    };

    // Workgroup barrier that orders LDS traffic only: global loads that are still in
    // flight (the next tile's gather) are not waited for.
    __device__ inline void w_lds_barrier()
    {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }

    // Epilogue of the 32/64-bit kernels: D = alpha * acc (+ beta * C) for one wave tile, or the partial
    // sums of a split-K slice into the workspace.  pw / qw: the first row of the wave tile and this
    // lane's column in it; rows / columns from p_own / q_own on are the workgroup tile's to store.
    template <typename Tr, int TP, int TQ>
    __device__ __forceinline__ void
        epilogue_w(const KArgs& a, typename Tr::Acc (&acc)[TP][TQ], int pw, int qw, int p_own, int q_own, int lane)
    {
        typedef typename Tr::E E;
        typedef typename Tr::O O;
        constexpr int          TILE = Tr::TILE;
        auto                   p_in = [&](int p) { return p >= p_own && p < a.P; };
        auto                   q_in = [&](int q) { return q >= q_own && q < a.Q; };
        if(a.split_k > 1)
        {
            O* ws = (O*)a.ws + (size_t)blockIdx.z * (size_t)a.P * (size_t)a.Q;
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int r = 0; r < Tr::NREG; r++)
                {
                    const int p = pw + i * TILE + Tr::p_of(r, lane);
                    if(!p_in(p))
                        continue;
                    O* wrow = ws + (size_t)p * a.Q;
#pragma unroll
                    for(int j = 0; j < TQ; j++)
                    {
                        const int q = qw + j * TILE;
                        if(q_in(q))
                            wrow[q] = Tr::get(acc[i][j], r);
                    }
                }
            return;
        }
        E*         Dp  = (E*)a.D;
        const E*   Cp  = (const E*)a.C;
        const bool bil = a.bilinear != 0;
        const bool aff = a.cd_affine != 0; // C / D offsets are index * stride: no table lookups
        // D may alias C (and, for all the compiler knows, the offset tables), so written naively
        // every element is one dependent round trip: offset, C element, D store.  The offsets and C
        // elements of four accumulator rows are therefore fetched together, ahead of their stores.
        // A lane outside the extents fetches element (0, 0) instead, a valid address, and stores
        // nothing.
        uint32_t dqo[TQ], cqo[TQ];
        bool     qok[TQ];
#pragma unroll
        for(int j = 0; j < TQ; j++)
        {
            const int q  = qw + j * TILE;
            qok[j]       = q_in(q);
            const int qv = qok[j] ? q : 0;
            dqo[j]       = aff ? (uint32_t)qv * (uint32_t)a.dq_stride : (uint32_t)a.dq[qv];
            cqo[j]       = !bil ? 0u : aff ? (uint32_t)qv * (uint32_t)a.cq_stride : (uint32_t)a.cq[qv];
        }
        constexpr int RB = 4;
        static_assert(Tr::NREG % RB == 0, "accumulator rows are fetched four at a time");
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int rb = 0; rb < Tr::NREG; rb += RB)
            {
                uint32_t dpo[RB], cpo[RB];
                bool     pok[RB];
#pragma unroll
                for(int t = 0; t < RB; t++)
                {
                    const int p  = pw + i * TILE + Tr::p_of(rb + t, lane);
                    pok[t]       = p_in(p);
                    const int pv = pok[t] ? p : 0;
                    dpo[t]       = aff ? (uint32_t)pv * (uint32_t)a.dp_stride : (uint32_t)a.dp[pv];
                    cpo[t]       = !bil ? 0u : aff ? (uint32_t)pv * (uint32_t)a.cp_stride : (uint32_t)a.cp[pv];
                }
                E cv[RB][TQ];
                if(bil)
                {
#pragma unroll
                    for(int t = 0; t < RB; t++)
#pragma unroll
                        for(int j = 0; j < TQ; j++)
                            cv[t][j] = Cp[cpo[t] + cqo[j]];
                }
#pragma unroll
                for(int t = 0; t < RB; t++)
#pragma unroll
                    for(int j = 0; j < TQ; j++)
                    {
                        if(pok[t] && qok[j])
                        {
                            const E val = Tr::finish(Tr::get(acc[i][j], rb + t), a.alpha, a.beta, bil, &cv[t][j]);
                            if constexpr(std::is_arithmetic<E>::value)
                                __builtin_nontemporal_store(val, Dp + (dpo[t] + dqo[j]));
                            else
                                Dp[dpo[t] + dqo[j]] = val;
                        }
                    }
            }
    }

    template <typename Tr, int BP, int BQ, int BK, int WP, int WQ, int XM, int YM>
    __global__ void __launch_bounds__(WP* WQ * 64, 2) contract_w_kernel(const KArgs a)
    {
        constexpr int NT   = WP * WQ * 64;
        constexpr int TILE = Tr::TILE;
        constexpr int WTP = BP / WP, WTQ = BQ / WQ;
        constexpr int TP = WTP / TILE, TQ = WTQ / TILE;
        constexpr int KS = BK / Tr::KM;
        static_assert(WTP % TILE == 0 && WTQ % TILE == 0 && BK % Tr::KM == 0 && KS >= 2, "tile shape");
        typedef typename Tr::S        S;
        typedef typename Tr::E        E;
        typedef typename Tr::O        O;
        typedef WStager<Tr, XM, BP, BK, NT> SX;
        typedef WStager<Tr, YM, BQ, BK, NT> SY;
        constexpr int                 STAGE = SX::ELEMS + SY::ELEMS;

        extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
        S* lds = (S*)lds_raw;

        const int tid  = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int wp   = wave / WQ;
        const int wq   = wave % WQ;

        int tp, tq;
        tile_coords(blockIdx.x, a.tiles_p, a.tiles_q, tp, tq);
        // rows / columns from p_own / q_own on are this tile's to store; with shift_p / shift_q the
        // last tile is moved back to end exactly at P / Q (and recomputes some of its neighbour's)
        const int p_own = tp * BP, q_own = tq * BQ;
        const int p0    = (a.shift_p && p_own + BP > a.P) ? a.P - BP : p_own;
        const int q0    = (a.shift_q && q_own + BQ > a.Q) ? a.Q - BQ : q_own;
        auto      p_in  = [&](int p) { return p >= p_own && p < a.P; };
        auto      q_in  = [&](int q) { return q >= q_own && q < a.Q; };

        const int kt_begin = blockIdx.z * a.ktiles_per_split;
        int       kt_end   = kt_begin + a.ktiles_per_split;
        const int kt_all   = (a.K + BK - 1) / BK;
        if(kt_end > kt_all)
            kt_end = kt_all;

        SX sx;
        SY sy;
        sx.init(a.xp, p0, tid);
        sy.init(a.yq, q0, tid);

        typename Tr::Acc acc[TP][TQ];
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int j = 0; j < TQ; j++)
                Tr::zero(acc[i][j]);

        const int row   = lane & (TILE - 1);
        const int kslot = Tr::kslot(lane);
        const int xfo   = kslot * SX::PITCH + wp * WTP + row;
        const int yfo   = kslot * SY::PITCH + wq * WTQ + row;

        // tiles below kt_full lie entirely inside K
        const int kt_full = a.K / BK;

        auto fetch_tile = [&](int t) {
            if(t < kt_full)
            {
                sx.template fetch<false>(a.X, t * BK, a.K);
                sy.template fetch<false>(a.Y, t * BK, a.K);
            }
            else
            {
                sx.template fetch<true>(a.X, t * BK, a.K);
                sy.template fetch<true>(a.Y, t * BK, a.K);
            }
        };
        auto compute = [&](const S* lx, const S* ly, int ks) {
            typename Tr::XF xf[TP];
            typename Tr::YF yf[TQ];
#pragma unroll
            for(int i = 0; i < TP; i++)
                xf[i] = Tr::prep_x(lx[xfo + ks * Tr::KM * SX::PITCH + i * TILE], lane);
#pragma unroll
            for(int j = 0; j < TQ; j++)
                yf[j] = Tr::prep_y(ly[yfo + ks * Tr::KM * SY::PITCH + j * TILE], lane);
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int j = 0; j < TQ; j++)
                    Tr::mma(xf[i], yf[j], acc[i][j]);
        };

        // Software pipeline over K tiles.  While tile t is being multiplied out of one LDS
        // buffer, tile t+1 moves from registers into the other buffer and tile t+2 is
        // gathered from global memory into those registers; one barrier per tile.
        if(kt_begin < kt_end)
        {
            sx.load_koffs(a.xk, kt_begin * BK);
            sy.load_koffs(a.yk, kt_begin * BK);
            fetch_tile(kt_begin);
            sx.load_koffs(a.xk, (kt_begin + 1) * BK);
            sy.load_koffs(a.yk, (kt_begin + 1) * BK);
            sx.commit(lds);
            sy.commit(lds + SX::ELEMS);
            if(kt_begin + 1 < kt_end)
            {
                fetch_tile(kt_begin + 1);
                sx.load_koffs(a.xk, (kt_begin + 2) * BK);
                sy.load_koffs(a.yk, (kt_begin + 2) * BK);
            }
            w_lds_barrier();
        }

        int buf = 0;
        int kt  = kt_begin;
        // steady state: tile kt+2 exists and is a full tile
        const int steady_end = (kt_end < kt_full ? kt_end : kt_full) - 2;
        for(; kt < steady_end; kt++)
        {
            const S* lx = lds + buf * STAGE;
            const S* ly = lx + SX::ELEMS;
            S*       nx = lds + (buf ^ 1) * STAGE;
            S*       ny = nx + SX::ELEMS;
#pragma unroll
            for(int ks = 0; ks < KS; ks++)
            {
                compute(lx, ly, ks);
                // registers of an operand are refilled right after they are stored, so a
                // gather has a whole tile's worth of MFMA time to arrive
                if(ks == 0)
                {
                    sx.commit(nx);
                    sx.template fetch<false>(a.X, (kt + 2) * BK, a.K);
                    sx.load_koffs(a.xk, (kt + 3) * BK);
                }
                if(ks == 1)
                {
                    sy.commit(ny);
                    sy.template fetch<false>(a.Y, (kt + 2) * BK, a.K);
                    sy.load_koffs(a.yk, (kt + 3) * BK);
                }
            }
            w_lds_barrier();
            buf ^= 1;
        }
        // drain: at most the last three tiles (and every tile of a short K)
        for(; kt < kt_end; kt++)
        {
            const S* lx = lds + buf * STAGE;
            const S* ly = lx + SX::ELEMS;
            S*       nx = lds + (buf ^ 1) * STAGE;
            S*       ny = nx + SX::ELEMS;
#pragma unroll
            for(int ks = 0; ks < KS; ks++)
                compute(lx, ly, ks);
            if(kt + 1 < kt_end)
            {
                sx.commit(nx);
                sy.commit(ny);
                if(kt + 2 < kt_end)
                {
                    fetch_tile(kt + 2);
                    sx.load_koffs(a.xk, (kt + 3) * BK);
                    sy.load_koffs(a.yk, (kt + 3) * BK);
                }
            }
            w_lds_barrier();
            buf ^= 1;
        }

        epilogue_w<Tr, TP, TQ>(a, acc, p0 + wp * WTP, q0 + wq * WTQ + Tr::q_of(lane), p_own, q_own, lane);
    }

    template <typename Tr, int BP, int BQ, int BK>
    constexpr int lds_bytes_w()
    {
        return 2 * (WStager<Tr, 0, BP, BK, 256>::ELEMS + WStager<Tr, 0, BQ, BK, 256>::ELEMS)
               * (int)sizeof(typename Tr::S);
    }

    template <typename Tr, int BP, int BQ, int BK, int WP, int WQ, int XM, int YM>
    int launch_w(const KArgs& a, hipStream_t stream)
    {
        constexpr int LDS  = lds_bytes_w<Tr, BP, BQ, BK>();
        auto          kern = contract_w_kernel<Tr, BP, BQ, BK, WP, WQ, XM, YM>;
        static const hipError_t attr = hipFuncSetAttribute(
            (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if(attr != hipSuccess)
            return (int)attr;
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(kern, grid, dim3(WP * WQ * 64), LDS, stream, a);
        return (int)hipGetLastError();
    }
}

// gather mode <-> (kfast, vec) as the registry describes it
#define HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, XM, YM)                                      \
    {                                                                                          \
        hiptk::TR::CLS, ID, (XM != hiptk::GATHER_MN_VEC && XM != hiptk::GATHER_MN_HALF),       \
            (YM != hiptk::GATHER_MN_VEC && YM != hiptk::GATHER_MN_HALF),                       \
            (XM == hiptk::GATHER_SCALAR ? 1 : XM >= hiptk::GATHER_MN_HALF ? hiptk::TR::VMAX / 2 : hiptk::TR::VMAX), \
            (YM == hiptk::GATHER_SCALAR ? 1 : YM >= hiptk::GATHER_MN_HALF ? hiptk::TR::VMAX / 2 : hiptk::TR::VMAX), 0, BP, BQ, BK, WP *WQ * 64, \
            hiptk::lds_bytes_w<hiptk::TR, BP, BQ, BK>(), #TR "_" #BP "x" #BQ "x" #BK "_" #XM #YM, \
            &hiptk::launch_w<hiptk::TR, BP, BQ, BK, WP, WQ, XM, YM>                            \
    }

#define HIPTK_W_TILE(TR, ID, BP, BQ, BK, WP, WQ)                                               \
    HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 0, 0), HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 0, 1), \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 0, 2),                                       \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 1, 0),                                       \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 1, 1),                                       \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 1, 2),                                       \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 2, 0),                                       \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 2, 1),                                       \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 2, 2)
// ... with both operands in vectors of VMAX / 2
#define HIPTK_W_TILE_HALF(TR, ID, BP, BQ, BK, WP, WQ)                                          \
    HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 3, 3), HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 3, 4), \
        HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 4, 3), HIPTK_W_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, 4, 4)
