// 16-bit (f16 / bf16) contraction kernel for gfx950.
//
//   acc[p][q] = sum_k X[xp[p] + xk[k]] * Y[yq[q] + yk[k]]        (f32 accumulate)
//   D[dp[p] + dq[q]] = alpha * acc (+ beta * C[cp[p] + cq[q]])    (f32 epilogue, one rounding)
//
// One workgroup of WP x WQ wavefronts (64 lanes each) owns a BP x BQ output tile and
// walks K in steps of BK.  Per step the X and Y tiles are gathered from global memory
// through the offset tables into registers (one step ahead of their use), written
// into one of two LDS buffers, and consumed by v_mfma_f32_32x32x16_{f16,bf16}.
//
// LDS layout depends on which way an operand's contiguous vectors run:
//   vectors along k  ("k-fast"):  tile[row][BK + 8]; a lane's MFMA operand (8
//       consecutive k of one row) is one ds_read_b128, the +8 pad (16 B) staggers
//       rows over the banks.
//   vectors along the row index:  tile[k][BR + 16]; the operand is assembled by two
//       ds_read_b64_tr_b16 (the transposing LDS read of CDNA4), so no software
//       transpose is needed.  The +16 pad (32 B) puts the four k-rows a 16-lane group
//       touches into disjoint bank ranges.
//
// MFMA operand / result register layouts used here (verified on hardware):
//   operand: lane l holds row (l % 32), k = 8 * (l / 32) .. + 7
//   result : lane l, register r holds p = 8 * (r / 4) + 4 * (l / 32) + r % 4, q = l % 32
// X feeds the first MFMA operand (p is register-varying), Y the second (q is
// lane-varying), so at a fixed register the 32 lanes of a half-wave write 32
// consecutive q: the planner orients the problem so that q is D's contiguous index.
#pragma once
#include <type_traits>

#include "kargs.h"

namespace hiptk
{
    typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
    typedef __bf16   bf16x8_t __attribute__((ext_vector_type(8)));
    typedef float    f32x16_t __attribute__((ext_vector_type(16)));
    typedef short    short4_t __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
// D is written once and not read again by this launch: its vector stores are non-temporal, which
// leaves the L2 to the operand panels (4096^3 f16: scale 123.4 -> 121.5 us, bilinear 128.3 -> 127.2 us).
// Reading C the same way costs 5 % (135.0 us) and is not done.
#define HIPTK_STORE_D(ptr, val) __builtin_nontemporal_store((val), (ptr))
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    typedef float    f32x4_t __attribute__((ext_vector_type(4)));

    // Workgroup barrier that orders LDS traffic only: global loads that are still in
    // flight (the next tile's gather) are not waited for.
    __device__ inline void lds_barrier()
    {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }

    // f32 -> bf16, round to nearest even: v_cvt_pk_bf16_f32 on gfx950 (NaNs come out quiet)
    __device__ inline uint16_t f32_to_bf16_rne(float f)
    {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }

    struct TraitsF16
    {
        static constexpr int CLS = HIPTK_F16;
        typedef uint16_t     src_t; // storage of A and B
        typedef uint16_t     out_t; // storage of C and D
        static __device__ inline f32x16_t mfma(u32x4_t x, u32x4_t y, f32x16_t acc)
        {
            return __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(half8_t, x), __builtin_bit_cast(half8_t, y), acc, 0, 0, 0);
        }
        static __device__ inline uint16_t from_f32(float f)
        {
            return __builtin_bit_cast(uint16_t, (_Float16)f);
        }
        static __device__ inline float to_f32(uint16_t h)
        {
            return (float)__builtin_bit_cast(_Float16, h);
        }
        static __device__ inline uint16_t stage(uint16_t v) { return v; }
        static __device__ inline out_t    out_from_f32(float f) { return from_f32(f); }
        static __device__ inline float    out_to_f32(out_t v) { return to_f32(v); }
        static __device__ inline float    axpby(float al, float x, float be, float c, bool bil)
        {
            return bil ? al * x + be * c : al * x;
        }
    };

    struct TraitsBF16
    {
        static constexpr int CLS = HIPTK_BF16;
        typedef uint16_t     src_t;
        typedef uint16_t     out_t;
        static __device__ inline f32x16_t mfma(u32x4_t x, u32x4_t y, f32x16_t acc)
        {
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8_t, x), __builtin_bit_cast(bf16x8_t, y), acc, 0, 0, 0);
        }
        static __device__ inline uint16_t from_f32(float f) { return f32_to_bf16_rne(f); }
        static __device__ inline float    to_f32(uint16_t h)
        {
            return __uint_as_float((uint32_t)h << 16);
        }
        static __device__ inline uint16_t stage(uint16_t v) { return v; }
        static __device__ inline out_t    out_from_f32(float f) { return from_f32(f); }
        static __device__ inline float    out_to_f32(out_t v) { return to_f32(v); }
        static __device__ inline float    axpby(float al, float x, float be, float c, bool bil)
        {
            return bil ? al * x + be * c : al * x;
        }
    };

    // f32 storage, operands rounded to f16 / bf16 when they are staged into LDS (the
    // reference's "compute type" for these rows), f32 accumulate, f32 results.
    struct TraitsF32AsF16 : TraitsF16
    {
        static constexpr int CLS = HIPTK_F32_AS_F16;
        typedef float        src_t;
        typedef float        out_t;
        static __device__ inline uint16_t stage(float v) { return TraitsF16::from_f32(v); }
        static __device__ inline out_t    out_from_f32(float f) { return f; }
        static __device__ inline float    out_to_f32(out_t v) { return v; }
        // separately rounded products, as the CPU path computes alpha * x + beta * c
        static __device__ inline float axpby(float al, float x, float be, float c, bool bil)
        {
            const float y = __fmul_rn(al, x);
            return bil ? __fadd_rn(y, __fmul_rn(be, c)) : y;
        }
    };

    struct TraitsF32AsBF16 : TraitsBF16
    {
        static constexpr int CLS = HIPTK_F32_AS_BF16;
        typedef float        src_t;
        typedef float        out_t;
        static __device__ inline uint16_t stage(float v) { return f32_to_bf16_rne(v); }
        static __device__ inline out_t    out_from_f32(float f) { return f; }
        static __device__ inline float    out_to_f32(out_t v) { return v; }
        static __device__ inline float    axpby(float al, float x, float be, float c, bool bil)
        {
            const float y = __fmul_rn(al, x);
            return bil ? __fadd_rn(y, __fmul_rn(be, c)) : y;
        }
    };

    // LDS tile geometry of one operand (16-bit elements).
    template <bool KF, int BR, int BK>
    struct TileLds
    {
        static constexpr int PITCH = KF ? BK + 8 : BR + 16;
        static constexpr int ELEMS = (KF ? BR : BK) * PITCH;
    };

    // Global -> register -> LDS staging of one operand tile.
    //
    // KAFF: the reduction index maps to memory with one stride (all K modes fused into
    // one), so k offsets are a multiply instead of a table lookup.
    // Loads are never predicated: beyond K the k offset is 0 (the tables are zero padded;
    // the affine form clamps), which is a valid element of the same row, and the loaded
    // bits are masked to zero afterwards.  Keeping the loads unconditional lets all of a
    // tile's loads be in flight together.
    template <typename Tr, bool KF, int V, int BR, int BK, int NT, bool KAFF>
    struct Stager
    {
        typedef typename Tr::src_t src_t;
        static constexpr int PER   = KF ? BK / V : BR / V; // vectors along the vector direction
        static constexpr int STEP  = NT / PER; // rows (k-fast) or k's covered per pass
        static constexpr int N     = (BR * BK / V) / NT; // vectors per thread
        static constexpr int W     = V >= 2 ? V / 2 : 1; // 32-bit words per staged vector
        static constexpr int PITCH = TileLds<KF, BR, BK>::PITCH;
        static_assert(NT % PER == 0, "thread count must cover whole vector rows");
        static_assert((BR * BK / V) % NT == 0 && N >= 1, "tile must split evenly over threads");
        static constexpr bool SRC32 = sizeof(src_t) == 4; // f32 storage, rounded when staged
        static_assert(!SRC32 || V == 4 || V == 1, "f32 sources are gathered 16 bytes or one element at a time");

        uint32_t data[N][W];
        int32_t  roff[KF ? N : 1]; // row-table offsets (loop invariant)
        int32_t  koff[KF ? 1 : N]; // k-table offsets of the tile being fetched
        int      a, b; // k-fast: a = vector slot along k, b = first row; else a = row vector, b = first k

        __device__ inline void init(const int32_t* rtab, int r0, int tid)
        {
            a = tid % PER;
            b = tid / PER;
            if constexpr(KF)
            {
#pragma unroll
                for(int i = 0; i < N; i++)
                    roff[i] = rtab[r0 + b + i * STEP];
            }
            else
                roff[0] = rtab[r0 + a * V];
        }

        // k offsets of the tile that starts at k0 (table form; one tile ahead of its fetch)
        __device__ inline void load_koffs(const int32_t* ktab, int k0)
        {
            if constexpr(!KAFF)
            {
                if constexpr(KF)
                    koff[0] = ktab[k0 + a * V];
                else
                {
#pragma unroll
                    for(int i = 0; i < N; i++)
                        koff[i] = ktab[k0 + b + i * STEP];
                }
            }
        }

        __device__ inline void fetch_one(const src_t* p, uint32_t mask, uint32_t (&d)[W])
        {
            if constexpr(SRC32 && V == 4)
            {
                const f32x4_t v = *(const f32x4_t*)p;
                d[0] = ((uint32_t)Tr::stage(v[0]) | ((uint32_t)Tr::stage(v[1]) << 16)) & mask;
                d[1] = ((uint32_t)Tr::stage(v[2]) | ((uint32_t)Tr::stage(v[3]) << 16)) & mask;
            }
            else if constexpr(SRC32)
                d[0] = (uint32_t)Tr::stage(*p) & mask;
            else if constexpr(V == 8)
            {
                const u32x4_t v = *(const u32x4_t*)p;
                d[0]            = v[0] & mask;
                d[1]            = v[1] & mask;
                d[2]            = v[2] & mask;
                d[3]            = v[3] & mask;
            }
            else if constexpr(V == 4)
            {
                const u32x2_t v = *(const u32x2_t*)p;
                d[0]            = v[0] & mask;
                d[1]            = v[1] & mask;
            }
            else if constexpr(V == 2)
                d[0] = *(const uint32_t*)p & mask;
            else
                d[0] = (uint32_t)*p & mask;
        }

        // d holds V staged 16-bit elements, element e in bits 16 * (e % 2) of word e / 2.  Moves
        // element e + s to element e (s = 1 .. V - 1, the same for the whole wave) and clears the
        // top s elements.
        __device__ static inline void shift_down(uint32_t (&d)[W], int s)
        {
            if constexpr(V >= 2)
            {
                uint32_t t[2 * W];
#pragma unroll
                for(int i = 0; i < W; i++)
                {
                    t[i]     = d[i];
                    t[W + i] = 0u;
                }
                const int ws = s >> 1;
                // s is uniform: a switch over the word shift keeps every register index static
                switch(ws)
                {
#define HIPTK_SHIFT_CASE(WS)                                                                        \
    case WS:                                                                                        \
        _Pragma("unroll") for(int i = 0; i < W; i++)                                                \
        {                                                                                           \
            const uint32_t lo = (i + WS < 2 * W) ? t[(i + WS) % (2 * W)] : 0u;                      \
            const uint32_t hi = (i + WS + 1 < 2 * W) ? t[(i + WS + 1) % (2 * W)] : 0u;              \
            d[i]              = (s & 1) ? __builtin_amdgcn_alignbit(hi, lo, 16) : lo;               \
        }                                                                                           \
        break;
                    HIPTK_SHIFT_CASE(0)
                    HIPTK_SHIFT_CASE(1)
                    HIPTK_SHIFT_CASE(2)
                    HIPTK_SHIFT_CASE(3)
#undef HIPTK_SHIFT_CASE
                default: break;
                }
            }
        }

        // Fetch the tile whose first k is k0.  TAIL: the tile may reach beyond K.
        //
        // k-fast vectors and a K that is not a multiple of the vector (the planner allows that
        // when k is one contiguous run): the vector that straddles K is loaded V elements back
        // from the end of the run - inside the tensor - and moved down in registers, which also
        // clears the slots from K on.
        template <bool TAIL>
        __device__ inline void fetch(const void* base, int k0, int K, int kstride)
        {
            const src_t* bp = (const src_t*)base;
            if constexpr(KF)
            {
                const int      k       = k0 + a * V;
                const bool     partial = TAIL && V > 1 && k < K && k + V > K;
                const int      over    = k + V - K; // elements of a straddling vector beyond K
                const uint32_t mask    = (!TAIL || k < K) ? 0xFFFFFFFFu : 0u;
                uint32_t       ko;
                if constexpr(KAFF)
                    ko = (uint32_t)((TAIL && k >= K) ? 0 : (partial ? k - over : k)) * (uint32_t)kstride;
                else
                    ko = (uint32_t)koff[0] - (partial ? (uint32_t)over : 0u); // (k is this operand's unit-stride index)
#pragma unroll
                for(int i = 0; i < N; i++)
                    fetch_one(bp + ((uint32_t)roff[i] + ko), mask, data[i]);
                if constexpr(TAIL && V > 1)
                {
                    const int r = K % V; // uniform; 0 when no vector straddles K
                    if(r != 0)
                    {
#pragma unroll
                        for(int i = 0; i < N; i++)
                        {
                            uint32_t sh[W];
#pragma unroll
                            for(int w = 0; w < W; w++)
                                sh[w] = data[i][w];
                            shift_down(sh, V - r);
#pragma unroll
                            for(int w = 0; w < W; w++)
                                data[i][w] = partial ? sh[w] : data[i][w];
                        }
                    }
                }
            }
            else
            {
#pragma unroll
                for(int i = 0; i < N; i++)
                {
                    const int      k    = k0 + b + i * STEP;
                    const uint32_t mask = (!TAIL || k < K) ? 0xFFFFFFFFu : 0u;
                    uint32_t       ko;
                    if constexpr(KAFF)
                        ko = (uint32_t)((TAIL && k >= K) ? 0 : k) * (uint32_t)kstride;
                    else
                        ko = (uint32_t)koff[i];
                    fetch_one(bp + ((uint32_t)roff[0] + ko), mask, data[i]);
                }
            }
        }

        __device__ inline void commit(uint16_t* lds)
        {
#pragma unroll
            for(int i = 0; i < N; i++)
            {
                uint16_t* dst = lds + (b + i * STEP) * PITCH + a * V;
                if constexpr(V == 8)
                {
                    u32x4_t v = {data[i][0], data[i][1], data[i][2], data[i][3]};
                    *(u32x4_t*)dst = v;
                }
                else if constexpr(V == 4)
                {
                    u32x2_t v      = {data[i][0], data[i][1]};
                    *(u32x2_t*)dst = v;
                }
                else if constexpr(V == 2)
                    *(uint32_t*)dst = data[i][0];
                else
                    *dst = (uint16_t)data[i][0];
            }
        }
    };

    // Orders one wave's own LDS writes before its later LDS reads (and the reverse): enough
    // when the data never leaves the wave, since a wave's LDS operations execute in order.
    __device__ inline void wave_lds_fence()
    {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
    }

    // MFMA operand fetch from LDS for the 32-row block starting at row r0, k-substep ks.
    template <bool KF, int PITCH>
    __device__ inline int frag_base(int lane)
    {
        if constexpr(KF)
            return (lane & 31) * PITCH + 8 * (lane >> 5);
        else
            return (8 * (lane >> 5) + ((lane & 15) >> 2)) * PITCH + 16 * ((lane >> 4) & 1)
                   + 4 * (lane & 3);
    }

    template <bool KF, int PITCH>
    __device__ inline u32x4_t frag_load(const uint16_t* lds, int base, int r0, int ks)
    {
        if constexpr(KF)
            return *(const u32x4_t*)(lds + base + r0 * PITCH + ks * 16);
        else
        {
            typedef short4_t __attribute__((address_space(3))) * lds_s4_ptr;
            const uint16_t* p  = lds + base + ks * 16 * PITCH + r0;
            short4_t        lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p));
            short4_t        hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p + 4 * PITCH));
            u32x2_t         l2 = __builtin_bit_cast(u32x2_t, lo);
            u32x2_t         h2 = __builtin_bit_cast(u32x2_t, hi);
            u32x4_t         v  = {l2[0], l2[1], h2[0], h2[1]};
            return v;
        }
    }

    // Where a lane's accumulators of one 32-row slab of its wave tile lie, for the epilogue: as QUADS
    // groups of 4 consecutive rows at one column, quad q = c * NRQ + g being the g-th of the lane's
    // NRQ row groups at its c-th of NCOL columns.
    //   row0(q, lane): first of the quad's rows within the slab;  col(q, lane): its column within the wave tile;
    //   get(i, q, e):  the accumulator of row row0 + e of slab i.
    // v_mfma_f32_32x32x16: blocks of 32 x 32, 16 registers per lane (register r: row 8 (r / 4) + 4 (lane / 32) + r % 4,
    // column lane % 32)
    template <int TP, int TQ>
    struct Acc32
    {
        f32x16_t (&a)[TP][TQ];
        static constexpr int NCOL = TQ, NRQ = 4, QUADS = NCOL * NRQ;
        __device__ static inline int row0(int q, int lane) { return 8 * (q & 3) + 4 * (lane >> 5); }
        __device__ static inline int col(int q, int lane) { return 32 * (q >> 2) + (lane & 31); }
        __device__ inline float      get(int i, int q, int e) const { return a[i][q >> 2][4 * (q & 3) + e]; }
    };
    // v_mfma_f32_16x16x32: blocks of 16 x 16, 4 registers per lane (register r: row 4 (lane / 16) + r, column lane % 16)
    template <int TP, int TQ>
    struct Acc16
    {
        f32x4_t (&a)[2 * TP][2 * TQ];
        static constexpr int NCOL = 2 * TQ, NRQ = 2, QUADS = NCOL * NRQ;
        __device__ static inline int row0(int q, int lane) { return 16 * (q & 1) + 4 * (lane >> 4); }
        __device__ static inline int col(int q, int lane) { return 16 * (q >> 1) + (lane & 15); }
        __device__ inline float      get(int i, int q, int e) const { return a[2 * i + (q & 1)][q >> 1][e]; }
    };

    // Epilogue of the 16-bit kernels: D = alpha * acc (+ beta * C) for the wave tiles of one
    // workgroup tile.  `lds` is the workgroup's whole LDS allocation of LDSCAP bytes, free by
    // now (every wave has passed the main loop's last barrier); p0 / q0 are the first row / column
    // the tile computed, p_own / q_own the first it stores (they differ for a tile that was moved
    // back to end at P / Q).
    // DEEP: two slabs of C in flight also for the 128-wide wave tiles (for kernels whose main loop
    // leaves the registers for it).
    template <typename Tr, int WP, int WQ, int TP, int TQ, int LDSCAP, bool DEEP, typename Acc>
    __device__ __forceinline__ void epilogue_acc(const KArgs& a, const Acc acc, uint16_t* lds, int p0, int q0, int p_own, int q_own)
    {
        constexpr int QUADS = Acc::QUADS;
        constexpr int WTP = TP * 32, WTQ = TQ * 32;
        const int     tid  = threadIdx.x;
        const int     lane = tid & 63;
        const int     wave = tid >> 6;
        const int     wp   = wave / WQ;
        const int     wq   = wave % WQ;
        auto          p_in = [&](int p) { return p >= p_own && p < a.P; };
        auto          q_in = [&](int q) { return q >= q_own && q < a.Q; };
        // a vector of 8 columns is stored when any of it is this tile's (the others are the
        // neighbour's, recomputed here to the same values)
        auto q_in8 = [&](int q) { return q + 8 > q_own && q < a.Q; };
        const float alpha = (float)a.alpha[0];
        const float beta  = (float)a.beta[0];
        if(a.split_k > 1)
        {
            float* ws = (float*)a.ws + (size_t)blockIdx.z * (size_t)a.P * (size_t)a.Q;
#pragma unroll
            for(int u = 0; u < QUADS; u++)
            {
                const int q = q0 + wq * WTQ + Acc::col(u, lane);
                if(!q_in(q))
                    continue;
#pragma unroll
                for(int i = 0; i < TP; i++)
#pragma unroll
                    for(int e = 0; e < 4; e++)
                    {
                        const int p = p0 + wp * WTP + i * 32 + Acc::row0(u, lane) + e;
                        if(p_in(p))
                            ws[(size_t)p * a.Q + q] = acc.get(i, u, e);
                    }
            }
            return;
        }
        typedef typename Tr::out_t out_t;
        out_t*       Dp = (out_t*)a.D;
        const out_t* Cp = (const out_t*)a.C;
        // (measured: a gain only for the wide wave tiles; and the staging has to fit)
        if constexpr(sizeof(out_t) == 2 && WTQ >= 128 && 2 * WTQ * 36 * 2 * WP * WQ <= LDSCAP)
        if(a.cd_vec == 8 && !a.bilinear)
        {
            // Scale with D contiguous along q in runs of 8.  The results are converted to their
            // 16-bit type in the accumulator layout (lane = column q, 4 consecutive registers =
            // 4 consecutive rows p) and transposed through LDS at half the f32 volume: a slab is
            // staged as [q][32 rows + 4] halves with one ds_write_b64 per 4 registers, and read
            // back with the transposing ds_read_b64_tr_b16, which hands every lane 4 consecutive
            // q of one row; two of them make the 16-byte store.  A 16-lane group covers 4 rows x
            // 32 q, a store instruction 4 rows x 256 contiguous bytes (8 x 128 for 64-wide wave
            // tiles).  The 72-byte column pitch keeps both the writes and the reads conflict free.
            constexpr int PH   = 36; // halves per staged column: 32 rows + pad
            constexpr int NVEC = (32 * WTQ / 8) / 64; // 16-byte stores per lane and slab
            constexpr int QB   = WTQ / 32; // 32-column blocks per wave tile
            static_assert(2 * WTQ * PH * 2 * WP * WQ <= LDSCAP, "epilogue staging must fit the operand buffers");
            typedef short4_t __attribute__((address_space(3))) * lds_s4_ptr;
            uint16_t* const st0 = lds + wave * (2 * WTQ * PH);
            const int       pw  = p0 + wp * WTP;
            const int       qw  = q0 + wq * WTQ;
            const bool      aff = a.cd_affine != 0;
            const int       L   = lane & 15;
            const int       G   = lane >> 4;
            // this lane's row within a slab and first column, per store vector
            int      prow[NVEC], qcol[NVEC];
            uint32_t dqo[NVEC];
            bool     qok[NVEC];
#pragma unroll
            for(int v = 0; v < NVEC; v++)
            {
                const int u = v * 4 + G; // (row quad, column block) unit of this 16-lane group
                prow[v]     = 4 * (u / QB) + (L & 3);
                qcol[v]     = 32 * (u % QB) + 8 * (L >> 2);
                const int q = qw + qcol[v];
                qok[v]      = q_in8(q);
                dqo[v]      = !qok[v] ? 0u : aff ? (uint32_t)q * (uint32_t)a.dq_stride : (uint32_t)a.dq[q];
            }
            uint32_t doff[2][NVEC];
            auto     offsets = [&](int i, uint32_t (&d)[NVEC]) {
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                {
                    const int p = pw + i * 32 + prow[v];
                    d[v] = !(qok[v] && p_in(p)) ? 0u : (aff ? (uint32_t)p * (uint32_t)a.dp_stride : (uint32_t)a.dp[p]) + dqo[v];
                }
            };
            auto write_slab = [&](int i, uint16_t* dst) {
#pragma unroll
                for(int u = 0; u < QUADS; u++)
                {
                    u32x2_t w;
                    w[0] = (uint32_t)Tr::from_f32(alpha * acc.get(i, u, 0)) | ((uint32_t)Tr::from_f32(alpha * acc.get(i, u, 1)) << 16);
                    w[1] = (uint32_t)Tr::from_f32(alpha * acc.get(i, u, 2)) | ((uint32_t)Tr::from_f32(alpha * acc.get(i, u, 3)) << 16);
                    *(u32x2_t*)(dst + Acc::col(u, lane) * PH + Acc::row0(u, lane)) = w;
                }
            };
            offsets(0, doff[0]);
            write_slab(0, st0);
            wave_lds_fence();
#pragma unroll
            for(int i = 0; i < TP; i++)
            {
                const uint16_t* cur = st0 + (i & 1) * (WTQ * PH);
                if(i + 1 < TP)
                {
                    offsets(i + 1, doff[(i + 1) & 1]);
                    write_slab(i + 1, st0 + ((i + 1) & 1) * (WTQ * PH));
                }
                u32x4_t o[NVEC];
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                {
                    // the word this lane supplies: column qcol-block + 8 * (L % 4) + L / 4, the group's 4 rows
                    const int       u   = v * 4 + G;
                    const uint16_t* src = cur + (32 * (u % QB) + 8 * (L & 3) + (L >> 2)) * PH + 4 * (u / QB);
                    const short4_t  lo  = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(src));
                    const short4_t  hi  = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(src + 4 * PH));
                    const u32x2_t   l2  = __builtin_bit_cast(u32x2_t, lo);
                    const u32x2_t   h2  = __builtin_bit_cast(u32x2_t, hi);
                    o[v]                = u32x4_t{l2[0], l2[1], h2[0], h2[1]};
                }
                // table-driven offsets are loads: await the next slab's before this slab's stores
                // go out (loads and stores share one in-order counter)
                if(!aff)
                    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                    if(qok[v] && p_in(pw + i * 32 + prow[v]))
                        HIPTK_STORE_D((u32x4_t*)(Dp + doff[i & 1][v]), o[v]);
                wave_lds_fence();
            }
            return;
        }
        if constexpr(sizeof(out_t) == 2)
        if(a.cd_vec == 8)
        {
            // C and D are contiguous along q in runs of 8: route each 32-row slab of the
            // wave's accumulators through LDS (the operand buffers are free now) so that a
            // lane ends up with 8 consecutive q of one row and moves them as one 16-byte
            // access; 16 lanes cover 256 contiguous bytes of a row.
            constexpr int EP   = WTQ + 4; // floats per staged row
            constexpr int VPR  = WTQ / 8; // 8-element vectors per staged row
            constexpr int NVEC = (32 * WTQ / 8) / 64; // vectors per lane and slab
            static_assert(32 * EP * 4 * WP * WQ <= LDSCAP, "epilogue staging must fit the operand buffers");
            const int pw = p0 + wp * WTP;
            const int qw = q0 + wq * WTQ;
            // One slab of C in flight, requested (after the look-ups behind its addresses) while the
            // slab before it is staged.
            auto one_in_flight = [&]() {
            const bool bil = a.bilinear != 0;
            const bool aff = a.cd_affine != 0;
            // Offsets and C values of a slab are fetched while the slab before it is being
            // written, so that table look-ups, C loads and D stores of different vectors are
            // all in flight together instead of one dependent round trip per vector.  (The
            // compiler cannot hoist them itself: D may alias C.)  A lane reads every C element
            // before it writes the D element at the same place, so exact aliasing stays valid.
            uint32_t dqo[NVEC], cqo[NVEC];
            bool     qok[NVEC];
#pragma unroll
            for(int v = 0; v < NVEC; v++)
            {
                const int q = qw + ((v * 64 + lane) % VPR) * 8;
                qok[v]      = q_in8(q);
                // affine C / D (every benchmark-style packed layout): offsets are computed, so the
                // epilogue starts without a round trip to the offset tables
                dqo[v] = !qok[v] ? 0u : aff ? (uint32_t)q * (uint32_t)a.dq_stride : (uint32_t)a.dq[q];
                cqo[v] = !(qok[v] && bil) ? 0u : aff ? (uint32_t)q * (uint32_t)a.cq_stride : (uint32_t)a.cq[q];
            }
            struct Slab
            {
                u32x4_t  c[NVEC];
                uint32_t doff[NVEC];
                bool     ok[NVEC];
            };
            Slab sl[2];
            // Offsets from tables, in a kernel with registers to spare (DEEP): the row look-ups of all
            // slabs are made here, before the first store.  Inside the loop a look-up sits behind the
            // stores of the slab before it, and the wait for it (its result is the address of a C
            // load) is then also a wait for those stores: one store drain per slab.
            // (The tables are padded beyond every index a tile reaches, so these need no guard.)
            constexpr bool HOIST = DEEP && TP * NVEC <= 32;
            uint32_t       hd[HOIST ? TP : 1][NVEC], hc[HOIST ? TP : 1][NVEC];
            if constexpr(HOIST)
            {
                if(!aff)
                {
#pragma unroll
                    for(int i = 0; i < TP; i++)
#pragma unroll
                        for(int v = 0; v < NVEC; v++)
                        {
                            const int p = pw + i * 32 + (v * 64 + lane) / VPR;
                            hd[i][v]    = (uint32_t)a.dp[p] + dqo[v];
                            hc[i][v]    = bil ? (uint32_t)a.cp[p] + cqo[v] : 0u;
                        }
                }
            }
            auto prefetch = [&](int i, Slab& s) {
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                {
                    const int p = pw + i * 32 + (v * 64 + lane) / VPR;
                    s.ok[v]     = qok[v] && p_in(p);
                    uint32_t dof, cof;
                    if(HOIST && !aff)
                    {
                        dof = hd[HOIST ? i : 0][v];
                        cof = hc[HOIST ? i : 0][v];
                    }
                    else
                    {
                        dof = !s.ok[v] ? 0u : (aff ? (uint32_t)p * (uint32_t)a.dp_stride : (uint32_t)a.dp[p]) + dqo[v];
                        cof = !(s.ok[v] && bil) ? 0u : (aff ? (uint32_t)p * (uint32_t)a.cp_stride : (uint32_t)a.cp[p]) + cqo[v];
                    }
                    s.doff[v]  = s.ok[v] ? dof : 0u;
                    u32x4_t c4 = {0u, 0u, 0u, 0u};
                    if(s.ok[v] && bil)
                        c4 = *(const u32x4_t*)(Cp + cof);
                    s.c[v] = c4;
                }
            };
            // Two staging buffers per wave when the operand buffers have room for them: slab
            // i+1 is written to LDS while slab i is read back, converted and stored.
            constexpr bool DB = 2 * 32 * EP * 4 * WP * WQ <= LDSCAP;
            float* const   st0 = (float*)lds + wave * ((DB ? 2 : 1) * 32 * EP);
            auto write_slab = [&](int i, float* dst) {
#pragma unroll
                for(int u = 0; u < QUADS; u++)
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        dst[(Acc::row0(u, lane) + e) * EP + Acc::col(u, lane)] = acc.get(i, u, e);
            };
            prefetch(0, sl[0]);
            if constexpr(DB)
            {
                write_slab(0, st0);
                wave_lds_fence();
            }
#pragma unroll
            for(int i = 0; i < TP; i++)
            {
                const float* cur_st = st0 + (DB ? (i & 1) * 32 * EP : 0);
                if constexpr(DB)
                {
                    if(i + 1 < TP)
                    {
                        prefetch(i + 1, sl[(i + 1) & 1]);
                        write_slab(i + 1, st0 + ((i + 1) & 1) * 32 * EP);
                    }
                }
                else
                {
                    write_slab(i, st0);
                    if(i + 1 < TP)
                        prefetch(i + 1, sl[(i + 1) & 1]);
                    wave_lds_fence();
                }
                const Slab& cur = sl[i & 1];
                // all of the slab's vectors are read from LDS before any is converted and stored
                f32x4_t lo[NVEC], hi[NVEC];
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                {
                    const int    slot = v * 64 + lane;
                    const float* src  = cur_st + (slot / VPR) * EP + (slot % VPR) * 8;
                    lo[v]             = *(const f32x4_t*)src;
                    hi[v]             = *(const f32x4_t*)(src + 4);
                }
                u32x4_t o[NVEC];
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                {
                    float v8[8] = {lo[v][0], lo[v][1], lo[v][2], lo[v][3], hi[v][0], hi[v][1], hi[v][2], hi[v][3]};
                    if(bil)
                    {
                        const u32x4_t c4 = cur.c[v];
#pragma unroll
                        for(int e = 0; e < 8; e++)
                        {
                            const uint16_t cb = (uint16_t)(c4[e >> 1] >> ((e & 1) * 16));
                            v8[e]             = alpha * v8[e] + beta * Tr::to_f32(cb);
                        }
                    }
                    else
                    {
#pragma unroll
                        for(int e = 0; e < 8; e++)
                            v8[e] = alpha * v8[e];
                    }
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        o[v][e] = (uint32_t)Tr::from_f32(v8[2 * e]) | ((uint32_t)Tr::from_f32(v8[2 * e + 1]) << 16);
                }
                // Loads and stores share one in-order counter, so waiting for a load also waits
                // for every store issued before it.  The next slab's prefetch is therefore
                // awaited here, before this slab's stores are issued: the only stores it can
                // wait for are the previous slab's, a whole slab old, and this slab's stores
                // then drain while the next slab is converted.
                // (With computed offsets and no C there are no loads, and nothing to wait for.)
                if(bil || !aff)
                    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                    if(cur.ok[v])
                        HIPTK_STORE_D((u32x4_t*)(Dp + cur.doff[v]), o[v]);
                wave_lds_fence();
            }
            };
            // Two slabs in flight.  One copy of the code per case (C read or not; offsets computed):
            // where the choice is made at run time inside the loop, the compiler has to wait for
            // every outstanding load wherever the paths join, and the overlap below is lost.
            auto run = [&](auto aff_c, auto bil_c) {
            constexpr bool aff = decltype(aff_c)::value;
            constexpr bool bil = decltype(bil_c)::value;
            // The C vectors of a slab are requested two slabs ahead of their use, and the table
            // look-ups behind their addresses one slab before that.  (The compiler cannot move any
            // of this itself: D may alias C and, for all it knows, the offset tables.)  Loads and
            // stores complete in issue order, so a wait for a load also waits for every store issued
            // before it: with this lead the youngest stores such a wait can catch are a slab old,
            // and C loads, LDS staging and D stores of neighbouring slabs overlap.  A lane reads
            // each C element before it writes the D element at the same place, and no lane reads an
            // element another lane writes, so exact aliasing stays valid.
            uint32_t dqo[NVEC], cqo[NVEC];
            bool     qok[NVEC];
#pragma unroll
            for(int v = 0; v < NVEC; v++)
            {
                const int q = qw + ((v * 64 + lane) % VPR) * 8;
                qok[v]      = q_in8(q);
                // affine C / D (every benchmark-style packed layout): offsets are computed; else
                // looked up (the tables are padded beyond every index a tile reaches, with the
                // offset of index 0, so the look-ups need no guard)
                dqo[v] = aff ? (uint32_t)q * (uint32_t)a.dq_stride : (uint32_t)a.dq[q];
                cqo[v] = !bil ? 0u : aff ? (uint32_t)q * (uint32_t)a.cq_stride : (uint32_t)a.cq[q];
            }
            struct Offsets
            {
                uint32_t d[NVEC], c[NVEC];
                bool     ok[NVEC];
            };
            auto prepare = [&](int i, Offsets& o) {
#pragma unroll
                for(int v = 0; v < NVEC; v++)
                {
                    const int p        = pw + i * 32 + (v * 64 + lane) / VPR;
                    o.ok[v]            = qok[v] && p_in(p);
                    const uint32_t dpo = aff ? (uint32_t)p * (uint32_t)a.dp_stride : (uint32_t)a.dp[p];
                    const uint32_t cpo = !bil ? 0u : aff ? (uint32_t)p * (uint32_t)a.cp_stride : (uint32_t)a.cp[p];
                    // a vector outside the extents reads element 0 of C, a valid address, and is not stored
                    o.d[v] = o.ok[v] ? dpo + dqo[v] : 0u;
                    o.c[v] = o.ok[v] ? cpo + cqo[v] : 0u;
                }
            };
            // two slabs in flight, and the offsets of the slab that is requested next
            constexpr int NB = 2;
            Offsets       off[NB], nxt;
            u32x4_t       cbuf[NB][NVEC];
            auto          request = [&](int b) {
                if(bil)
                {
#pragma unroll
                    for(int v = 0; v < NVEC; v++)
                        cbuf[b][v] = *(const u32x4_t*)(Cp + off[b].c[v]);
                }
            };
            // Two staging buffers per wave when the operand buffers have room for them: slab
            // i+1 is written to LDS while slab i is read back, converted and stored.
            constexpr bool DB = 2 * 32 * EP * 4 * WP * WQ <= LDSCAP;
            float* const   st0 = (float*)lds + wave * ((DB ? 2 : 1) * 32 * EP);
            auto write_slab = [&](int i, float* dst) {
#pragma unroll
                for(int u = 0; u < QUADS; u++)
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        dst[(Acc::row0(u, lane) + e) * EP + Acc::col(u, lane)] = acc.get(i, u, e);
            };
            // (all look-ups of the first two slabs before their first C load: one wait, not two)
            prepare(0, off[0]);
            if constexpr(TP > 1)
                prepare(1, off[1]);
            request(0);
            if constexpr(TP > 1)
                request(1);
            if constexpr(TP > NB)
                prepare(NB, nxt);
            if constexpr(DB)
            {
                write_slab(0, st0);
                wave_lds_fence();
            }
#pragma unroll
            for(int i = 0; i < TP; i++)
            {
                const float* cur_st = st0 + (DB ? (i & 1) * 32 * EP : 0);
                if constexpr(DB)
                {
                    if(i + 1 < TP)
                        write_slab(i + 1, st0 + ((i + 1) & 1) * 32 * EP);
                }
                else
                {
                    write_slab(i, st0);
                    wave_lds_fence();
                }
                // up to four of the slab's vectors are read from LDS together, then converted and stored
                constexpr int HV = NVEC > 4 ? 4 : NVEC;
#pragma unroll
                for(int h = 0; h < NVEC; h += HV)
                {
                    f32x4_t lo[HV], hi[HV];
#pragma unroll
                    for(int w = 0; w < HV; w++)
                    {
                        const int    slot = (h + w) * 64 + lane;
                        const float* src  = cur_st + (slot / VPR) * EP + (slot % VPR) * 8;
                        lo[w]             = *(const f32x4_t*)src;
                        hi[w]             = *(const f32x4_t*)(src + 4);
                    }
                    u32x4_t o[HV];
#pragma unroll
                    for(int w = 0; w < HV; w++)
                    {
                        float v8[8] = {lo[w][0], lo[w][1], lo[w][2], lo[w][3], hi[w][0], hi[w][1], hi[w][2], hi[w][3]};
                        if(bil)
                        {
                            const u32x4_t c4 = cbuf[i % NB][h + w];
#pragma unroll
                            for(int e = 0; e < 8; e++)
                            {
                                const uint16_t cb = (uint16_t)(c4[e >> 1] >> ((e & 1) * 16));
                                v8[e]             = alpha * v8[e] + beta * Tr::to_f32(cb);
                            }
                        }
                        else
                        {
#pragma unroll
                            for(int e = 0; e < 8; e++)
                                v8[e] = alpha * v8[e];
                        }
#pragma unroll
                        for(int e = 0; e < 4; e++)
                            o[w][e] = (uint32_t)Tr::from_f32(v8[2 * e]) | ((uint32_t)Tr::from_f32(v8[2 * e + 1]) << 16);
                    }
#pragma unroll
                    for(int w = 0; w < HV; w++)
                        if(off[i % NB].ok[h + w])
                            HIPTK_STORE_D((u32x4_t*)(Dp + off[i % NB].d[h + w]), o[w]);
                }
                // this slab's registers are free: request the slab NB ahead, then look up the
                // offsets of the one after that
                if(i + NB < TP)
                {
                    off[i % NB] = nxt;
                    request(i % NB);
                }
                if(i + NB + 1 < TP)
                    prepare(i + NB + 1, nxt);
                wave_lds_fence();
            }
            };
            typedef std::integral_constant<bool, true>  Yes;
            typedef std::integral_constant<bool, false> No;
            // The 128-wide wave tiles of the four-wave kernels hold 8 vectors per lane and slab and
            // have no registers to spare for a second slab.  With offsets from the tables the
            // deeper lead did not pay either (rank-6 benchmark layout: 366-372 us against 374).
            if constexpr(NVEC * TP > 16 && !DEEP)
                one_in_flight();
            else
            {
                if(a.cd_affine == 0)
                    one_in_flight();
                else if(a.bilinear != 0)
                    run(Yes{}, Yes{});
                else
                    run(Yes{}, No{});
            }
            return;
        }
        {
            // Element by element through the offset tables.  D may alias C (and, for all the
            // compiler knows, the tables), so it would fetch one offset, one C element and store
            // one D element at a time; the offsets of a slab's 16 rows are therefore fetched once,
            // ahead of the columns, and the 16 C elements of a column before the first store.
            constexpr int NCOL = Acc::NCOL, NRQ = Acc::NRQ, NROW = 4 * NRQ; // a lane's columns, and its rows per slab
            const int     pw = p0 + wp * WTP;
            const int     qw = q0 + wq * WTQ;
            const bool    bil = a.bilinear != 0;
            uint32_t      dqo[NCOL], cqo[NCOL];
            bool          qok[NCOL];
#pragma unroll
            for(int j = 0; j < NCOL; j++)
            {
                const int q = qw + Acc::col(j * NRQ, lane);
                qok[j]      = q_in(q);
                // (the tables are padded beyond every index a tile can reach, with the offset of
                // index 0: loads need no guard, only the stores do)
                dqo[j] = (uint32_t)a.dq[q];
                cqo[j] = bil ? (uint32_t)a.cq[q] : 0u;
            }
#pragma unroll
            for(int i = 0; i < TP; i++)
            {
                uint32_t dpo[NROW], cpo[NROW];
                bool     pok[NROW];
#pragma unroll
                for(int r = 0; r < NROW; r++)
                {
                    const int p = pw + i * 32 + Acc::row0(r >> 2, lane) + (r & 3);
                    pok[r]      = p_in(p);
                    dpo[r]      = (uint32_t)a.dp[p];
                    cpo[r]      = bil ? (uint32_t)a.cp[p] : 0u;
                }
#pragma unroll
                for(int j = 0; j < NCOL; j++)
                {
                    if(!qok[j])
                        continue;
                    float c[NROW];
#pragma unroll
                    for(int r = 0; r < NROW; r++)
                        c[r] = 0.f;
                    if(bil)
                    {
#pragma unroll
                        for(int r = 0; r < NROW; r++)
                            c[r] = Tr::out_to_f32(Cp[cpo[r] + cqo[j]]);
                    }
#pragma unroll
                    for(int r = 0; r < NROW; r++)
                        if(pok[r])
                            Dp[dpo[r] + dqo[j]] = Tr::out_from_f32(Tr::axpby(alpha, acc.get(i, j * NRQ + (r >> 2), r & 3), beta, c[r], bil));
                }
            }
        }
    }

    // ... for accumulators of v_mfma_f32_32x32x16 blocks
    template <typename Tr, int WP, int WQ, int TP, int TQ, int LDSCAP, bool DEEP = false>
    __device__ __forceinline__ void epilogue_h(const KArgs& a, f32x16_t (&acc)[TP][TQ], uint16_t* lds, int p0, int q0, int p_own, int q_own)
    {
        epilogue_acc<Tr, WP, WQ, TP, TQ, LDSCAP, DEEP>(a, Acc32<TP, TQ>{acc}, lds, p0, q0, p_own, q_own);
    }
    // ... and of v_mfma_f32_16x16x32 blocks (TP x TQ still counts blocks of 32 x 32)
    template <typename Tr, int WP, int WQ, int TP, int TQ, int LDSCAP, bool DEEP = false>
    __device__ __forceinline__ void epilogue_h16(const KArgs& a, f32x4_t (&acc)[2 * TP][2 * TQ], uint16_t* lds, int p0, int q0, int p_own, int q_own)
    {
        epilogue_acc<Tr, WP, WQ, TP, TQ, LDSCAP, DEEP>(a, Acc16<TP, TQ>{acc}, lds, p0, q0, p_own, q_own);
    }

    template <typename Tr,
              int  BP,
              int  BQ,
              int  BK,
              int  WP,
              int  WQ,
              bool XKF,
              bool YKF,
              int  XV,
              int  YV,
              bool KAFF,
              bool PIPE>
    __global__ void __launch_bounds__(WP* WQ * 64, ((BP / WP) * (BQ / WQ) > 128 * 64 ? 1 : 2)) contract_h_kernel(const KArgs a)
    {
        constexpr int NT  = WP * WQ * 64;
        constexpr int WTP = BP / WP, WTQ = BQ / WQ;
        constexpr int TP = WTP / 32, TQ = WTQ / 32;
        static_assert(WTP % 32 == 0 && WTQ % 32 == 0 && BK % 16 == 0, "tile shape");
        typedef TileLds<XKF, BP, BK> LX;
        typedef TileLds<YKF, BQ, BK> LY;
        constexpr int STAGE = LX::ELEMS + LY::ELEMS;

        extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

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

        const int kt_begin = blockIdx.z * a.ktiles_per_split;
        int       kt_end   = kt_begin + a.ktiles_per_split;
        const int kt_all   = (a.K + BK - 1) / BK;
        if(kt_end > kt_all)
            kt_end = kt_all;

        Stager<Tr, XKF, XV, BP, BK, NT, KAFF> sx;
        Stager<Tr, YKF, YV, BQ, BK, NT, KAFF> sy;
        sx.init(a.xp, p0, tid);
        sy.init(a.yq, q0, tid);

        f32x16_t acc[TP][TQ];
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int j = 0; j < TQ; j++)
#pragma unroll
                for(int r = 0; r < 16; r++)
                    acc[i][j][r] = 0.f;

        const int xbase = frag_base<XKF, LX::PITCH>(lane) + (XKF ? wp * WTP * LX::PITCH : wp * WTP);
        const int ybase = frag_base<YKF, LY::PITCH>(lane) + (YKF ? wq * WTQ * LY::PITCH : wq * WTQ);

        // tiles below kt_full lie entirely inside K
        const int kt_full = a.K / BK;

        auto fetch_tile = [&](int t) {
            if(t < kt_full)
            {
                sx.template fetch<false>(a.X, t * BK, a.K, a.xk_stride);
                sy.template fetch<false>(a.Y, t * BK, a.K, a.yk_stride);
            }
            else
            {
                sx.template fetch<true>(a.X, t * BK, a.K, a.xk_stride);
                sy.template fetch<true>(a.Y, t * BK, a.K, a.yk_stride);
            }
        };
        auto compute = [&](const uint16_t* lx, const uint16_t* ly, int ks) {
            u32x4_t xf[TP], yf[TQ];
#pragma unroll
            for(int i = 0; i < TP; i++)
                xf[i] = frag_load<XKF, LX::PITCH>(lx, xbase, i * 32, ks);
#pragma unroll
            for(int j = 0; j < TQ; j++)
                yf[j] = frag_load<YKF, LY::PITCH>(ly, ybase, j * 32, ks);
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int j = 0; j < TQ; j++)
                    acc[i][j] = Tr::mfma(xf[i], yf[j], acc[i][j]);
        };
        constexpr int KS = BK / 16;

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
            sy.commit(lds + LX::ELEMS);
            if(kt_begin + 1 < kt_end)
            {
                fetch_tile(kt_begin + 1);
                sx.load_koffs(a.xk, (kt_begin + 2) * BK);
                sy.load_koffs(a.yk, (kt_begin + 2) * BK);
            }
            lds_barrier();
        }

        int buf = 0;
        int kt  = kt_begin;
        // steady state: tile kt+2 exists and is a full tile
        const int steady_end = (kt_end < kt_full ? kt_end : kt_full) - 2;
        if constexpr(PIPE)
        {
            // Register-level pipeline for one wavefront per SIMD: the MFMA operands of
            // k-substep s+1 are read from LDS while substep s is multiplied, across the tile
            // boundary as well.  The tile's barrier sits between substeps KS-2 and KS-1: by
            // then every wave has issued its last reads of the current buffer and finished
            // writing the next one, so substep KS-1 overlaps the first operand reads of the
            // next tile.  sched_group_barrier pins the interleaving of MFMA, LDS and global
            // instructions that the compiler would otherwise bunch together.
            static_assert(KS >= 4 && KS % 2 == 0, "pipelined loop needs an even number of k-substeps");
            constexpr int RX = TP * (XKF ? 1 : 2), RY = TQ * (YKF ? 1 : 2); // LDS reads per substep
            constexpr int NM = TP * TQ; // MFMAs per substep
            u32x4_t       xf[2][TP], yf[2][TQ];
            auto load_frags = [&](const uint16_t* lx, const uint16_t* ly, int ks, int slot) {
#pragma unroll
                for(int i = 0; i < TP; i++)
                    xf[slot][i] = frag_load<XKF, LX::PITCH>(lx, xbase, i * 32, ks);
#pragma unroll
                for(int j = 0; j < TQ; j++)
                    yf[slot][j] = frag_load<YKF, LY::PITCH>(ly, ybase, j * 32, ks);
            };
            auto mma = [&](int slot) {
#pragma unroll
                for(int i = 0; i < TP; i++)
#pragma unroll
                    for(int j = 0; j < TQ; j++)
                        acc[i][j] = Tr::mfma(xf[slot][i], yf[slot][j], acc[i][j]);
            };
            // NM MFMAs with the substep's LDS reads spread over the first half of them and
            // `extra` instructions of class `mask` (LDS writes or global loads) over the rest
            auto interleave = [&](auto mask_c, auto extra_c) {
                constexpr int mask  = decltype(mask_c)::value;
                constexpr int extra = decltype(extra_c)::value;
                constexpr int H     = NM / 2;
                constexpr int RPM   = (RX + RY + H - 1) / H;
                constexpr int EPM   = (extra + (NM - H) - 1) / (NM - H);
#pragma unroll
                for(int m = 0; m < H; m++)
                {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, RPM, 0);
                }
#pragma unroll
                for(int m = H; m < NM; m++)
                {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if constexpr(extra > 0)
                        __builtin_amdgcn_sched_group_barrier(mask, EPM, 0);
                }
            };
            typedef std::integral_constant<int, 0x200> DsWrite;
            typedef std::integral_constant<int, 0x020> VmemRead;
            if(kt < steady_end)
                load_frags(lds, lds + LX::ELEMS, 0, 0);
            for(; kt < steady_end; kt++)
            {
                const uint16_t* lx = lds + buf * STAGE;
                const uint16_t* ly = lx + LX::ELEMS;
                uint16_t*       nx = lds + (buf ^ 1) * STAGE;
                uint16_t*       ny = nx + LX::ELEMS;
#pragma unroll
                for(int ks = 0; ks < KS; ks++)
                {
                    if(ks == KS - 1)
                    {
                        lds_barrier();
                        load_frags(nx, ny, 0, (ks + 1) & 1);
                    }
                    else
                        load_frags(lx, ly, ks + 1, (ks + 1) & 1);
                    mma(ks & 1);
                    // an operand's staging registers are refilled right after they are stored:
                    // the gather of tile kt+2 then has a whole tile of MFMA time to arrive
                    if(ks == 0)
                    {
                        sx.commit(nx);
                        sx.template fetch<false>(a.X, (kt + 2) * BK, a.K, a.xk_stride);
                        sx.load_koffs(a.xk, (kt + 3) * BK);
                        interleave(DsWrite{}, std::integral_constant<int, decltype(sx)::N>{});
                    }
                    else if(ks == 1)
                    {
                        sy.commit(ny);
                        sy.template fetch<false>(a.Y, (kt + 2) * BK, a.K, a.yk_stride);
                        sy.load_koffs(a.yk, (kt + 3) * BK);
                        interleave(DsWrite{}, std::integral_constant<int, decltype(sy)::N>{});
                    }
                    else
                        interleave(DsWrite{}, std::integral_constant<int, 0>{});
                }
                buf ^= 1;
            }
        }
        else
        for(; kt < steady_end; kt++)
        {
            const uint16_t* lx = lds + buf * STAGE;
            const uint16_t* ly = lx + LX::ELEMS;
            uint16_t*       nx = lds + (buf ^ 1) * STAGE;
            uint16_t*       ny = nx + LX::ELEMS;
#pragma unroll
            for(int ks = 0; ks < KS; ks++)
            {
                compute(lx, ly, ks);
                // registers of an operand are refilled right after they are stored, so a
                // gather has a whole tile's worth of MFMA time to arrive
                if(ks == 0)
                {
                    sx.commit(nx);
                    sx.template fetch<false>(a.X, (kt + 2) * BK, a.K, a.xk_stride);
                    sx.load_koffs(a.xk, (kt + 3) * BK);
                }
                if(ks == (KS > 1 ? 1 : 0))
                {
                    sy.commit(ny);
                    sy.template fetch<false>(a.Y, (kt + 2) * BK, a.K, a.yk_stride);
                    sy.load_koffs(a.yk, (kt + 3) * BK);
                }
            }
            lds_barrier();
            buf ^= 1;
        }
        // drain: at most the last three tiles (and every tile of a short K)
        for(; kt < kt_end; kt++)
        {
            const uint16_t* lx = lds + buf * STAGE;
            const uint16_t* ly = lx + LX::ELEMS;
            uint16_t*       nx = lds + (buf ^ 1) * STAGE;
            uint16_t*       ny = nx + LX::ELEMS;
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
            lds_barrier();
            buf ^= 1;
        }

        epilogue_h<Tr, WP, WQ, TP, TQ, 2 * STAGE * 2>(a, acc, lds, p0, q0, p_own, q_own);
    }

    template <typename Tr,
              int  BP,
              int  BQ,
              int  BK,
              int  WP,
              int  WQ,
              bool XKF,
              bool YKF,
              int  XV,
              int  YV,
              bool KAFF,
              bool PIPE>
    int launch_h(const KArgs& a, hipStream_t stream)
    {
        typedef TileLds<XKF, BP, BK> LX;
        typedef TileLds<YKF, BQ, BK> LY;
        constexpr int                LDS = 2 * (LX::ELEMS + LY::ELEMS) * 2;
        auto kern = contract_h_kernel<Tr, BP, BQ, BK, WP, WQ, XKF, YKF, XV, YV, KAFF, PIPE>;
        static const hipError_t attr = hipFuncSetAttribute(
            (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if(attr != hipSuccess)
            return (int)attr;
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(kern, grid, dim3(WP * WQ * 64), LDS, stream, a);
        return (int)hipGetLastError();
    }

    template <int BP, int BQ, int BK, bool XKF, bool YKF>
    constexpr int lds_bytes_h()
    {
        return 2 * (TileLds<XKF, BP, BK>::ELEMS + TileLds<YKF, BQ, BK>::ELEMS) * 2;
    }
}

// One registry line: class traits, tile id, tile shape, wave grid, layouts, vectors,
// affine-K flag.
#define HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, XKF, YKF, XV, YV, KAFF)                   \
    {                                                                                       \
        TR::CLS, ID, XKF, YKF, XV, YV, KAFF, BP, BQ, BK, WP *WQ * 64,                       \
            hiptk::lds_bytes_h<BP, BQ, BK, XKF, YKF>(),                                     \
            #TR "_" #BP "x" #BQ "x" #BK "_x" #XKF #XV "_y" #YKF #YV "_kaff" #KAFF,          \
            &hiptk::launch_h<hiptk::TR, BP, BQ, BK, WP, WQ, XKF, YKF, XV, YV, KAFF, false>  \
    }

// The same with the register-level pipeline (one wavefront per SIMD, accumulators in AGPRs).
#define HIPTK_HP_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, XKF, YKF, XV, YV, KAFF)                  \
    {                                                                                       \
        TR::CLS, ID, XKF, YKF, XV, YV, KAFF, BP, BQ, BK, WP *WQ * 64,                       \
            hiptk::lds_bytes_h<BP, BQ, BK, XKF, YKF>(),                                     \
            #TR "_" #BP "x" #BQ "x" #BK "_x" #XKF #XV "_y" #YKF #YV "_kaff" #KAFF "_pipe" #WP "x" #WQ, \
            &hiptk::launch_h<hiptk::TR, BP, BQ, BK, WP, WQ, XKF, YKF, XV, YV, KAFF, true>   \
    }

// The four layout combinations of a tile whose operands are both gathered V wide.
#define HIPTK_H_TILE_VV(TR, ID, BP, BQ, BK, WP, WQ, V, KAFF)                   \
    HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, true, V, V, KAFF),         \
        HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, false, V, V, KAFF),    \
        HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, false, true, V, V, KAFF),    \
        HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, false, false, V, V, KAFF)
#define HIPTK_H_TILE_V8(TR, ID, BP, BQ, BK, WP, WQ, KAFF) HIPTK_H_TILE_VV(TR, ID, BP, BQ, BK, WP, WQ, 8, KAFF)
#define HIPTK_HP_TILE_VV(TR, ID, BP, BQ, BK, WP, WQ, V, KAFF)                   \
    HIPTK_HP_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, true, V, V, KAFF),         \
        HIPTK_HP_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, false, V, V, KAFF),    \
        HIPTK_HP_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, false, true, V, V, KAFF),    \
        HIPTK_HP_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, false, false, V, V, KAFF)
#define HIPTK_HP_TILE_V8(TR, ID, BP, BQ, BK, WP, WQ, KAFF) HIPTK_HP_TILE_VV(TR, ID, BP, BQ, BK, WP, WQ, 8, KAFF)

// Combinations in which at least one operand is a scalar gather (always staged k-fast).
#define HIPTK_H_TILE_V1V(TR, ID, BP, BQ, BK, WP, WQ, V)                     \
    HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, true, 1, 1, false),     \
        HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, true, V, 1, false), \
        HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, false, true, V, 1, false), \
        HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, true, 1, V, false), \
        HIPTK_H_ENTRY(TR, ID, BP, BQ, BK, WP, WQ, true, false, 1, V, false)
#define HIPTK_H_TILE_V1(TR, ID, BP, BQ, BK, WP, WQ) HIPTK_H_TILE_V1V(TR, ID, BP, BQ, BK, WP, WQ, 8)
