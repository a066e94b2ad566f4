// 32/64-bit (f32, f64, complex f32) contraction kernel for gfx950 whose operand tiles go from global
// memory straight into LDS (global_load_lds_dwordx4), for the layout in which both operands are
// contiguous along their row index (packed column-major: every benchmark configuration of these
// types).  (Complex f64 is not instantiated: two K tiles of its operands do not fit the registers,
// and without them it measured 8 % behind the eight-wave tile of contract_w.hpp.)
//
// Same MFMA use, complex product and epilogue as contract_w.hpp; what differs is how a tile gets
// into LDS and from there into registers.  There, a gather passes through registers and has one K
// tile of MFMA time to arrive, which a CU covers only when several workgroups share it.  Here:
//
//   * 64 x 64 output tile on four waves (wave tile 32 x 32), K in steps of BK, a ring of NS LDS stages
//     (tile[k][64 rows] of X, then of Y; one element per lane and MFMA operand, consecutive lanes
//     read consecutive rows: unpadded rows are conflict free here, no swizzle).  A direct load writes
//     64 lanes x 16 bytes to consecutive LDS addresses: 16 / sizeof(element) consecutive rows at one k
//     per lane, 1 KiB per instruction, each wave loading its share of a stage.
//   * A wave holds the operands of two K tiles in registers: while tile t is multiplied, tile t + 1 is
//     read from LDS and tile t + NS is requested into the stage tile t has just left, so a load has
//     NS - 1 tiles of MFMA time to land and an LDS read one: the lead a single resident workgroup
//     needs (1024 x 1024 x 512 complex f32 in one pass: 59 us through registers, 48 us here).  The
//     order of MFMAs, requests and reads inside a K tile is fixed by hand (see `step`).
//   * The loads are inline assembly (dma_lds.hpp), invisible to the compiler, so the waits are placed
//     by hand: loads complete in issue order, and before the barrier that hands tile t + 1 to the
//     readers each wave waits until only the loads of the NS - 2 tiles after it are outstanding.
//     Tiles requested beyond the K range are not branched around: they re-read the last tile into
//     spare LDS behind the ring, so every wait sees the same number of younger loads.
//
// Restrictions (the dispatcher checks them): both operands gathered in 16-byte vectors along their
// row index, on 16-byte boundaries; one K stride per operand; K a multiple of BK; byte offsets inside
// each operand below 2^32.
#pragma once
#include <utility>

#include "contract_w.hpp"
#include "dma_lds.hpp"
#include "hd_addr.hpp"

namespace hiptk
{
    // f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
    template <typename F, int... I>
    __device__ __forceinline__ void wd_static_for_impl(F& f, std::integer_sequence<int, I...>)
    {
        (f(std::integral_constant<int, I>{}), ...);
    }
    template <int N, typename F>
    __device__ __forceinline__ void wd_static_for(F&& f)
    {
        wd_static_for_impl(f, std::make_integer_sequence<int, N>{});
    }

    template <typename Tr, int BK, int NS>
    struct WdGeom
    {
        static constexpr int BP = 64, BQ = 64;
        static constexpr int ES       = (int)sizeof(typename Tr::S);
        static constexpr int V        = 16 / ES; // elements per 16-byte vector
        static constexpr int OP_BYTES = BK * 64 * ES; // one operand in one stage
        static constexpr int NLW      = OP_BYTES / 4096; // direct loads (1 KiB) per wave, operand and K tile
        static constexpr int STAGE_BYTES = 2 * OP_BYTES;
        static constexpr int RING        = NS * STAGE_BYTES;
        static constexpr int SPARE       = RING; // NLW KiB per wave: where loads beyond the K range land
        static constexpr int LDS_BYTES   = RING + 4 * NLW * 1024;
        static_assert(OP_BYTES % 4096 == 0 && NLW >= 1, "every wave loads whole KiB of an operand stage");
        static_assert(std::is_same<typename Tr::S, typename Tr::E>::value, "a direct load cannot convert");
        static_assert(NS >= 4 && NS % 2 == 0 && (NS - 1) * 2 * NLW < 64, "the wait counts must fit vmcnt");
        static_assert(LDS_BYTES <= 160 * 1024, "LDS of one CU");
    };

    template <typename Tr, int BK, int NS>
    __global__ void __launch_bounds__(256, 2) contract_wd_kernel(const KArgs a)
    {
        typedef WdGeom<Tr, BK, NS> G;
        typedef typename Tr::S     S;
        constexpr int              TILE = Tr::TILE;
        constexpr int              TP = 32 / TILE, TQ = 32 / TILE;
        constexpr int              KS = BK / Tr::KM;
        constexpr int              NLW = G::NLW, ES = G::ES;
        constexpr int              LPT = 2 * NLW; // loads per wave and K tile
        static_assert(BK % Tr::KM == 0, "whole MFMA k-steps per tile");

        extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

        const int tid  = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wp   = wave >> 1;
        const int wq   = wave & 1;

        int tp, tq;
        tile_coords(blockIdx.x, a.tiles_p, a.tiles_q, tp, tq);
        // (no tile is moved back: the dispatcher offers this kernel only without shift_p / shift_q; a
        // tile that overhangs P or Q reads the padding of the row tables, offset 0, and stores nothing there)
        const int p0 = tp * G::BP, q0 = tq * G::BQ;

        const int kt_begin = blockIdx.z * a.ktiles_per_split;
        int       kt_end   = kt_begin + a.ktiles_per_split;
        const int kt_all   = a.K / BK; // K is a multiple of BK
        if(kt_end > kt_all)
            kt_end = kt_all;
        const int nt = kt_end - kt_begin;

        // this lane's 16 bytes of each of its loads, as byte offsets from the tile's k origin
        uint32_t xv[NLW], yv[NLW];
#pragma unroll
        for(int i = 0; i < NLW; i++)
        {
            const HdSlot sl = wd_slot<G::V>((wave * NLW + i) * 64 + lane);
            xv[i]           = (uint32_t)ES * ((uint32_t)a.xp[p0 + sl.row] + (uint32_t)sl.k * (uint32_t)a.xk_stride);
            yv[i]           = (uint32_t)ES * ((uint32_t)a.yq[q0 + sl.row] + (uint32_t)sl.k * (uint32_t)a.yk_stride);
        }
        // k origin of the next tile to be requested (tiles beyond the slice's last one repeat it), as a
        // 32-bit byte offset from the operand's base, kept in scalar registers
        const uint32_t xkb   = (uint32_t)ES * (uint32_t)a.xk_stride;
        const uint32_t ykb   = (uint32_t)ES * (uint32_t)a.yk_stride;
        const int      klast = (kt_begin + nt - 1) * BK;
        int            ko    = kt_begin * BK;
        int            lu    = 0; // index of the next tile to be requested
        const char*    xsrc  = (const char*)a.X + (uint64_t)((uint32_t)ko * xkb);
        const char*    ysrc  = (const char*)a.Y + (uint64_t)((uint32_t)ko * ykb);

        typedef unsigned char __attribute__((address_space(3))) * lds_u8_ptr;
        const uint32_t lds0   = (uint32_t)(uintptr_t)(lds_u8_ptr)lds_raw; // LDS byte address of the ring
        const uint32_t wdx    = lds0 + (uint32_t)wave * (NLW * 1024u); // this wave's share of an X stage
        const uint32_t wdy    = wdx + G::OP_BYTES;
        const uint32_t wspare = lds0 + G::SPARE + (uint32_t)wave * (NLW * 1024u);

        // request tile `lu` into ring stage ST
        auto issue = [&](auto st_c) {
            constexpr int  ST   = decltype(st_c)::value;
            const bool     real = lu < nt;
            const uint32_t dx   = real ? wdx + ST * G::STAGE_BYTES : wspare;
            const uint32_t dy   = real ? wdy + ST * G::STAGE_BYTES : wspare;
#pragma unroll
            for(int i = 0; i < NLW; i++)
            {
                dma_dst_at(dx, i * 1024);
                dma_load(xv[i], xsrc);
            }
#pragma unroll
            for(int i = 0; i < NLW; i++)
            {
                dma_dst_at(dy, i * 1024);
                dma_load(yv[i], ysrc);
            }
            lu++;
            ko   = wd_next_origin(ko, klast, BK);
            xsrc = (const char*)a.X + (uint64_t)((uint32_t)ko * xkb);
            ysrc = (const char*)a.Y + (uint64_t)((uint32_t)ko * ykb);
        };

        typename Tr::Acc acc[TP][TQ];
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int j = 0; j < TQ; j++)
                Tr::zero(acc[i][j]);

        const int row   = lane & (TILE - 1);
        const int kslot = Tr::kslot(lane);
        const int xfo   = kslot * 64 + wp * 32 + row;
        const int yfo   = kslot * 64 + wq * 32 + row;

        // This wave's operands of one K tile, in registers: tile t + 1 is read from LDS while tile t
        // is multiplied, so that a wave alone on its SIMD does not wait for LDS either.
        struct Frags
        {
            S x[KS][TP], y[KS][TQ];
        };
        Frags fr[2];
        // the operands of k-step ks of the tile in ring stage ST
        auto read_k = [&](auto st_c, Frags& f, int ks) {
            constexpr int ST = decltype(st_c)::value;
            const S*      lx = (const S*)(lds_raw + ST * G::STAGE_BYTES);
            const S*      ly = (const S*)(lds_raw + ST * G::STAGE_BYTES + G::OP_BYTES);
#pragma unroll
            for(int i = 0; i < TP; i++)
                f.x[ks][i] = lx[xfo + ks * Tr::KM * 64 + i * TILE];
#pragma unroll
            for(int j = 0; j < TQ; j++)
                f.y[ks][j] = ly[yfo + ks * Tr::KM * 64 + j * TILE];
        };
        auto read_tile = [&](auto st_c, Frags& f) {
#pragma unroll
            for(int ks = 0; ks < KS; ks++)
                read_k(st_c, f, ks);
        };
        auto mma_k = [&](const Frags& f, int ks) {
            typename Tr::XF xf[TP];
            typename Tr::YF yf[TQ];
#pragma unroll
            for(int i = 0; i < TP; i++)
                xf[i] = Tr::prep_x(f.x[ks][i], lane);
#pragma unroll
            for(int j = 0; j < TQ; j++)
                yf[j] = Tr::prep_y(f.y[ks][j], lane);
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int j = 0; j < TQ; j++)
                    Tr::mma(xf[i], yf[j], acc[i][j]);
        };
        int t = 0;
        // K tile t, in ring stage ST = t % NS and (already) in fr[ST & 1].  The order is fixed by hand
        // (the scheduler may not move anything across the marks): the first k-step's MFMAs cover the
        // wait and the barrier; the requests for tile t + NS and the LDS reads of tile t + 1 go
        // between the MFMAs of the other k-steps, the last reads one k-step before the end, so that
        // the next barrier does not wait for them.
        auto step = [&](auto st_c) {
            constexpr int ST = decltype(st_c)::value;
            typedef std::integral_constant<int, (ST + 1) % NS> Next;
            Frags&        cur = fr[ST & 1];
            Frags&        nxt = fr[(ST + 1) & 1];
            mma_k(cur, 0);
            __builtin_amdgcn_sched_barrier(0);
            // tile t + 1 has landed when only the loads of the NS - 2 tiles after it are outstanding;
            // behind the barrier every wave sees it, and every wave has tile t in registers
            __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * LPT));
            w_lds_barrier();
            issue(st_c); // tile t + NS, into tile t's stage
            // (behind the slice's last tile these read a stage nothing was loaded into, for nobody)
            if constexpr(KS == 1)
                read_k(Next{}, nxt, 0);
#pragma unroll
            for(int ks = 1; ks < KS; ks++)
            {
                read_k(Next{}, nxt, ks - 1);
                if(ks == 1)
                    read_k(Next{}, nxt, KS - 1);
                __builtin_amdgcn_sched_barrier(0);
                mma_k(cur, ks);
                __builtin_amdgcn_sched_barrier(0);
            }
            t++;
        };
        static_assert(NS % 2 == 0, "the register copies alternate with the ring stages");
        if(nt > 0)
        {
            wd_static_for<NS>(issue); // tiles 0 .. NS - 1
            __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 1) * LPT));
            w_lds_barrier();
            read_tile(std::integral_constant<int, 0>{}, fr[0]);
            while(t + NS <= nt)
                wd_static_for<NS>(step);
            wd_static_for<NS - 1>([&](auto i_c) {
                if(t < nt)
                    step(i_c);
            });
        }
        epilogue_w<Tr, TP, TQ>(a, acc, p0 + wp * 32, q0 + wq * 32 + Tr::q_of(lane), p0, q0, lane);
        // the loads beyond the K range (into the spare KiB) must not outlive the workgroup's LDS
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    }

    template <typename Tr, int BK, int NS>
    int launch_wd(const KArgs& a, hipStream_t stream)
    {
        typedef WdGeom<Tr, BK, NS> G;
        if(a.K < BK || a.K % BK != 0 || a.shift_p || a.shift_q)
            return (int)hipErrorInvalidValue;
        auto                    kern = contract_wd_kernel<Tr, BK, NS>;
        static const hipError_t attr = hipFuncSetAttribute(
            (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if(attr != hipSuccess)
            return (int)attr;
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(kern, grid, dim3(256), G::LDS_BYTES, stream, a);
        return (int)hipGetLastError();
    }
}

// Registry line of a direct-load tile: both operands in row-index vectors, one K stride, K a multiple of BK.
// (A class whose element fills the 16 bytes would have no vectors: every problem of it is described
// as "scalar, k-fast", and any row table would do.)
#define HIPTK_WD_ENTRY(TR, ID, BK, NS)                                                              \
    {                                                                                               \
        hiptk::TR::CLS, ID, hiptk::TR::VMAX == 1, hiptk::TR::VMAX == 1, hiptk::TR::VMAX,            \
            hiptk::TR::VMAX, 1, 64, 64, BK, 256,                                                    \
            hiptk::WdGeom<hiptk::TR, BK, NS>::LDS_BYTES, #TR "_64x64x" #BK "_direct" #NS,        \
            &hiptk::launch_wd<hiptk::TR, BK, NS>, BK                                                  \
    }
