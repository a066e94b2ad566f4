// 16-bit (f16 / bf16) contraction kernel for gfx950 whose operand tiles go from global memory
// straight into LDS (global_load_lds_dwordx4), without passing through registers.
//
// Same problem statement and epilogue as contract_h.hpp; what differs is the main loop:
//
//   * 256 x 256 output tile on four wavefronts (one per SIMD, wave tile 128 x 128), K in steps of 32,
//     four LDS stages of 32 KiB (16 KiB per operand) used as a ring.  The loads of K tile t + 4 are
//     issued while tile t and t + 1 are multiplied, so a load has two to three tiles of MFMA time to
//     land, and no staging registers, no register -> LDS stores and no write bank conflicts remain.
//   * A direct load writes 64 lanes x 16 bytes to consecutive LDS addresses, so rows cannot be padded.
//     Bank conflicts of the operand reads are avoided by an XOR swizzle instead: the 16-byte chunk at
//     LDS position c of a row holds the chunk c ^ f(row) of that row, which each lane realises by
//     choosing its global source address; the reads apply the same XOR.
//       row-index-contiguous operand: stage[k][256], f(k) = 2 * (k % 4); read with ds_read_b64_tr_b16
//           (a 16-lane group touches 4 k-rows x 32 bytes: 4 disjoint bank ranges)
//       k-contiguous operand:         stage[row][32], f(row) = (row / 4) % 4; read with ds_read_b128
//           (16 consecutive rows, one chunk each: 4 x 4 disjoint bank ranges)
//   * The texture path takes one 1 KiB load per 16 cycles and CU, and a wavefront whose load is not
//     accepted stalls with all its MFMAs behind it.  The four wavefronts run in lock step, so each
//     issues its loads in MFMA slots of its own (slot % 4 == wave): the path then sees one load per
//     MFMA instead of four at once.
//   * The compiler does not see these loads (inline assembly: it would otherwise wait for every
//     outstanding direct load before each LDS read), so the waits are placed by hand: loads complete
//     in issue order, and before the barrier that hands tile t + 1 to the readers each wavefront waits
//     until at most the 16 loads of tiles t + 2 and t + 3 are outstanding.
//
// Restrictions (the dispatcher checks them): both operands gathered in 16-byte vectors, K a
// multiple of 32 with one stride per operand (affine K).
#pragma once
#include "contract_h.hpp"

namespace hiptk
{
    // Direct load, in two halves so that another instruction (an MFMA) can sit between the write of
    // M0 and the load that reads it (one wait state is required there):
    //   dma_dst:  M0 <- LDS byte address lds_base + off (wave-uniform)
    //   dma_load: 16 bytes per lane from global memory (base + 32-bit byte offset voff) to LDS address
    //             M0 + 16 * lane.  Counted by vmcnt.
    // Nothing else in these kernels uses M0.
    // The compiler's hazard recognizer does not look inside inline assembly, so the wait states an
    // instruction needs are provided here: a VMEM instruction must not read an SGPR within 5 wait
    // states of a VALU instruction writing it (the compiler reloads spilled SGPRs with v_readlane,
    // possibly right in front of the asm statement), and M0 needs 1 wait state before the load that
    // reads it: s_nop 4 in front of the load covers both.
    template <int OFF>
    __device__ __forceinline__ void dma_dst(uint32_t lds_base)
    {
        asm volatile("s_add_u32 m0, %0, %1" : : "s"(lds_base), "n"(OFF) : "scc");
    }
    __device__ __forceinline__ void dma_load(uint32_t voff, const void* base)
    {
        asm volatile("s_nop 4\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base) : "memory");
    }

    // s_waitcnt immediates (gfx9 encoding): vmcnt(N) with the other counters left alone
    constexpr int waitcnt_vm(int n)
    {
        return (n & 15) | ((n >> 4) << 14) | 0x0F70;
    }

    template <typename Tr, bool XKF, bool YKF>
    struct HdGeom
    {
        static constexpr int BP = 256, BQ = 256, BK = 32, NS = 4;
        static constexpr int OPND  = 256 * BK; // elements of one operand in one stage
        static constexpr int STAGE = 2 * OPND;
        // (a little more than the ring: the bilinear epilogue double-buffers its staging in 132 KiB)
        static constexpr int LDS_BYTES = NS * STAGE * 2 + 8192 + 16384; // + 4 spare KiB per wave
    };

    // One operand's share of a wavefront's direct loads: 4 loads of 1 KiB per K tile.
    template <bool KF>
    struct HdLoader
    {
        uint32_t voff[4]; // byte offsets of this lane's 16 bytes, relative to the tile's k origin

        // rtab: row offset table; r0: first row of the tile; kstride: element stride of k
        __device__ inline void init(const int32_t* rtab, int r0, int kstride, int wave, int lane)
        {
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                const int j = wave * 4 + i; // which KiB of the operand stage
                if constexpr(KF)
                {
                    const int row = 16 * j + (lane >> 2);
                    const int c   = (lane & 3) ^ ((row >> 2) & 3);
                    voff[i]       = 2u * ((uint32_t)rtab[r0 + row] + (uint32_t)(8 * c) * (uint32_t)kstride);
                }
                else
                {
                    const int kk = 2 * j + (lane >> 5);
                    const int c  = (lane & 31) ^ (2 * (kk & 3));
                    voff[i]      = 2u * ((uint32_t)rtab[r0 + 8 * c] + (uint32_t)kk * (uint32_t)kstride);
                }
            }
        }
    };

    // MFMA operand fetch of the 32-row block i of a wave tile, k-substep ks (16 k), from a swizzled stage.
    template <bool KF>
    struct HdFrag
    {
        int base[KF ? 2 : 4]; // element offsets inside the operand stage

        __device__ inline void init(int wrow, int lane)
        {
            if constexpr(KF)
            {
                const int row = wrow + (lane & 31);
                const int sw  = (lane >> 2) & 3; // (row / 4) % 4: wrow and 32 * i are multiples of 16
#pragma unroll
                for(int ks = 0; ks < 2; ks++)
                    base[ks] = row * 32 + (((2 * ks + (lane >> 5)) ^ sw) << 3);
            }
            else
            {
                const int k  = 8 * (lane >> 5) + ((lane & 15) >> 2);
                const int sw = 2 * ((lane >> 2) & 3); // 2 * (k % 4); k + 4 and k + 16 swizzle alike
#pragma unroll
                for(int i = 0; i < 4; i++)
                {
                    const int r = wrow + i * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                    base[i]     = k * 256 + ((((r >> 3) ^ sw) << 3) | (r & 7));
                }
            }
        }

        __device__ inline u32x4_t load(const uint16_t* opnd, int i, int ks) const
        {
            if constexpr(KF)
                return *(const u32x4_t*)(opnd + base[ks] + i * 32 * 32);
            else
            {
                typedef short4_t __attribute__((address_space(3))) * lds_s4_ptr;
                const uint16_t* p  = opnd + base[i] + ks * 16 * 256;
                const short4_t  lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p));
                const short4_t  hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p + 4 * 256));
                const u32x2_t   l2 = __builtin_bit_cast(u32x2_t, lo);
                const u32x2_t   h2 = __builtin_bit_cast(u32x2_t, hi);
                return u32x4_t{l2[0], l2[1], h2[0], h2[1]};
            }
        }
    };

    template <typename Tr, bool XKF, bool YKF>
    __global__ void __launch_bounds__(256, 1) contract_hd_kernel(const KArgs a)
    {
        typedef HdGeom<Tr, XKF, YKF> G;
        constexpr int BP = G::BP, BQ = G::BQ, BK = G::BK, NS = G::NS;
        constexpr int TP = 4, TQ = 4, WP = 2, WQ = 2;

        extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

        const int tid  = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wp   = wave / WQ;
        const int wq   = wave % WQ;

        int tp, tq;
        tile_coords(blockIdx.x, a.tiles_p, a.tiles_q, tp, tq);
        const int p_own = tp * BP, q_own = tq * BQ;
        const int p0    = (a.shift_p && p_own + BP > a.P) ? a.P - BP : p_own;
        const int q0    = (a.shift_q && q_own + BQ > a.Q) ? a.Q - BQ : q_own;

        const int kt_begin = blockIdx.z * a.ktiles_per_split;
        int       kt_end   = kt_begin + a.ktiles_per_split;
        const int kt_all   = a.K / BK; // K is a multiple of BK
        if(kt_end > kt_all)
            kt_end = kt_all;
        const int nt = kt_end - kt_begin;

        HdLoader<XKF> gx;
        HdLoader<YKF> gy;
        gx.init(a.xp, p0, a.xk_stride, wave, lane);
        gy.init(a.yq, q0, a.yk_stride, wave, lane);
        HdFrag<XKF> fx;
        HdFrag<YKF> fy;
        fx.init(wp * 128, lane);
        fy.init(wq * 128, lane);

        // k origin of a tile, per operand (wave-uniform 64-bit addresses)
        const uint64_t xstep = 2ull * BK * (uint64_t)(uint32_t)a.xk_stride;
        const uint64_t ystep = 2ull * BK * (uint64_t)(uint32_t)a.yk_stride;
        const char*    xg    = (const char*)a.X + (uint64_t)kt_begin * xstep;
        const char*    yg    = (const char*)a.Y + (uint64_t)kt_begin * ystep;

        typedef uint16_t __attribute__((address_space(3))) * lds_u16_ptr;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_u16_ptr)lds; // LDS byte address of the ring
        // this wave's four KiB of an operand stage
        const uint32_t wdst = lds0 + (uint32_t)wave * 4096u;

        f32x16_t acc[TP][TQ];
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int j = 0; j < TQ; j++)
#pragma unroll
                for(int r = 0; r < 16; r++)
                    acc[i][j][r] = 0.f;

        u32x4_t xf[2][TP], yf[2][TQ];

        // Loads of tiles beyond the K range are not skipped (the loop stays free of branches and
        // every wait sees the same number of younger loads): they re-read the last tile and land in
        // four spare KiB per wave behind the ring.
        const uint32_t wspare = lds0 + NS * G::STAGE * 2 + 8192 + (uint32_t)wave * 4096u;
        // source of the next X / Y tile to be requested, its index, and where it goes
        const char* xsrc = xg;
        const char* ysrc = yg;
        int         xu = 0, yu = 0;
        uint32_t    xdst = wdst, ydst = wdst + G::OPND * 2;
        // after the loads of a tile have been issued: move on to the next tile; S = its ring stage
        auto x_next = [&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            xu++;
            const bool more = xu < nt;
            xsrc            = more ? xsrc + xstep : xsrc;
            xdst            = more ? wdst + S * (G::STAGE * 2) : wspare;
        };
        auto y_next = [&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            yu++;
            const bool more = yu < nt;
            ysrc            = more ? ysrc + ystep : ysrc;
            ydst            = more ? wdst + S * (G::STAGE * 2) + G::OPND * 2 : wspare;
        };

        // One k-substep: 16 MFMAs out of register set `slot`; the 8 operand fetches `(nstage, nks)`
        // into the other set spread over its first 8 MFMAs in the order the next substep needs them
        // (x0 y0 y1 y2 y3 x1 x2 x3); and 4 direct loads (X or Y) in the MFMA slots of this wave, each
        // with its M0 write one MFMA earlier.  sched_barrier(0) after every MFMA keeps the issue order
        // as written.
        auto substep = [&](auto wv_c, auto slot_c, const uint16_t* nstage, auto nks_c, auto isx_c) {
            constexpr int  WV   = decltype(wv_c)::value;
            constexpr int  slot = decltype(slot_c)::value;
            constexpr int  nks  = decltype(nks_c)::value;
            constexpr bool ISX  = decltype(isx_c)::value;
#pragma unroll
            for(int m = 0; m < 16; m++)
            {
                // fetch f (0..7: x0 y0 y1 y2 y3 x1 x2 x3) goes before MFMA f
#pragma unroll
                for(int f = 0; f < 8; f++)
                    if(f == m)
                    {
                        if(f == 0)
                            xf[slot ^ 1][0] = fx.load(nstage, 0, nks);
                        else if(f <= 4)
                            yf[slot ^ 1][f - 1] = fy.load(nstage + G::OPND, f - 1, nks);
                        else
                            xf[slot ^ 1][f - 4] = fx.load(nstage, f - 4, nks);
                    }
                // load i = m / 4 of this substep goes after MFMA slot 4 * i + WV - 1 .. its M0 one slot earlier
                constexpr int LS = WV; // slot of the load within each group of four MFMAs
                if((m & 3) == ((LS + 3) & 3) && (LS != 0 || m != 15) )
                {
                    // M0 for the load that follows the next MFMA
                    const int i = LS == 0 ? (m + 1) >> 2 : m >> 2;
                    if(i == 0) dma_dst<0>(ISX ? xdst : ydst);
                    if(i == 1) dma_dst<1024>(ISX ? xdst : ydst);
                    if(i == 2) dma_dst<2048>(ISX ? xdst : ydst);
                    if(i == 3) dma_dst<3072>(ISX ? xdst : ydst);
                }
                if(LS == 0 && m == 0)
                {
                    // (first slot of the substep: no earlier MFMA in it)
                    dma_dst<0>(ISX ? xdst : ydst);
                }
                if((m & 3) == LS)
                    dma_load(ISX ? gx.voff[m >> 2] : gy.voff[m >> 2], ISX ? xsrc : ysrc);
                acc[m >> 2][m & 3] = Tr::mfma(xf[slot][m >> 2], yf[slot][m & 3], acc[m >> 2][m & 3]);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;

        // K tile t, whose ring stage is S = t % 4
        auto tile_step = [&](auto wv_c, auto s_c) {
            constexpr int   S   = decltype(s_c)::value;
            const uint16_t* cur = lds + S * G::STAGE;
            const uint16_t* nxt = lds + ((S + 1) & (NS - 1)) * G::STAGE;
            // substep 0: multiply k 0..15 of tile t, fetch k 16..31; the Y loads of tile t + 3
            substep(wv_c, I0{}, cur, I1{}, std::false_type{});
            y_next(std::integral_constant<int, S>{}); // tile t + 4 shares tile t's stage
            // Every wave has issued its reads of tile t.  Tile t + 1 must have landed: the 16
            // younger loads are those of tiles t + 2 and t + 3.
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(16));
            lds_barrier();
            __builtin_amdgcn_sched_barrier(0);
            // substep 1: multiply k 16..31 of tile t, fetch k 0..15 of tile t + 1 (beyond the last
            // tile: stale data, not used); the X loads of tile t + 4 go into the stage tile t has
            // just left
            substep(wv_c, I1{}, nxt, I0{}, std::true_type{});
            x_next(std::integral_constant<int, (S + 1) & (NS - 1)>{}); // tile t + 5
        };

        auto main_loop = [&](auto wv_c) {
            // prologue: tiles 0, 1, 2 and the X half of tile 3
#pragma unroll
            for(int t = 0; t < NS; t++)
            {
#pragma unroll
                for(int i = 0; i < 4; i++)
                {
                    asm volatile("s_add_u32 m0, %0, %1" : : "s"(xdst), "s"(i * 1024) : "scc");
                    dma_load(gx.voff[i], xsrc);
                }
                if(t == 0) x_next(I1{});
                if(t == 1) x_next(std::integral_constant<int, 2>{});
                if(t == 2) x_next(std::integral_constant<int, 3>{});
                if(t == 3) x_next(I0{});
                if(t < NS - 1)
                {
#pragma unroll
                    for(int i = 0; i < 4; i++)
                    {
                        asm volatile("s_add_u32 m0, %0, %1" : : "s"(ydst), "s"(i * 1024) : "scc");
                        dma_load(gy.voff[i], ysrc);
                    }
                    if(t == 0) y_next(I1{});
                    if(t == 1) y_next(std::integral_constant<int, 2>{});
                    if(t == 2) y_next(std::integral_constant<int, 3>{});
                }
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(16)); // tile 0 has landed (and 4 loads of tile 1)
            lds_barrier();
#pragma unroll
            for(int i = 0; i < TP; i++)
                xf[0][i] = fx.load(lds, i, 0);
#pragma unroll
            for(int j = 0; j < TQ; j++)
                yf[0][j] = fy.load(lds + G::OPND, j, 0);
            __builtin_amdgcn_sched_barrier(0);

            int t = 0;
            for(; t + 4 <= nt; t += 4)
            {
                tile_step(wv_c, I0{});
                tile_step(wv_c, I1{});
                tile_step(wv_c, std::integral_constant<int, 2>{});
                tile_step(wv_c, std::integral_constant<int, 3>{});
            }
            if(t < nt)
                tile_step(wv_c, I0{});
            if(t + 1 < nt)
                tile_step(wv_c, I1{});
            if(t + 2 < nt)
                tile_step(wv_c, std::integral_constant<int, 2>{});
        };

        // One copy of loop and epilogue per wave position: the loop bodies differ in where the direct
        // loads sit, and joining them before the epilogue made the compiler spill accumulators.
        auto run = [&](auto wv_c) {
            if(nt > 0)
                main_loop(wv_c);
            // the epilogue stages through LDS: every wave must be done reading operands
            lds_barrier();
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int j = 0; j < TQ; j++)
                    asm volatile("" : "+a"(acc[i][j]));
            epilogue_h<Tr, WP, WQ, TP, TQ, NS * G::STAGE * 2 + 8192, true>(a, acc, lds, p0, q0, p_own, q_own);
        };
        switch(wave)
        {
        case 0: run(std::integral_constant<int, 0>{}); break;
        case 1: run(std::integral_constant<int, 1>{}); break;
        case 2: run(std::integral_constant<int, 2>{}); break;
        default: run(std::integral_constant<int, 3>{}); break;
        }
        // the loads beyond the K range (into the spare KiB) must not outlive the workgroup's LDS
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    }

    template <typename Tr, bool XKF, bool YKF>
    int launch_hd(const KArgs& a, hipStream_t stream)
    {
        typedef HdGeom<Tr, XKF, YKF> G;
        auto                         kern = contract_hd_kernel<Tr, XKF, YKF>;
        static const hipError_t      attr = hipFuncSetAttribute(
            (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if(attr != hipSuccess)
            return (int)attr;
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(kern, grid, dim3(256), G::LDS_BYTES, stream, a);
        return (int)hipGetLastError();
    }
}

// Registry line of the direct-load kernel: affine K only, K a multiple of 32.
#define HIPTK_HD_ENTRY(TR, ID, XKF, YKF)                                                          \
    {                                                                                             \
        TR::CLS, ID, XKF, YKF, 8, 8, true, 256, 256, 32, 256, hiptk::HdGeom<hiptk::TR, XKF, YKF>::LDS_BYTES, \
            #TR "_256x256x32_x" #XKF "8_y" #YKF "8_kafftrue_direct2x2", &hiptk::launch_hd<hiptk::TR, XKF, YKF>, 32 \
    }
#define HIPTK_HD_TILE(TR, ID)                                                                     \
    HIPTK_HD_ENTRY(TR, ID, true, true), HIPTK_HD_ENTRY(TR, ID, true, false),                      \
        HIPTK_HD_ENTRY(TR, ID, false, true), HIPTK_HD_ENTRY(TR, ID, false, false)
