// 32/64-bit (f32, f64, complex f32, complex f64) contraction kernel for gfx950 whose operand tiles go from global
// memory straight into LDS (global_load_lds_dwordx4), for operands that are each contiguous along
// their row index (both: packed column-major, every benchmark configuration of these types; described
// below) or along k (both: packed row-major, what NULL strides mean; the differences are at wd_slot_kf
// in hd_addr.hpp and at read_op).  (Complex f64, one element per 16-byte
// vector, runs the k-contiguous form on any layout with one K stride.)
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
//     needs (1024 x 1024 x 512 complex f32 in one pass: 50.7 us through registers, 38.7 us here).  The
//     order of MFMAs, requests and reads inside a K tile is fixed by hand (see `step`).
//   * The loads are inline assembly (dma_lds.hpp), invisible to the compiler, so the waits are placed
//     by hand: loads complete in issue order, and before the barrier that hands tile t + 1 to the
//     readers each wave waits until only the loads of the NS - 2 tiles after it are outstanding.
//     Tiles requested beyond the K range are not branched around: they re-read the last tile into
//     spare LDS behind the ring, so every wait sees the same number of younger loads.
//   * Nothing but MFMAs, loads, LDS reads and scalar instructions in a step: a vector instruction between
//     the MFMAs waits for the matrix pipe, and a branch cuts the step into blocks.  So the LDS address of
//     every read is a register that was set before the loop plus an offset that fits the instruction
//     (`xat`, `yat`), and each kernel is instantiated twice: for K a multiple of BK, and with the test for
//     a short last K tile in its steps (launch_wd picks).  With the address additions in the loop
//     1920 x 1920 x 768 f64 took 107.7 us, without them 100.5, without the test 98.0.
//
// Restrictions (the dispatcher checks them): both operands gathered in 16-byte vectors, along their
// row index or along k, on 16-byte boundaries; one K stride per operand; K at least BK (a last tile
// shorter than BK loads the vectors beyond K from zeros), and a multiple of the vector where an operand
// is contiguous along k; byte offsets inside each operand below 2^32.
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

    // WK = false: 64 x 64 tile, the four waves (2 x 2) share one ring.  WK = true: 32 x 32 tile, every wave
    // multiplies all of it over its own quarter of the K range out of a ring of its own (no barrier in the
    // loop), and the four partial tiles are added through LDS at the end: for outputs too small to fill the
    // device with 64 x 64 tiles, in one launch.
    template <typename Tr, int BK, int NS, bool WK, bool XKF = false, bool YKF = false>
    struct WdGeom
    {
        static constexpr int ROWS = WK ? 32 : 64; // rows of an operand tile
        static constexpr int BP = ROWS, BQ = ROWS;
        static constexpr int ES       = (int)sizeof(typename Tr::S);
        static constexpr int V        = 16 / ES; // elements per 16-byte vector
        static constexpr int OP_BYTES = BK * ROWS * ES; // one operand in one stage
        static constexpr int NLW      = WK ? OP_BYTES / 1024 : OP_BYTES / 4096; // direct loads (1 KiB) per wave, operand and K tile
        static constexpr int STAGE_BYTES = 2 * OP_BYTES;
        static constexpr int RING        = NS * STAGE_BYTES;
        static constexpr int RINGS       = WK ? 4 : 1;
        static constexpr int SPARE       = RINGS * RING; // NLW KiB per wave: where loads beyond the K range land
        static constexpr int LDS_BYTES   = SPARE + 4 * NLW * 1024;
        static_assert(OP_BYTES % (WK ? 1024 : 4096) == 0 && NLW >= 1, "every wave loads whole KiB of an operand stage");
        static_assert(std::is_same<typename Tr::S, typename Tr::E>::value, "a direct load cannot convert");
        static_assert(NS >= 4 && NS % 2 == 0 && (NS - 1) * 2 * NLW < 64, "the wait counts must fit vmcnt");
        static_assert(!WK || RING >= (32 / Tr::TILE) * (32 / Tr::TILE) * Tr::NREG * 64 * (int)sizeof(typename Tr::O),
                      "a wave's partial tile is handed over in its own ring");
        static_assert(LDS_BYTES <= 160 * 1024, "LDS of one CU");
        static_assert(!(XKF || YKF) || (BK / Tr::KM) % V == 0, "a k-contiguous vector feeds whole k-steps");
    };

    // what the vectors of a short last K tile that lie beyond K are loaded from
    static __device__ __attribute__((aligned(16))) const unsigned char wd_zero16[16] = {0};

    // sizeof(T) = 4, 8 or 16 bytes of LDS at byte address `at` (a multiple of that size)
    template <typename T>
    __device__ __forceinline__ T lds_read(uint32_t at)
    {
        typedef uint32_t __attribute__((ext_vector_type(sizeof(T) / 4))) R;
        typedef __attribute__((address_space(3))) R                      RL;
        const R r = *(const RL*)(uintptr_t)at;
        T       t;
        __builtin_memcpy(&t, &r, sizeof(T));
        return t;
    }

    __device__ __forceinline__ float   wd_add(float x, float y) { return __fadd_rn(x, y); }
    __device__ __forceinline__ double  wd_add(double x, double y) { return __dadd_rn(x, y); }
    __device__ __forceinline__ float2  wd_add(float2 x, float2 y) { return make_float2(__fadd_rn(x.x, y.x), __fadd_rn(x.y, y.y)); }
    __device__ __forceinline__ double2 wd_add(double2 x, double2 y) { return make_double2(__dadd_rn(x.x, y.x), __dadd_rn(x.y, y.y)); }

    // The epilogue of these kernels in two halves: `fetch`, before the main loop, looks up the wave tile's
    // C / D offsets and requests its C elements; `store`, after it, writes D = alpha * acc (+ beta * C).
    // contract_w.hpp's epilogue_w fetches four accumulator rows at a time behind the stores of the four
    // before (D may alias C), one memory latency per batch, which other workgroups on the CU cover there;
    // here a workgroup may be alone, and the registers for all of a lane's C elements are free.
    // (Reading C early is safe when D aliases it: every element is read and written by the same lane,
    // these kernels never move a tile back over a neighbour's rows.)
    template <typename Tr, int TP, int TQ>
    struct WdEpilogue
    {
        typedef typename Tr::E E;
        uint32_t               dpo[TP][Tr::NREG], dqo[TQ];
        uint32_t               pmask, qmask;
        E                      cv[TP][Tr::NREG][TQ];

        __device__ __forceinline__ void fetch(const KArgs& a, int pw, int qw, int p_own, int q_own, int lane)
        {
            constexpr int TILE = Tr::TILE;
            static_assert(TP * Tr::NREG <= 32 && TQ <= 32, "one bit per row and column");
            const E*   Cp  = (const E*)a.C;
            const bool bil = a.bilinear != 0;
            const bool aff = a.cd_affine != 0;
            // A lane outside the extents fetches element (0, 0) instead, a valid address, and stores nothing.
            uint32_t cqo[TQ], cpo[TP][Tr::NREG];
            pmask = 0;
            qmask = 0;
#pragma unroll
            for(int j = 0; j < TQ; j++)
            {
                const int  q  = qw + j * TILE;
                const bool ok = q >= q_own && q < a.Q;
                qmask |= ok ? 1u << j : 0u;
                const int qv = ok ? q : 0;
                dqo[j]       = aff ? (uint32_t)qv * (uint32_t)a.dq_stride : (uint32_t)a.dq[qv];
                cqo[j]       = !bil ? 0u : aff ? (uint32_t)qv * (uint32_t)a.cq_stride : (uint32_t)a.cq[qv];
            }
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int r = 0; r < Tr::NREG; r++)
                {
                    const int  p  = pw + i * TILE + Tr::p_of(r, lane);
                    const bool ok = p >= p_own && p < a.P;
                    pmask |= ok ? 1u << (i * Tr::NREG + r) : 0u;
                    const int pv = ok ? p : 0;
                    dpo[i][r]    = aff ? (uint32_t)pv * (uint32_t)a.dp_stride : (uint32_t)a.dp[pv];
                    cpo[i][r]    = !bil ? 0u : aff ? (uint32_t)pv * (uint32_t)a.cp_stride : (uint32_t)a.cp[pv];
                }
            if(bil)
            {
#pragma unroll
                for(int i = 0; i < TP; i++)
#pragma unroll
                    for(int r = 0; r < Tr::NREG; r++)
#pragma unroll
                        for(int j = 0; j < TQ; j++)
                            cv[i][r][j] = Cp[cpo[i][r] + cqo[j]];
            }
        }

        __device__ __forceinline__ void store(const KArgs& a, typename Tr::Acc (&acc)[TP][TQ])
        {
            E*         Dp  = (E*)a.D;
            const bool bil = a.bilinear != 0;
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int r = 0; r < Tr::NREG; r++)
#pragma unroll
                    for(int j = 0; j < TQ; j++)
                    {
                        if(((pmask >> (i * Tr::NREG + r)) & 1u) && ((qmask >> j) & 1u))
                        {
                            const E val = Tr::finish(Tr::get(acc[i][j], r), a.alpha, a.beta, bil, &cv[i][r][j]);
                            if constexpr(std::is_arithmetic<E>::value)
                                __builtin_nontemporal_store(val, Dp + (dpo[i][r] + dqo[j]));
                            else
                                Dp[dpo[i][r] + dqo[j]] = val;
                        }
                    }
        }
    };

    // Tile t + 1 has landed when only the loads of the N / LPT tiles after it are outstanding.  With a common
    // ring the barrier behind the wait shows it to every wave, and says that every wave has tile t in
    // registers; a wave with a ring of its own waits for its own LDS reads of tile t instead, before it lets
    // tile t + NS be written over them.
    template <bool WK, int N>
    __device__ __forceinline__ void wd_hand_over()
    {
        if(WK)
        {
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(N) & ~0x0F00); // ... and lgkmcnt(0)
            asm volatile("" : : : "memory");
        }
        else
        {
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(N));
            w_lds_barrier();
        }
    }

    // TAIL: K need not be a multiple of BK.  (The test for the short last tile is a branch in every step of the
    // main loop, which costs 2-5 %: problems without such a tile run the instantiation without it.)
    template <typename Tr, int BK, int NS, bool WK, bool XKF, bool YKF, bool TAIL>
    __global__ void __launch_bounds__(256, 2) contract_wd_kernel(const KArgs a)
    {
        typedef WdGeom<Tr, BK, NS, WK, XKF, YKF> G;
        // with a k-contiguous operand the k-slots of one k-step are V apart in k (see wd_slot_kf), for both operands
        constexpr bool VAPART = XKF || YKF;
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
        const int wp   = WK ? 0 : wave >> 1;
        const int wq   = WK ? 0 : wave & 1;
        constexpr int ROWS = G::ROWS;

        int tp, tq;
        tile_coords(blockIdx.x, a.tiles_p, a.tiles_q, tp, tq);
        // (no tile is moved back; a tile that overhangs P or Q reads the padding of the row tables, offset 0,
        // and stores nothing there)
        const int p0 = tp * G::BP, q0 = tq * G::BQ;

        int       kt_begin = blockIdx.z * a.ktiles_per_split;
        int       kt_end   = kt_begin + a.ktiles_per_split;
        const int kt_all   = (a.K + BK - 1) / BK; // the last tile may hold fewer than BK k
        if(kt_end > kt_all)
            kt_end = kt_all;
        if(WK)
        {
            // this wave's quarter of the slice (the last waves of a short slice have none)
            const WdChunk c = wd_wave_chunk(kt_end - kt_begin, wave);
            kt_begin += c.first;
            kt_end = kt_begin + c.count;
        }
        const int nt = kt_end - kt_begin;

        // this lane's 16 bytes of each of its loads, as byte offsets from the tile's k origin; and, bit i,
        // whether load i of a short last tile lies inside K
        const int tail_k      = TAIL ? a.K % BK : 0;
        const int tail_origin = tail_k ? (kt_all - 1) * BK : -1;
        uint32_t  xin = 0, yin = 0;
        uint32_t  xv[NLW], yv[NLW];
#pragma unroll
        for(int i = 0; i < NLW; i++)
        {
            const int    s_ = ((WK ? 0 : wave * NLW) + i) * 64 + lane;
            const HdSlot sx = XKF ? wd_slot_kf<G::V, ROWS>(s_) : wd_slot<G::V, ROWS>(s_);
            const HdSlot sy = YKF ? wd_slot_kf<G::V, ROWS>(s_) : wd_slot<G::V, ROWS>(s_);
            xv[i]           = (uint32_t)ES * ((uint32_t)a.xp[p0 + sx.row] + (uint32_t)sx.k * (uint32_t)a.xk_stride);
            yv[i]           = (uint32_t)ES * ((uint32_t)a.yq[q0 + sy.row] + (uint32_t)sy.k * (uint32_t)a.yk_stride);
            xin |= wd_tail_inside(XKF, sx.k, G::V, tail_k) ? 1u << i : 0u;
            yin |= wd_tail_inside(YKF, sy.k, G::V, tail_k) ? 1u << i : 0u;
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
        // this wave's share of an X stage of the common ring, or its own ring
        const uint32_t wdx    = lds0 + (uint32_t)wave * (WK ? (uint32_t)G::RING : NLW * 1024u);
        const unsigned char* const ring = lds_raw + (WK ? wave * G::RING : 0);
        const uint32_t wdy    = wdx + G::OP_BYTES;
        const uint32_t wspare = lds0 + G::SPARE + (uint32_t)wave * (NLW * 1024u);

        // request tile `lu` into ring stage ST
        auto issue = [&](auto st_c) {
            constexpr int  ST   = decltype(st_c)::value;
            const bool     real = lu < nt;
            const uint32_t dx   = real ? wdx + ST * G::STAGE_BYTES : wspare;
            const uint32_t dy   = real ? wdy + ST * G::STAGE_BYTES : wspare;
            if(TAIL && ko == tail_origin)
            {
                // the short last tile (or a repeat of it): the same number of loads, each lane from where its
                // vector lies if that is inside K, else from zeros: the tile then multiplies as a whole one
#pragma unroll
                for(int i = 0; i < NLW; i++)
                {
                    dma_dst_at(dx, i * 1024);
                    dma_load_at((xin >> i) & 1u ? (const void*)(xsrc + xv[i]) : (const void*)wd_zero16);
                }
#pragma unroll
                for(int i = 0; i < NLW; i++)
                {
                    dma_dst_at(dy, i * 1024);
                    dma_load_at((yin >> i) & 1u ? (const void*)(ysrc + yv[i]) : (const void*)wd_zero16);
                }
            }
            else
            {
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
            }
            lu++;
            ko   = wd_next_origin(ko, klast, BK);
            xsrc = (const char*)a.X + (uint64_t)((uint32_t)ko * xkb);
            ysrc = (const char*)a.Y + (uint64_t)((uint32_t)ko * ykb);
        };

        // C and the C / D offsets of the wave tile this wave will store (with waves that split K: wave 0,
        // all of the tile), unless the launch is a split-K slice, which stores partial sums
        // (complex f64 has no registers for it: 64 for its C elements beside 96 of accumulators and 64 of operands)
        constexpr bool EARLY_C = TP * TQ * Tr::NREG * sizeof(typename Tr::E) <= 128;
        WdEpilogue<Tr, TP, TQ> epi;
        const bool             whole_k = EARLY_C && a.split_k == 1;
        const bool             storer  = !WK || wave == 0;
        if(whole_k && storer)
            epi.fetch(a, p0 + wp * 32, q0 + wq * 32 + Tr::q_of(lane), p0, q0, lane);
        // (requested before the first operand tile: loads return in order, so they are back before it)
        __builtin_amdgcn_sched_barrier(0);

        typename Tr::Acc acc[TP][TQ];
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int j = 0; j < TQ; j++)
                Tr::zero(acc[i][j]);

        const int row   = lane & (TILE - 1);
        const int kslot = Tr::kslot(lane);
        // (a k-contiguous operand's stage is indexed in 16-byte vectors, [k / V][ROWS]; a row-contiguous one's in
        // elements, [k][ROWS], where the k-slots of a k-step are 1 or V rows of the stage apart)
        const int xfo = kslot * (!XKF && VAPART ? G::V : 1) * ROWS + wp * 32 + row;
        const int yfo = kslot * (!YKF && VAPART ? G::V : 1) * ROWS + wq * 32 + row;

        // This wave's operands of one K tile, in registers: tile t + 1 is read from LDS while tile t
        // is multiplied, so that a wave alone on its SIMD does not wait for LDS either.
        struct Frags
        {
            S x[KS][TP], y[KS][TP];
        };
        Frags fr[2];
        // the operands of k-step ks of the tile in ring stage ST (k-contiguous operands: of the V k-steps from
        // ks on, when ks is the first of them: one 16-byte read per operand row block)
        struct alignas(16) SVec
        {
            S e[G::V];
        };
        // one operand's part of it: KF: a vector of V k-steps' elements when ks is the first of them; else one
        // element, at k-slot distance 1 or (next to a k-contiguous operand) V
        // (`at`: the LDS byte address of this lane's first element of the operand's stage, and the addresses every
        // PIN_BYTES behind it: what the offset field of a paired 8-byte read spans)
        constexpr int PIN_BYTES = 2048;
        constexpr int PINS      = G::OP_BYTES > PIN_BYTES ? G::OP_BYTES / PIN_BYTES : 1;
        auto read_op = [&](auto kf_c, const uint32_t (&at)[PINS], S (&dst)[KS][TP], int ks) {
            static_assert(TP == TQ, "one reader for both operands");
            if constexpr(decltype(kf_c)::value)
            {
                if(ks % G::V != 0)
                    return;
#pragma unroll
                for(int i = 0; i < TP; i++)
                {
                    const int  off = ((ks / G::V) * Tr::KM * ROWS + i * TILE) * (int)sizeof(SVec);
                    const SVec v   = lds_read<SVec>(at[off / PIN_BYTES] + (uint32_t)(off % PIN_BYTES));
#pragma unroll
                    for(int j = 0; j < G::V; j++)
                        dst[ks + j][i] = v.e[j];
                }
            }
            else
            {
                const int k0 = VAPART ? ((ks / G::V) * Tr::KM * G::V + ks % G::V) : ks * Tr::KM;
#pragma unroll
                for(int i = 0; i < TP; i++)
                {
                    const int off = (k0 * ROWS + i * TILE) * (int)sizeof(S);
                    dst[ks][i]    = lds_read<S>(at[off / PIN_BYTES] + (uint32_t)(off % PIN_BYTES));
                }
            }
        };
        // Those addresses, per ring stage, in registers of their own that the compiler cannot tell apart from
        // any other value: it would otherwise add the stage's offset before every read, and a vector
        // instruction between the MFMAs waits for the matrix pipe.  Every read is then one of them plus an offset
        // that fits the instruction.
        uint32_t xat[NS][PINS], yat[NS][PINS];
#pragma unroll
        for(int st = 0; st < NS; st++)
#pragma unroll
            for(int pin = 0; pin < PINS; pin++)
            {
                const uint32_t stage = (uint32_t)(uintptr_t)(lds_u8_ptr)ring + st * G::STAGE_BYTES + pin * PIN_BYTES;
                xat[st][pin]         = stage + (uint32_t)xfo * (uint32_t)(XKF ? sizeof(SVec) : sizeof(S));
                yat[st][pin]         = stage + G::OP_BYTES + (uint32_t)yfo * (uint32_t)(YKF ? sizeof(SVec) : sizeof(S));
                asm volatile("" : "+v"(xat[st][pin]), "+v"(yat[st][pin]));
            }
        auto read_k = [&](auto st_c, Frags& f, int ks) {
            constexpr int ST = decltype(st_c)::value;
            read_op(std::integral_constant<bool, XKF>{}, xat[ST], f.x, ks);
            read_op(std::integral_constant<bool, YKF>{}, yat[ST], f.y, ks);
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
            wd_hand_over<WK, (NS - 2) * LPT>();
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
            wd_hand_over<WK, (NS - 1) * LPT>();
            read_tile(std::integral_constant<int, 0>{}, fr[0]);
            while(t + NS <= nt)
                wd_static_for<NS>(step);
            wd_static_for<NS - 1>([&](auto i_c) {
                if(t < nt)
                    step(i_c);
            });
        }
        if constexpr(WK)
        {
            // The four partial tiles are added in wave order (the order of split-K slices) by wave 0, which
            // then stores the tile: a wave's ring is its own again once its last loads have landed.
            typedef typename Tr::O O;
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0) & ~0x0F00);
            asm volatile("" : : : "memory");
            if(wave != 0)
            {
                O* mine = (O*)(lds_raw + wave * G::RING);
#pragma unroll
                for(int i = 0; i < TP; i++)
#pragma unroll
                    for(int j = 0; j < TQ; j++)
#pragma unroll
                        for(int r = 0; r < Tr::NREG; r++)
                            mine[((i * TQ + j) * Tr::NREG + r) * 64 + lane] = Tr::get(acc[i][j], r);
            }
            w_lds_barrier();
            if(wave != 0)
                return;
#pragma unroll
            for(int i = 0; i < TP; i++)
#pragma unroll
                for(int j = 0; j < TQ; j++)
#pragma unroll
                    for(int r = 0; r < Tr::NREG; r++)
                    {
                        O sum = Tr::get(acc[i][j], r);
#pragma unroll
                        for(int w = 1; w < 4; w++)
                            sum = wd_add(sum, ((const O*)(lds_raw + w * G::RING))[((i * TQ + j) * Tr::NREG + r) * 64 + lane]);
                        Tr::put(acc[i][j], r, sum);
                    }
            if(whole_k)
                epi.store(a, acc);
            else
                epilogue_w<Tr, TP, TQ>(a, acc, p0, q0 + Tr::q_of(lane), p0, q0, lane);
        }
        else
        {
            if(whole_k)
                epi.store(a, acc);
            else
                epilogue_w<Tr, TP, TQ>(a, acc, p0 + wp * 32, q0 + wq * 32 + Tr::q_of(lane), p0, q0, lane);
            // the loads beyond the K range (into the spare KiB) must not outlive the workgroup's LDS
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        }
    }

    template <typename Tr, int BK, int NS, bool WK, bool XKF, bool YKF>
    int launch_wd(const KArgs& a, hipStream_t stream)
    {
        typedef WdGeom<Tr, BK, NS, WK, XKF, YKF> G;
        // (a tile is never moved back here.  Row-contiguous operands that would need it are not offered this
        // kernel; with k-contiguous ones the flag can only come from C / D's vectors, which the element-wise
        // epilogue does not use: an overhanging tile reads the row tables' padding and stores nothing there)
        if(a.K < BK || ((XKF || YKF) && a.K % G::V != 0) || (!XKF && a.shift_p) || (!YKF && a.shift_q))
            return (int)hipErrorInvalidValue;
        auto whole = contract_wd_kernel<Tr, BK, NS, WK, XKF, YKF, false>;
        auto tail  = contract_wd_kernel<Tr, BK, NS, WK, XKF, YKF, true>;
        static const hipError_t attr_whole = hipFuncSetAttribute(
            (const void*)whole, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        static const hipError_t attr_tail = hipFuncSetAttribute(
            (const void*)tail, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if(attr_whole != hipSuccess || attr_tail != hipSuccess)
            return (int)(attr_whole != hipSuccess ? attr_whole : attr_tail);
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(a.K % BK == 0 ? whole : tail, grid, dim3(256), G::LDS_BYTES, stream, a);
        return (int)hipGetLastError();
    }
}

// Registry line of a direct-load tile: both operands in row-index vectors, one K stride, any K from BK on.
// (A class whose element fills the 16 bytes would have no vectors: every problem of it is described
// as "scalar, k-fast", and any row table would do.)
#define HIPTK_WD_ENTRY(TR, ID, BK, NS)                                                              \
    {                                                                                               \
        hiptk::TR::CLS, ID, hiptk::TR::VMAX == 1, hiptk::TR::VMAX == 1, hiptk::TR::VMAX,            \
            hiptk::TR::VMAX, 1, 64, 64, BK, 256,                                                    \
            hiptk::WdGeom<hiptk::TR, BK, NS, false>::LDS_BYTES, #TR "_64x64x" #BK "_direct" #NS,\
            &hiptk::launch_wd<hiptk::TR, BK, NS, false, false, false>, 1                                         \
    }

// ... and of the 32 x 32 tile whose four waves split the K range between them.
#define HIPTK_WK_ENTRY(TR, ID, BK, NS)                                                              \
    {                                                                                               \
        hiptk::TR::CLS, ID, hiptk::TR::VMAX == 1, hiptk::TR::VMAX == 1, hiptk::TR::VMAX,            \
            hiptk::TR::VMAX, 1, 32, 32, BK, 256,                                                    \
            hiptk::WdGeom<hiptk::TR, BK, NS, true>::LDS_BYTES, #TR "_32x32x" #BK "_direct" #NS "k4", \
            &hiptk::launch_wd<hiptk::TR, BK, NS, true, false, false>, 1                                        \
    }

// ... and of both where X (XKF) and / or Y (YKF) are contiguous along k instead (16-byte vectors of k, one K stride).
#define HIPTK_WD_ENTRY_KF(TR, ID, BK, NS, XKF, YKF)                                                 \
    {                                                                                               \
        hiptk::TR::CLS, ID, XKF, YKF, hiptk::TR::VMAX, hiptk::TR::VMAX, 1, 64, 64, BK, 256,         \
            hiptk::WdGeom<hiptk::TR, BK, NS, false, XKF != 0, YKF != 0>::LDS_BYTES,                 \
            #TR "_64x64x" #BK "_direct" #NS "kf" #XKF #YKF,                                         \
            &hiptk::launch_wd<hiptk::TR, BK, NS, false, XKF != 0, YKF != 0>, hiptk::TR::VMAX                     \
    }
#define HIPTK_WK_ENTRY_KF(TR, ID, BK, NS, XKF, YKF)                                                 \
    {                                                                                               \
        hiptk::TR::CLS, ID, XKF, YKF, hiptk::TR::VMAX, hiptk::TR::VMAX, 1, 32, 32, BK, 256,         \
            hiptk::WdGeom<hiptk::TR, BK, NS, true, XKF != 0, YKF != 0>::LDS_BYTES,                  \
            #TR "_32x32x" #BK "_direct" #NS "k4kf" #XKF #YKF,                                       \
            &hiptk::launch_wd<hiptk::TR, BK, NS, true, XKF != 0, YKF != 0>, hiptk::TR::VMAX                     \
    }
