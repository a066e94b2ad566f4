// 16-bit (f16 / bf16) contraction kernel for gfx950 built on v_mfma_f32_16x16x32 whose operand tiles
// go from global memory straight into LDS (global_load_lds_dwordx4) in K tiles of 64.
//
// Same problem statement and epilogue as contract_h.hpp and the same ideas as contract_hd.hpp (direct
// loads as inline assembly with hand-placed waits, one copy of the loop per wave position, XOR swizzle
// instead of padding).  What differs, and why:
//
//   * v_mfma_f32_16x16x32 instead of 32x32x16.  This part's clock under a matrix load is set by
//     power, and a loop of 32x32x16 MFMAs pays for every LDS read and every direct load beside them
//     with clock (one ds_read_b128 per MFMA: - 8 %; one direct load per two: - 8 %), while beside
//     16x16x32 MFMAs the same reads and loads are free.  Measured on 4096^3 with both operands
//     k-contiguous: main loop 93.7 -> 84.2 us with nothing else changed.
//   * A single wave per SIMD gets one issue slot every four cycles, and a 16x16x32 MFMA runs for 16:
//     three slots beside each MFMA.  s_nop N holds N + 1 of them, so the loop contains none (the
//     loads inside it are issued without the wait states dma_load puts in front of a load: see
//     dma_load_in_loop), and the MFMAs are inline assembly that accumulates in place (left to itself
//     the register allocator, which for 16x16 results need not reuse the addend's registers, moved
//     accumulators around all through the loop: three moves per MFMA).
//   * K in steps of 64.  A direct load writes 64 lanes x 16 bytes to consecutive LDS addresses, so
//     the rows of a stage are as long as the runs a load fetches: with K tiles of 32 a k-contiguous
//     operand is fetched in 64-byte runs, half a cache line per row and K tile, and the other half of
//     every line is fetched again one tile later.  A k-contiguous operand's stage is stage[row][64]
//     (one load = 8 rows x 128 bytes, every line requested once); a row-contiguous operand's is
//     stage[k][rows] as in contract_hd.hpp, 64 k deep.
//   * 256 x 256 output tile on four wavefronts (one per SIMD, wave tile 128 x 128 = 8 x 8 MFMA blocks,
//     accumulators in 256 AGPRs).  A stage is 32 KiB per operand; the X stages form a ring of NSX, the Y
//     stages a ring of NSY (2 + 2 = 128 KiB; a third stage for one of them measured no gain).
//   * A K tile is two k-steps of 32.  The operand registers of the next k-step are read from LDS while
//     the current one is multiplied (a whole k-step ahead: 128 registers), so every wave has issued its
//     last read of tile t when the last k-step of tile t begins: there, after the barrier that also hands
//     tile t + 1 to the readers, the stages of tile t are free, and the loads of tile t + NSY (Y) and
//     t + NSX (X) are issued into them during the 128 MFMAs that follow, one every SP MFMAs per wave,
//     the operand with the shorter ring first.
//   * Swizzles.  k-contiguous: the 16-byte chunk at position c of a row holds chunk c ^ ((row / 2) % 8)
//     of that row (each lane picks its global source accordingly): 16 consecutive lanes of a
//     ds_read_b128, which read the same chunk of 16 consecutive rows, touch 16 disjoint bank ranges.
//     Row-contiguous: chunk c ^ 2 (k % 4) of a k-row, as in contract_hd.hpp, read with ds_read_b64_tr_b16.
//   * K tail: K may end 16, 32 or 48 elements into a tile.  That tile is loaded from K - 64, so that
//     no address leaves the tensor, and only its last k are multiplied (a k-step that starts inside
//     the tail has the X registers of its first 16 k zeroed).
//   * Loads of tiles beyond the K range are not branched around: they repeat the last tile into a
//     stage that is free by construction.  The epilogue stages through the same LDS, so every load
//     is awaited before it starts.
//
// Restrictions (the dispatcher checks them): both operands gathered in 16-byte vectors with one k
// stride each, K a multiple of 16 and at least 64, operand bases 16-byte aligned.
#pragma once
#include <utility>

#include "contract_h.hpp"
#include "dma_lds.hpp"
#include "hd_addr.hpp"

namespace hiptk
{
    template <int BQ_, int NSX_, int NSY_>
    struct HkGeom
    {
        static constexpr int BP = 256, BQ = BQ_, BK = HK_BK, NSX = NSX_, NSY = NSY_;
        static constexpr int OPX = BP * BK; // elements of X in one stage
        static constexpr int OPY = BQ * BK;
        static constexpr int NXL = BP / 32; // direct loads (1 KiB) per wavefront and K tile
        static constexpr int NYL = BQ / 32;
        static constexpr int YRING      = NSX * OPX; // element offset of the Y ring
        static constexpr int RING_BYTES = (NSX * OPX + NSY * OPY) * 2;
        // (the epilogue double-buffers its staging when it has 132 KiB)
        static constexpr int LDS_BYTES = RING_BYTES > 136 * 1024 ? RING_BYTES : 136 * 1024;
        static_assert(BQ == 256, "wave tiles of 128 columns (8 x 8 blocks: the Hilbert walk)");
        static_assert(NSX >= 2 && NSX <= 3 && NSY >= 2 && NSY <= 3, "rings of 2 or 3 stages");
        static_assert(LDS_BYTES <= 160 * 1024, "LDS of one CU");
    };

    template <typename F, int... I>
    __device__ __forceinline__ void hk_static_for_impl(F&& f, std::integer_sequence<int, I...>)
    {
        (f(std::integral_constant<int, I>{}), ...);
    }
    // f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
    template <int N, typename F>
    __device__ __forceinline__ void hk_static_for(F&& f)
    {
        hk_static_for_impl(f, std::make_integer_sequence<int, N>{});
    }

    // MFMA operand fetch of the 16-row block b of a wave tile, k-step ks (32 k), from a swizzled stage:
    // lane l of v_mfma_f32_16x16x32 holds row l % 16, k = 8 (l / 16) .. + 7.
    template <bool KF, int BR>
    struct HkFrag
    {
        // k-contiguous: one offset per k-step (the swizzle depends on (row / 2) % 8 only, and 16 b is a
        // multiple of 16); row-contiguous: one per block (the swizzle exchanges 8-row chunks within 64 rows)
        int base[KF ? 2 : BR / 32];

        __device__ inline void init(int wrow, int lane)
        {
            if constexpr(KF)
            {
                const int row = wrow + (lane & 15);
#pragma unroll
                for(int ks = 0; ks < 2; ks++)
                    base[ks] = row * HK_BK + (hk_chunk_pos(row, 4 * ks + (lane >> 4)) << 3);
            }
            else
            {
                // a transposing read hands lane L of a 16-lane group element L % 4 of the 64-bit words that
                // the lanes L / 4 + {0, 4, 8, 12} point at: with lane g of the group pointing at rows
                // 4 (g % 4) .. + 3 of k-row g / 4, lane L receives row L at four consecutive k
                const int k = 8 * (lane >> 4) + ((lane & 15) >> 2);
#pragma unroll
                for(int b = 0; b < BR / 32; b++)
                    base[b] = k * BR + hd_row_pos(wrow + 16 * b + 4 * (lane & 3), k);
            }
        }

        __device__ inline u32x4_t load(const uint16_t* opnd, int b, int ks) const
        {
            if constexpr(KF)
                return *(const u32x4_t*)(opnd + base[ks] + b * 16 * HK_BK);
            else
            {
                typedef short4_t __attribute__((address_space(3))) * lds_s4_ptr;
                const uint16_t* p  = opnd + base[b] + ks * 32 * BR;
                const short4_t  lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p));
                const short4_t  hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p + 4 * BR));
                const u32x2_t   l2 = __builtin_bit_cast(u32x2_t, lo);
                const u32x2_t   h2 = __builtin_bit_cast(u32x2_t, hi);
                return u32x4_t{l2[0], l2[1], h2[0], h2[1]};
            }
        }
    };

    // Which block (row i, column j) of the wave tile the m-th MFMA of a k-step multiplies: the 8 x 8 blocks
    // are walked in squares of 2 x 2, the squares row by row.  The order changes nothing in cycles but the
    // clock the device holds (4096^3, k-contiguous operands: 101.6 us row by row or column by column, 100.8
    // row by row in alternating directions, 99.9 in 2 x 2 squares, the same in 2 x 4 strips and along a
    // Z curve; a loop of nothing but these MFMAs: 1741 MHz row by row, 1949 in squares).
    constexpr int hk_block_i(int m, int nbq)
    {
        return 2 * ((m / 4) / (nbq / 2)) + (m % 4) / 2;
    }
    constexpr int hk_block_j(int m, int nbq)
    {
        return 2 * ((m / 4) % (nbq / 2)) + m % 2;
    }
    // ... and along a Hilbert curve through 8 x 8 blocks, where every MFMA shares an operand with the one before it (this
    // kernel's walk: another 0.1 - 0.5 us on 4096^3; the squares above are what the 8 x 6 blocks of contract_hr.hpp are walked in)
    constexpr int hk_hilbert(int m, bool want_i)
    {
        int x = 0, y = 0, t = m;
        for(int s = 1; s < 8; s *= 2)
        {
            const int rx = 1 & (t / 2), ry = 1 & (t ^ rx);
            if(ry == 0)
            {
                if(rx == 1)
                {
                    x = s - 1 - x;
                    y = s - 1 - y;
                }
                const int tmp = x;
                x             = y;
                y             = tmp;
            }
            x += s * rx;
            y += s * ry;
            t /= 4;
        }
        return want_i ? x : y;
    }

    // The MFMA of the main loop, as inline assembly that accumulates in place in AGPRs.  The compiler
    // does not know these are MFMAs, so whoever reads the accumulators afterwards waits first
    // (hk_mfma_drain).
    __device__ __forceinline__ void hk_mfma16_acc(TraitsF16, f32x4_t& acc, const u32x4_t& x, const u32x4_t& y)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
    }
    __device__ __forceinline__ void hk_mfma16_acc(TraitsBF16, f32x4_t& acc, const u32x4_t& x, const u32x4_t& y)
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
    }
    // more wait states than any MFMA needs before its result may be read
    __device__ __forceinline__ void hk_mfma_drain()
    {
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    }
    // ... and the same MFMA as the compiler knows it, for the K tail
    __device__ inline f32x4_t hk_mfma16(TraitsF16, u32x4_t x, u32x4_t y, f32x4_t acc)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, x), __builtin_bit_cast(half8_t, y), acc, 0, 0, 0);
    }
    __device__ inline f32x4_t hk_mfma16(TraitsBF16, u32x4_t x, u32x4_t y, f32x4_t acc)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, x), __builtin_bit_cast(bf16x8_t, y), acc, 0, 0, 0);
    }

    template <typename Tr, bool XKF, bool YKF, int BQ, int NSX, int NSY, int SP>
    __global__ void __launch_bounds__(256, 1) contract_hk_kernel(const KArgs a)
    {
        typedef HkGeom<BQ, NSX, NSY> G;
        constexpr int BP = G::BP, NXL = G::NXL, NYL = G::NYL;
        constexpr int TP = 4, TQ = BQ / 64, WP = 2, WQ = 2; // 32 x 32 blocks of a wave tile (what the epilogue walks)
        // MFMA blocks of a wave tile, k-steps per K tile, MFMAs per k-step, MFMAs between two loads of a wave
        constexpr int NBP = 2 * TP, NBQ = 2 * TQ, KST = 2, NM = NBP * NBQ, SPM = SP;
        constexpr int NL = NXL + NYL; // loads per wave and K tile
        // the operand with the shorter ring is requested first in every tile's window
        constexpr bool YFIRST = NSY <= NSX;
        // loads a wavefront may have outstanding when tile t + 1 must have landed: those of a ring of
        // three that were issued behind it
        constexpr int NWAIT = (NSX == 3 ? NXL : 0) + (NSY == 3 ? NYL : 0);
        static_assert(hk_load_slot(3, NL - 1, SPM) < NM, "a tile's loads are issued within the k-step behind the barrier");
        static_assert(6 * (NBP - 1) < NM && 6 * (NBQ - 1) + 3 < NM, "the operand fetches of a k-step fit under its MFMAs");

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

        const int     kt_begin = blockIdx.z * a.ktiles_per_split;
        const HkSlice sl       = hk_slice(a.K, kt_begin, a.ktiles_per_split);
        const int     nt = sl.nt, klast = sl.klast, tail = sl.tail;

        typedef uint16_t __attribute__((address_space(3))) * lds_u16_ptr;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_u16_ptr)lds; // LDS byte address of the X ring
        // this wave's share of stage 0 of either ring
        const uint32_t wdstx = lds0 + (uint32_t)wave * (NXL * 1024u);
        const uint32_t wdsty = lds0 + G::YRING * 2 + (uint32_t)wave * (NYL * 1024u);

        // byte offsets of this lane's 16 bytes in each of its loads, relative to the tile's k origin
        uint32_t xvoff[NXL], yvoff[NYL];
#pragma unroll
        for(int i = 0; i < NXL; i++)
        {
            const HdSlot s = hk_stage_slot<XKF, BP>((wave * NXL + i) * 64 + lane);
            // (one row mode: the offset is computed, which spares the prologue a round trip to the table; rows beyond P
            // read row 0, as the table has them)
            const int      pr  = p0 + s.row;
            const uint32_t row = a.xp_stride ? (pr < a.P ? (uint32_t)pr * (uint32_t)a.xp_stride : 0u) : (uint32_t)a.xp[pr];
            // (four loads share a write of M0: dma_lds.hpp)
            xvoff[i]           = 2u * (row + (uint32_t)s.k * (uint32_t)a.xk_stride) + (uint32_t)(DMA_BIAS - (i % 4) * 1024);
        }
#pragma unroll
        for(int i = 0; i < NYL; i++)
        {
            const HdSlot s = hk_stage_slot<YKF, BQ>((wave * NYL + i) * 64 + lane);
            const int      qr  = q0 + s.row;
            const uint32_t row = a.yq_stride ? (qr < a.Q ? (uint32_t)qr * (uint32_t)a.yq_stride : 0u) : (uint32_t)a.yq[qr];
            yvoff[i]           = 2u * (row + (uint32_t)s.k * (uint32_t)a.yk_stride) + (uint32_t)(DMA_BIAS - (i % 4) * 1024);
        }
        HkFrag<XKF, BP> fx;
        HkFrag<YKF, BQ> fy;
        fx.init(wp * 128, lane);
        fy.init(wq * (BQ / 2), lane);

        // k origin of the next tile to be requested, per operand (tiles beyond the slice's last one
        // repeat it), and the source and destination of the tile that is being requested
        const uint32_t xkb = 2u * (uint32_t)a.xk_stride;
        const uint32_t ykb = 2u * (uint32_t)a.yk_stride;
        int            xko = sl.k00, yko = sl.k00;
        const char *   xsrc = nullptr, *ysrc = nullptr;
        uint32_t       xdst = 0, ydst = 0;
        // (in two halves of three scalar instructions each, so that neither fills more than the three issue slots beside
        // an MFMA of the loop)
        const char* const xbase = (const char*)a.X - DMA_BIAS;
        const char* const ybase = (const char*)a.Y - DMA_BIAS;
        auto x_open_src = [&]() __attribute__((always_inline)) { xsrc = xbase + (uint64_t)((uint32_t)xko * xkb); };
        auto x_open_dst = [&](auto s_c) __attribute__((always_inline)) {
            constexpr int S = decltype(s_c)::value;
            xdst            = wdstx + S * (G::OPX * 2);
            xko             = hk_next_origin(xko, klast);
        };
        auto y_open_src = [&]() __attribute__((always_inline)) { ysrc = ybase + (uint64_t)((uint32_t)yko * ykb); };
        auto y_open_dst = [&](auto s_c) __attribute__((always_inline)) {
            constexpr int S = decltype(s_c)::value;
            ydst            = wdsty + S * (G::OPY * 2);
            yko             = hk_next_origin(yko, klast);
        };
        auto x_open = [&](auto s_c) __attribute__((always_inline)) {
            x_open_src();
            x_open_dst(s_c);
        };
        auto y_open = [&](auto s_c) __attribute__((always_inline)) {
            y_open_src();
            y_open_dst(s_c);
        };
        // load j of a tile's window: the first NYL (NXL) are Y's (X's) when Y (X) goes first
        auto set_m0 = [&](auto j_c) __attribute__((always_inline)) {
            constexpr int  j   = decltype(j_c)::value;
            constexpr bool isy = YFIRST ? j < NYL : j >= NXL;
            constexpr int  i   = YFIRST ? (j < NYL ? j : j - NYL) : (j < NXL ? j : j - NXL);
            // (the first of four loads into consecutive KiB writes M0 for all of them)
            if constexpr(i % 4 == 0)
                dma_dst<i * 1024>(isy ? ydst : xdst);
        };
        auto load = [&](auto j_c, auto bare_c) __attribute__((always_inline)) {
            constexpr int  j   = decltype(j_c)::value;
            constexpr bool isy = YFIRST ? j < NYL : j >= NXL;
            constexpr int  i   = YFIRST ? (j < NYL ? j : j - NYL) : (j < NXL ? j : j - NXL);
            if constexpr(decltype(bare_c)::value)
                dma_load_in_loop_off<(i % 4) * 1024>(isy ? yvoff[i] : xvoff[i], isy ? ysrc : xsrc);
            else
                dma_load_off<(i % 4) * 1024>(isy ? yvoff[i] : xvoff[i], isy ? ysrc : xsrc);
        };
        // what wave WV does about its loads in front of the MFMA of window slot g: M0 for a load
        // that follows the next MFMA, and the load whose turn it is
        auto window_slot = [&](auto wv_c, auto g_c, auto bare_c) __attribute__((always_inline)) {
            constexpr int WV = decltype(wv_c)::value;
            constexpr int g  = decltype(g_c)::value;
            hk_static_for<NL>([&](auto j_c) __attribute__((always_inline)) {
                constexpr int j  = decltype(j_c)::value;
                constexpr int ls = hk_load_slot(WV, j, SPM);
                if constexpr(ls == g + 1)
                    set_m0(j_c);
                if constexpr(ls == g)
                {
                    // (first slot of a window: inside the loop M0 is written in front of the last MFMA of the k-step
                    // before, see kstep; the prologue writes it here and keeps the load's wait states)
                    if constexpr(g == 0 && !decltype(bare_c)::value)
                        set_m0(j_c);
                    load(j_c, bare_c);
                }
            });
        };

        f32x4_t acc[NBP][NBQ];
#pragma unroll
        for(int i = 0; i < NBP; i++)
#pragma unroll
            for(int j = 0; j < NBQ; j++)
#pragma unroll
                for(int r = 0; r < 4; r++)
                    acc[i][j][r] = 0.f;

        // operand registers: two sets (the k-step that is multiplied, and the next one).  Every block is
        // fetched a whole k-step ahead of its use: a shorter lead would read blocks of tile t during its
        // last k-step, when the loads of tile t + 2 are already overwriting its stage.
        u32x4_t xf[2][NBP], yf[2][NBQ];

        // One k-step: NM MFMAs out of register set KS % 2; the operand fetches of the next k-step (k-step
        // NKS of the stages nx / ny) into the other set, X block i in front of MFMA 6 i and Y block j in
        // front of MFMA 6 j + 3; and this wave's loads of the window slots G0 .. G0 + NM - 1.
        // sched_barrier(0) after every MFMA keeps the issue order as written.
        auto kstep = [&](auto wv_c, auto ks_c, const uint16_t* nx, const uint16_t* ny, auto nks_c, auto g0_c, auto sx_c, auto sy_c) __attribute__((always_inline)) {
            constexpr int KS   = decltype(ks_c)::value;
            constexpr int NKS  = decltype(nks_c)::value;
            constexpr int G0   = decltype(g0_c)::value;
            constexpr int slot = KS & 1;
            hk_static_for<NM>([&](auto m_c) __attribute__((always_inline)) {
                constexpr int m = decltype(m_c)::value;
                // k-step 0: where the next window's tiles lie and go (scalar arithmetic under the MFMAs instead of behind
                // the barrier, where nothing covers it; this wave's loads of the window before have all been issued)
                if constexpr(KS == 0 && m == 7)
                    x_open_src();
                if constexpr(KS == 0 && m == 8)
                    x_open_dst(sx_c);
                if constexpr(KS == 0 && m == 13)
                    y_open_src();
                if constexpr(KS == 0 && m == 17)
                    y_open_dst(sy_c);
                // (all issued in the first three quarters of the k-step: the wait in front of the barrier that follows
                // k-step 0 is also a wait for this wave's own LDS reads, and a read issued four MFMAs before it had not returned)
                if constexpr(m % 6 == 0 && m / 6 < NBP)
                    xf[slot ^ 1][m / 6] = fx.load(nx, m / 6, NKS);
                if constexpr(m % 6 == 3 && m / 6 < NBQ)
                    yf[slot ^ 1][m / 6] = fy.load(ny, m / 6, NKS);
                window_slot(wv_c, std::integral_constant<int, G0 + m>{}, std::true_type{});
                // M0 for the load in the first slot of the window that opens behind this k-step's barrier (an s_nop between
                // the two there would hold up the MFMAs of the wave that every other wave then waits for at the next barrier)
                if constexpr(KS == 0 && m == NM - 1)
                    hk_static_for<NL>([&](auto j_c) __attribute__((always_inline)) {
                        if constexpr(hk_load_slot(decltype(wv_c)::value, decltype(j_c)::value, SPM) == 0)
                            set_m0(j_c);
                    });
                {
                    constexpr int bi = hk_hilbert(m, true), bj = hk_hilbert(m, false);
                    hk_mfma16_acc(Tr{}, acc[bi][bj], xf[slot][bi], yf[slot][bj]);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        };
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        typedef std::integral_constant<int, 2> I2;
        typedef std::integral_constant<int, 3> I3;

        // K tile t, whose ring stages are SX = t % NSX and SY = t % NSY
        auto tile_step = [&](auto wv_c, auto sx_c, auto sy_c) __attribute__((always_inline)) {
            constexpr int   SX = decltype(sx_c)::value;
            constexpr int   SY = decltype(sy_c)::value;
            const uint16_t* cx = lds + SX * G::OPX;
            const uint16_t* cy = lds + G::YRING + SY * G::OPY;
            const uint16_t* nx = lds + ((SX + 1) % NSX) * G::OPX;
            const uint16_t* ny = lds + G::YRING + ((SY + 1) % NSY) * G::OPY;
            // k-step 0 fetches k-step 1 (the window that opened in the last k-step of the tile before goes on)
            kstep(wv_c, I0{}, cx, cy, I1{}, std::integral_constant<int, NM>{}, sx_c, sy_c);
            // Every wave has issued its reads of tile t.  Tile t + 1 must have landed.
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(NWAIT));
            lds_barrier();
            __builtin_amdgcn_sched_barrier(0);
            // the stages of tile t are free: the window of tiles t + NSY (Y) and t + NSX (X) opens
            // k-step 1 fetches k-step 0 of tile t + 1 (beyond the last tile: stale data, not used)
            kstep(wv_c, I1{}, nx, ny, I0{}, I0{}, sx_c, sy_c);
        };

        auto main_loop = [&](auto wv_c) __attribute__((always_inline)) {
            // prologue: the tiles the rings hold when the first window opens, in the order the loop
            // would have requested them
            hk_static_for<3>([&](auto u_c) __attribute__((always_inline)) {
                constexpr int u = decltype(u_c)::value; // windows -3, -2, -1 before tile 0
                // window w requests Y(w + NSY) and X(w + NSX); the last one is opened by the loop's first step
                constexpr int ty = u - 3 + NSY, tx = u - 3 + NSX;
                auto          do_y = [&]() __attribute__((always_inline)) {
                    if constexpr(ty >= 0 && ty < NSY - 1)
                    {
                        y_open(std::integral_constant<int, (ty >= 0 ? ty : 0)>{});
                        hk_static_for<NYL>([&](auto i_c) __attribute__((always_inline)) {
                            constexpr int i = decltype(i_c)::value;
                            if constexpr(i % 4 == 0)
                                dma_dst<i * 1024>(ydst);
                            dma_load_off<(i % 4) * 1024>(yvoff[i], ysrc);
                        });
                    }
                };
                auto do_x = [&]() __attribute__((always_inline)) {
                    if constexpr(tx >= 0 && tx < NSX - 1)
                    {
                        x_open(std::integral_constant<int, (tx >= 0 ? tx : 0)>{});
                        hk_static_for<NXL>([&](auto i_c) __attribute__((always_inline)) {
                            constexpr int i = decltype(i_c)::value;
                            if constexpr(i % 4 == 0)
                                dma_dst<i * 1024>(xdst);
                            dma_load_off<(i % 4) * 1024>(xvoff[i], xsrc);
                        });
                    }
                };
                if constexpr(YFIRST)
                {
                    do_y();
                    do_x();
                }
                else
                {
                    do_x();
                    do_y();
                }
            });
            // tile 0 has landed
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(NWAIT));
            lds_barrier();
#pragma unroll
            for(int i = 0; i < NBP; i++)
                xf[0][i] = fx.load(lds, i, 0);
#pragma unroll
            for(int j = 0; j < NBQ; j++)
                yf[0][j] = fy.load(lds + G::YRING, j, 0);
            // the part of the window of tiles NSY - 1 / NSX - 1 that the last k-step in front of tile 0 would hold
            x_open(std::integral_constant<int, NSX - 1>{});
            y_open(std::integral_constant<int, NSY - 1>{});
            hk_static_for<NM>([&](auto g_c) __attribute__((always_inline)) { window_slot(wv_c, g_c, std::false_type{}); });
            __builtin_amdgcn_sched_barrier(0);

            // unrolled over the rings' common period, so that every LDS address is an immediate
            constexpr int PERIOD = NSX == NSY ? NSX : NSX * NSY;
            int           t      = 0;
            for(; t + PERIOD <= nt; t += PERIOD)
                hk_static_for<PERIOD>([&](auto u_c) __attribute__((always_inline)) {
                    constexpr int u = decltype(u_c)::value;
                    tile_step(wv_c, std::integral_constant<int, u % NSX>{}, std::integral_constant<int, u % NSY>{});
                });
            hk_static_for<PERIOD - 1>([&](auto u_c) __attribute__((always_inline)) {
                constexpr int u = decltype(u_c)::value;
                if(t + u < nt)
                    tile_step(wv_c, std::integral_constant<int, u % NSX>{}, std::integral_constant<int, u % NSY>{});
            });
        };

        switch(wave)
        {
        case 0: main_loop(I0{}); break;
        case 1: main_loop(I1{}); break;
        case 2: main_loop(I2{}); break;
        default: main_loop(I3{}); break;
        }
        // the last MFMAs have written their results, and every load has landed (those beyond the K range
        // too: the epilogue stages through this LDS)
        hk_mfma_drain();
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        lds_barrier();
        if(tail)
        {
            // tile nt was loaded from K - 64; its last `tail` runs of 16 k are the last of K.  A k-step
            // of 32 that starts 16 before them has the lanes that hold its first 16 k of X read as zero.
            const uint16_t* sx    = lds + (nt % NSX) * G::OPX;
            const uint16_t* sy    = lds + G::YRING + (nt % NSY) * G::OPY;
            const bool      upper = (lane >> 4) >= 2;
#pragma unroll
            for(int ks = 0; ks < 2; ks++)
                if(4 - tail < 2 * ks + 2)
                {
                    const bool whole = 4 - tail <= 2 * ks;
#pragma unroll
                    for(int j = 0; j < NBQ; j++)
                        yf[0][j] = fy.load(sy, j, ks);
#pragma unroll
                    for(int i = 0; i < NBP; i++)
                    {
                        const u32x4_t v = fx.load(sx, i, ks);
                        const u32x4_t x = (whole || upper) ? v : u32x4_t{0u, 0u, 0u, 0u};
#pragma unroll
                        for(int j = 0; j < NBQ; j++)
                            acc[i][j] = hk_mfma16(Tr{}, x, yf[0][j], acc[i][j]);
                    }
                }
            lds_barrier();
        }
        // (accumulators pinned in AGPRs: without it the compiler moved them to VGPRs and spilled)
#pragma unroll
        for(int i = 0; i < NBP; i++)
#pragma unroll
            for(int j = 0; j < NBQ; j++)
                asm volatile("" : "+a"(acc[i][j]));
        epilogue_h16<Tr, WP, WQ, TP, TQ, G::LDS_BYTES, true>(a, acc, lds, p0, q0, p_own, q_own);
    }

    template <typename Tr, bool XKF, bool YKF, int BQ, int NSX, int NSY, int SP>
    int launch_hk(const KArgs& a, hipStream_t stream)
    {
        typedef HkGeom<BQ, NSX, NSY> G;
        if(a.K < G::BK || a.K % 16 != 0)
            return (int)hipErrorInvalidValue;
        auto                    kern = contract_hk_kernel<Tr, XKF, YKF, BQ, NSX, NSY, SP>;
        static const hipError_t attr = hipFuncSetAttribute(
            (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if(attr != hipSuccess)
            return (int)attr;
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(kern, grid, dim3(256), G::LDS_BYTES, stream, a);
        return (int)hipGetLastError();
    }
}

// Registry lines: operands gathered in 16-byte vectors, one k stride each, K a multiple of 16, at least 64.
#define HIPTK_HK_ENTRY(TR, ID, BQ, XKF, YKF, NSX, NSY, SP)                                                  \
    {                                                                                                       \
        TR::CLS, ID, XKF, YKF, 8, 8, true, 256, BQ, 64, 256, hiptk::HkGeom<BQ, NSX, NSY>::LDS_BYTES,         \
            #TR "_256x" #BQ "x64_x" #XKF "8_y" #YKF "8_kafftrue_direct2x2_m16x16x32",                       \
            &hiptk::launch_hk<hiptk::TR, XKF, YKF, BQ, NSX, NSY, SP>, 16, 32                                  \
    }
#define HIPTK_HK_TILE(TR, ID, BQ, NSX, NSY, SP)                                                              \
    HIPTK_HK_ENTRY(TR, ID, BQ, true, true, NSX, NSY, SP), HIPTK_HK_ENTRY(TR, ID, BQ, true, false, NSX, NSY, SP), \
        HIPTK_HK_ENTRY(TR, ID, BQ, false, true, NSX, NSY, SP), HIPTK_HK_ENTRY(TR, ID, BQ, false, false, NSX, NSY, SP)
