// 16-bit (f16 / bf16) contraction kernel for gfx950 on v_mfma_f32_16x16x32 for operands whose reduction
// modes do not fuse into one stride (k offsets from tables): operand tiles go from global memory straight
// into a ring of four LDS stages in K tiles of 32.
//
// Same MFMAs, register layout, issue-slot rules and epilogue as contract_hk.hpp.  What differs is the
// ring: problems of this kind gather short runs from all over their tensors (the rank-6 benchmark
// layout: 64-byte runs of X, 16-byte runs of Y), their loads take long to land, and what covers a load
// is the number of K tiles between the moment its stage is free and the moment it is read.  A stage of
// K tiles of 64 is held until all 64 k are read, and two of them fill the LDS: a load has at most one
// tile of MFMA time (such a loop ran at 46 % MFMA issue on the rank-6 configuration); four stages of
// 32 k in the same bytes give it two to three, and the wait in front of the barrier costs nothing.
//
//   * 256 x 192 output tile on four wavefronts (wave tile 128 x 96 = 8 x 6 MFMA blocks, 192 AGPRs), K in
//     steps of 32 = one MFMA deep: a K tile is one k-step of 48 MFMAs.  The operand registers of tile
//     t + 1 are read from LDS while tile t is multiplied (two register sets; all reads are issued in the
//     first three quarters of the step), so at the barrier that opens step t every wave has finished
//     reading tile t: its stage is free, the loads of tile t + 4 are issued into it during the step, and
//     tile t + 1 - which the step reads - must have landed: loads complete in issue order, so each wave
//     waits until only the loads issued after those of tile t + 1 are outstanding (the table entries
//     requested right after them and the loads of two steps: 20).
//   * k offsets: the 32 + 32 table entries of a K tile are themselves loaded straight into LDS (a private
//     ring of four 512-byte slots per wave: no result of an asm load ever lands in a register the
//     compiler might copy before the data is there) at the end of the step nine tiles ahead of the
//     multiplication, read back with ds_read_b32 four steps later, when that step's wait has covered
//     them, and added to the lanes' row parts one step before the loads that use them go out (two sets
//     of offsets: a step's loads go on while the next step's offsets are formed).  Every address built
//     from such an entry is clamped to the last vector the tables address, so that an entry that did not
//     come out of LDS as it went in could give a wrong result but never a request outside the tensor.
//   * Stage layouts.  Row-contiguous operand: stage[k][rows], 8-row chunk c ^ 2 (k % 4), read with
//     ds_read_b64_tr_b16.  k-contiguous operand: stage[row][32] with chunk c ^ ((row / 4) % 4) as in
//     contract_hd.hpp, or, where the vectors of consecutive rows are neighbours in memory and those of
//     consecutive k are not (KArgs::x_chunked / y_chunked), chunk-major stage[4][rows][8]: what matters
//     is which 4 consecutive lanes of a load fetch 64 contiguous bytes, because the vector cache is
//     accessed once per distinct 64 bytes: with 4 lanes in 4 places a 1 KiB load costs 64 accesses
//     instead of 16, and on the rank-6 configuration the texture path was then busy all of the time
//     (main loop 137 k cycles; 117 k chunk-major; 98 k are MFMAs).
//   * K tail: K may end 16 elements into a tile.  That tile is loaded from K - 32, so that no address
//     leaves the tensor, and the lanes that hold its first 16 k of X read as zero.
//
// Restrictions (the dispatcher checks them): both operands gathered in 16-byte vectors, K a multiple of
// 16 and at least 32, operand bases 16-byte aligned.
#pragma once
#include "contract_hk.hpp"

namespace hiptk
{
    template <int BQ_>
    struct HrGeom
    {
        static constexpr int BP = 256, BQ = BQ_, BK = HD_BK, NS = 4;
        static constexpr int OPX = BP * BK, OPY = BQ * BK, STAGE = OPX + OPY; // elements
        static constexpr int NXL = BP / 64, NYL = BQ / 64; // direct loads (1 KiB) per wavefront and K tile
        static constexpr int RING_BYTES = NS * STAGE * 2;
        static constexpr int KTAB       = RING_BYTES; // per wave four slots of 64 + 64 entries
        static constexpr int LDS_BYTES  = KTAB + 4 * 4 * 512;
        static constexpr int EPI_BYTES  = BQ_ == 256 ? 136 * 1024 : 104 * 1024; // what the epilogue wants for two staging buffers
        static_assert(BQ == 256 || BQ == 192, "wave tiles of 128 or 96 columns");
        static_assert(LDS_BYTES >= EPI_BYTES && LDS_BYTES <= 160 * 1024, "LDS of one CU");
    };

    // MFMA operand fetch of the 16-row block b of a wave tile from a swizzled stage of 32 k:
    // lane l of v_mfma_f32_16x16x32 holds row l % 16, k = 8 (l / 16) .. + 7.
    template <bool KF, int BR>
    struct HrFrag
    {
        int base[BR / 32];

        __device__ inline void init(int wrow, int lane, bool chunked)
        {
            if constexpr(KF)
            {
#pragma unroll
                for(int b = 0; b < BR / 32; b++)
                    base[b] = hr_chunk_elem<BR>(wrow + 16 * b + (lane & 15), lane >> 4, chunked);
            }
            else
            {
                const int k = 8 * (lane >> 4) + ((lane & 15) >> 2);
#pragma unroll
                for(int b = 0; b < BR / 32; b++)
                    base[b] = k * BR + hd_row_pos(wrow + 16 * b + 4 * (lane & 3), k);
            }
        }
        __device__ inline u32x4_t load(const uint16_t* opnd, int b) const
        {
            if constexpr(KF)
                return *(const u32x4_t*)(opnd + base[b]);
            else
            {
                typedef short4_t __attribute__((address_space(3))) * lds_s4_ptr;
                const uint16_t* p  = opnd + base[b];
                const short4_t  lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p));
                const short4_t  hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p + 4 * BR));
                const u32x2_t   l2 = __builtin_bit_cast(u32x2_t, lo);
                const u32x2_t   h2 = __builtin_bit_cast(u32x2_t, hi);
                return u32x4_t{l2[0], l2[1], h2[0], h2[1]};
            }
        }
    };

    // The MFMA of a step in front of which the j-th table entry is read from LDS: from the fourth on, leaving out those that
    // hold an operand fetch (X's at m % 4 == 1, Y's at m % 6 == 2), so that with a direct load and a write of M0 no MFMA has
    // more than three instructions in front of it.
    constexpr int hr_table_read_slot(int j)
    {
        int m = 2;
        for(int n = -1; n < j;)
        {
            m++;
            if(m % 4 != 1 && m % 6 != 2)
                n++;
        }
        return m;
    }

    template <typename Tr, bool XKF, bool YKF, int BQ>
    __global__ void __launch_bounds__(256, 1) contract_hr_kernel(const KArgs a)
    {
        typedef HrGeom<BQ> G;
        constexpr int BP = G::BP, NS = G::NS, NXL = G::NXL, NYL = G::NYL, NL = NXL + NYL;
        constexpr int TP = 4, TQ = BQ / 64, WP = 2, WQ = 2; // 32 x 32 blocks of a wave tile (what the epilogue walks)
        constexpr int NBP = 2 * TP, NBQ = 2 * TQ, NM = NBP * NBQ; // MFMA blocks, MFMAs per K tile
        constexpr int SPM = NM / NL >= 5 ? 5 : NM / NL; // MFMAs between two loads of a wave (the last one in front of the first offset)
        // loads a wavefront issues per step: the tile's, then two of table entries; and how many may be
        // outstanding when tile t + 1 must have landed: the table entries requested right behind it and the loads
        // of the two steps after that
        constexpr int PER_STEP = NL + 2, NWAIT = 2 + (NS - 2) * PER_STEP;
        // MFMA slots of a step: the table request's two loads (each with its M0 write one MFMA earlier), the first offset
        constexpr int TRQ0 = NM - 6, TF0 = NM - 13;
        static_assert(hk_load_slot(3, NL - 1, SPM) + 1 < TRQ0 && TF0 > 4 * (NBP - 1) + 1 && TF0 > 6 * (NBQ - 1) + 2 && TF0 + NL <= TRQ0
                          && hr_table_read_slot(NL - 1) < TF0,
                      "a tile's loads and table work fit under its MFMAs, the offsets behind the last operand read");
        static_assert(NS == 4, "stage, table slot and offset set indices share the period 4");

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
        const HdSlice sl       = hd_slice(a.K, kt_begin, a.ktiles_per_split);
        const int     nt = sl.nt, kmax = sl.kmax;
        const bool    half = sl.half != 0;

        typedef uint16_t __attribute__((address_space(3))) * lds_u16_ptr;
        typedef const uint32_t __attribute__((address_space(3))) * lds_u32_cptr;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_u16_ptr)lds; // LDS byte address of the ring
        // this wave's share of either operand of stage 0, and its table slots
        const uint32_t     wdstx = lds0 + (uint32_t)wave * (NXL * 1024u);
        const uint32_t     wdsty = lds0 + G::OPX * 2 + (uint32_t)wave * (NYL * 1024u);
        const uint32_t     wtab  = lds0 + G::KTAB + (uint32_t)wave * 2048u;
        const lds_u32_cptr tab0  = (lds_u32_cptr)((lds_u16_ptr)lds + G::KTAB / 2 + wave * 1024);
        const uint32_t     tlane = 4u * (uint32_t)(lane & 31); // (32 entries per tile and table; the upper lanes load them again)

        // per load j (X's first): the row part of this lane's byte offset, and where its table entry lies in slot 0
        uint32_t     rowb[NL];
        lds_u32_cptr tent[NL];
        uint32_t     te[NL];
        uint32_t     voff[2][NL]; // the offsets of the loads of a tile, two sets
#pragma unroll
        for(int i = 0; i < NXL; i++)
        {
            const HdSlot s = hr_slot<XKF, BP>((wave * NXL + i) * 64 + lane, a.x_chunked != 0);
            rowb[i]        = 2u * (uint32_t)a.xp[p0 + s.row];
            tent[i]        = tab0 + s.k;
        }
#pragma unroll
        for(int i = 0; i < NYL; i++)
        {
            const HdSlot s = hr_slot<YKF, BQ>((wave * NYL + i) * 64 + lane, a.y_chunked != 0);
            rowb[NXL + i]  = 2u * (uint32_t)a.yq[q0 + s.row];
            tent[NXL + i]  = tab0 + 64 + s.k;
        }
        HrFrag<XKF, BP> fx;
        HrFrag<YKF, BQ> fy;
        fx.init(wp * 128, lane, a.x_chunked != 0);
        fy.init(wq * (BQ / 2), lane, a.y_chunked != 0);

        // table entries of the next tile to be requested (its origin before clamping: a tile beyond K is the
        // tail tile again, one beyond the slice a tile of the next slice: harmless, its stage is free)
        int      tk = kt_begin * HD_BK;
        uint64_t tofs = 0;
        // phase 0: the tile's (clamped) position in the tables; 1: the destination of X's entries; 2: X's entries; 3: the
        // destination of Y's; 4: Y's entries (no phase holds more than the three instructions an MFMA leaves room for)
        auto t_request_part = [&](auto slot_c, auto phase_c, auto bare_c) __attribute__((always_inline)) {
            constexpr int S = decltype(slot_c)::value, PH = decltype(phase_c)::value;
            if constexpr(PH == 0)
            {
                const int kc = tk < kmax ? tk : kmax;
                tofs         = 4ull * (uint64_t)(uint32_t)kc;
                tk += HD_BK;
            }
            if constexpr(PH == 1)
                dma_dst<S * 512>(wtab);
            if constexpr(PH == 3)
                dma_dst<S * 512 + 256>(wtab);
            if constexpr(PH == 2 || PH == 4)
            {
                const char* src = (const char*)(PH == 2 ? (const void*)a.xk : (const void*)a.yk) + tofs;
                if constexpr(decltype(bare_c)::value)
                    dma_load1_bare(tlane, src);
                else
                    dma_load1(tlane, src);
            }
        };
        auto t_request = [&](auto slot_c) __attribute__((always_inline)) {
            hk_static_for<5>([&](auto ph_c) __attribute__((always_inline)) { t_request_part(slot_c, ph_c, std::false_type{}); });
        };
        auto t_read = [&](auto slot_c, auto j_c) __attribute__((always_inline)) {
            constexpr int S = decltype(slot_c)::value, j = decltype(j_c)::value;
            te[j]           = tent[j][S * 128];
        };
        auto t_form = [&](auto j_c, auto vs_c) __attribute__((always_inline)) {
            constexpr int  j = decltype(j_c)::value, VS = decltype(vs_c)::value;
            const uint32_t last = j < NXL ? a.x_last_vec : a.y_last_vec;
            const uint32_t o    = rowb[j] + 2u * te[j];
            voff[VS][j]         = o < last ? o : last;
        };
        auto t_offsets = [&](auto slot_c, auto vs_c) __attribute__((always_inline)) {
            hk_static_for<NL>([&](auto j_c) __attribute__((always_inline)) { t_read(slot_c, j_c); });
            hk_static_for<NL>([&](auto j_c) __attribute__((always_inline)) { t_form(j_c, vs_c); });
        };
        // load j of the tile that goes into stage S, with the offsets of set VS
        auto set_m0 = [&](auto j_c, auto s_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value, S = decltype(s_c)::value;
            if constexpr(j < NXL)
                dma_dst<S * (G::STAGE * 2) + j * 1024>(wdstx);
            else
                dma_dst<S * (G::STAGE * 2) + (j - NXL) * 1024>(wdsty);
        };
        auto load = [&](auto j_c, auto vs_c, auto bare_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value, VS = decltype(vs_c)::value;
            if constexpr(decltype(bare_c)::value)
                dma_load_in_loop(voff[VS][j], j < NXL ? a.X : a.Y);
            else
                dma_load(voff[VS][j], j < NXL ? a.X : a.Y);
        };
        auto load_all = [&](auto s_c, auto vs_c) __attribute__((always_inline)) {
            hk_static_for<NL>([&](auto j_c) __attribute__((always_inline)) {
                set_m0(j_c, s_c);
                load(j_c, vs_c, std::false_type{});
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

        u32x4_t xf[2][NBP], yf[2][NBQ];

        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        typedef std::integral_constant<int, 2> I2;
        typedef std::integral_constant<int, 3> I3;

        // Step t (T = t % 4): multiplies tile t out of register set t % 2 while it fetches tile t + 1 into the other
        // set, issues this wave's loads of tile t + 4 into the stage tile t has left (offset set t % 2), turns the table
        // entries of tile t + 5 into the offsets of the next step's loads, and requests those of tile t + 9.
        auto tile_step = [&](auto wv_c, auto t_c) __attribute__((always_inline)) {
            constexpr int   WV = decltype(wv_c)::value, T = decltype(t_c)::value;
            const uint16_t* nx = lds + ((T + 1) & 3) * G::STAGE;
            const uint16_t* ny = nx + G::OPX;
            // Tile t + 1 must have landed; every wave has finished reading tile t.
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(NWAIT));
            lds_barrier();
            __builtin_amdgcn_sched_barrier(0);
            hk_static_for<NM>([&](auto m_c) __attribute__((always_inline)) {
                constexpr int m = decltype(m_c)::value;
                // table work: one entry out of LDS in front of each of NL early MFMAs (hr_table_read_slot); one offset each from MFMA TF0 on, behind
                // the step's last operand read (LDS reads return in order: the entries have long arrived; formed eight MFMAs
                // behind their reads, the wait in front of each cost 37 cycles a step)
                hk_static_for<NL>([&](auto j_c) __attribute__((always_inline)) {
                    if constexpr(hr_table_read_slot(decltype(j_c)::value) == m)
                        t_read(std::integral_constant<int, (T + 1) & 3>{}, j_c); // (tile t + 5: slot (t + 5) % 4)
                });
                if constexpr(m >= TF0 && m < TF0 + NL)
                    t_form(std::integral_constant<int, (m >= TF0 && m < TF0 + NL) ? m - TF0 : 0>{}, std::integral_constant<int, (T + 1) & 1>{});
                // operand fetches of tile t + 1: all issued in the first three quarters of the step, so that the barrier
                // of the next step does not wait for them
                if constexpr(m % 4 == 1 && m / 4 < NBP)
                    xf[(T + 1) & 1][m / 4] = fx.load(nx, m / 4);
                if constexpr(m % 6 == 2 && m / 6 < NBQ)
                    yf[(T + 1) & 1][m / 6] = fy.load(ny, m / 6);
                // this wave's loads of tile t + 4, each with its M0 write one MFMA earlier
                hk_static_for<NL>([&](auto j_c) __attribute__((always_inline)) {
                    constexpr int j  = decltype(j_c)::value;
                    constexpr int ls = hk_load_slot(WV, j, SPM) + 1;
                    if constexpr(ls == m + 1)
                        set_m0(j_c, std::integral_constant<int, T>{});
                    if constexpr(ls == m)
                        load(j_c, std::integral_constant<int, T & 1>{}, std::true_type{});
                });
                // the table entries of tile t + 9 (slot (t + 9) % 4: the entries read from it above have been used)
                if constexpr(m >= TRQ0 && m < TRQ0 + 5)
                    t_request_part(std::integral_constant<int, (T + 1) & 3>{}, std::integral_constant<int, (m >= TRQ0 && m < TRQ0 + 5) ? m - TRQ0 : 0>{}, std::true_type{});
                {
                    constexpr int bi = hk_block_i(m, NBQ), bj = hk_block_j(m, NBQ);
                    hk_mfma16_acc(Tr{}, acc[bi][bj], xf[T & 1][bi], yf[T & 1][bj]);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        };

        auto main_loop = [&](auto wv_c) __attribute__((always_inline)) {
            // Prologue.  The table entries of tiles 0 .. 8 and the loads of tiles 0 .. 3, each after its offsets, issued so
            // that as many loads follow those of tiles 2 and 3 as follow those of every later tile (20: the loop's wait
            // counts the loads issued after those of the tile it needs; tiles 0 and 1 are waited for here).
            t_request(I0{});
            t_request(I1{});
            t_request(I2{});
            t_request(I3{});
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0)); // (the slots are reused below: tiles 4 .. 7 go where 0 .. 3 were read)
            t_offsets(I0{}, I0{});
            load_all(I0{}, I0{});
            t_offsets(I1{}, I1{});
            load_all(I1{}, I1{});
            t_offsets(I2{}, I0{});
            t_offsets(I3{}, I1{}); // (read before its slot is overwritten; set 1 is free again: the loads of tile 1 are out)
            __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0);
            t_request(I0{}); // tiles 4, 5, 6
            t_request(I1{});
            t_request(I2{});
            load_all(I2{}, I0{});
            t_request(I3{}); // tile 7
            load_all(I3{}, I1{});
            // tiles 0 and 1 have landed, and the entries of tiles 4 .. 6 (everything but tile 2's loads, tile 7's
            // entries and tile 3's loads)
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(NL + 2 + NL));
            lds_barrier();
#pragma unroll
            for(int i = 0; i < NBP; i++)
                xf[0][i] = fx.load(lds, i);
#pragma unroll
            for(int j = 0; j < NBQ; j++)
                yf[0][j] = fy.load(lds + G::OPX, j);
            t_offsets(I0{}, I0{}); // the loads of tile 4, which step 0 issues
            t_request(I0{}); // tile 8
            __builtin_amdgcn_sched_barrier(0);

            int t = 0;
            for(; t + 4 <= nt; t += 4)
            {
                tile_step(wv_c, I0{});
                tile_step(wv_c, I1{});
                tile_step(wv_c, I2{});
                tile_step(wv_c, I3{});
            }
            if(t < nt)
                tile_step(wv_c, I0{});
            if(t + 1 < nt)
                tile_step(wv_c, I1{});
            if(t + 2 < nt)
                tile_step(wv_c, I2{});
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
        if(half)
        {
            // tile nt was loaded from K - 32; its k 16 .. 31 are the last 16 of K
            const uint16_t* sx    = lds + (nt & 3) * G::STAGE;
            const bool      upper = (lane >> 4) >= 2;
#pragma unroll
            for(int j = 0; j < NBQ; j++)
                yf[0][j] = fy.load(sx + G::OPX, j);
#pragma unroll
            for(int i = 0; i < NBP; i++)
            {
                const u32x4_t v = fx.load(sx, i);
                const u32x4_t x = upper ? v : u32x4_t{0u, 0u, 0u, 0u};
#pragma unroll
                for(int j = 0; j < NBQ; j++)
                    acc[i][j] = hk_mfma16(Tr{}, x, yf[0][j], acc[i][j]);
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

    template <typename Tr, bool XKF, bool YKF, int BQ>
    int launch_hr(const KArgs& a, hipStream_t stream)
    {
        typedef HrGeom<BQ> G;
        if(a.K < G::BK || a.K % 16 != 0)
            return (int)hipErrorInvalidValue;
        auto                    kern = contract_hr_kernel<Tr, XKF, YKF, BQ>;
        static const hipError_t attr = hipFuncSetAttribute(
            (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if(attr != hipSuccess)
            return (int)attr;
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(kern, grid, dim3(256), G::LDS_BYTES, stream, a);
        return (int)hipGetLastError();
    }
}

// Registry lines: operands gathered in 16-byte vectors, k offsets from tables, K a multiple of 16, at least 32.
#define HIPTK_HR_ENTRY(TR, ID, BQ, XKF, YKF)                                                             \
    {                                                                                                    \
        TR::CLS, ID, XKF, YKF, 8, 8, false, 256, BQ, 32, 256, hiptk::HrGeom<BQ>::LDS_BYTES,               \
            #TR "_256x" #BQ "x32_x" #XKF "8_y" #YKF "8_kafffalse_direct2x2_ring4_m16x16x32",             \
            &hiptk::launch_hr<hiptk::TR, XKF, YKF, BQ>, 16, 32                                               \
    }
