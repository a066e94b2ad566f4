// 16-bit (f16 / bf16) contraction kernel for gfx950 whose operand tiles go from global memory
// straight into LDS (global_load_lds_dwordx4), without passing through registers.
//
// Same problem statement and epilogue as contract_h.hpp; what differs is the main loop:
//
//   * 256 x 256 or 256 x 192 output tile on four wavefronts (one per SIMD, wave tile 128 x 128 or
//     128 x 96, accumulators in AGPRs), K in steps of 32, four LDS stages (16 KiB of X and 16 / 12 KiB
//     of Y each) used as a ring.  While K tile t is multiplied, the Y loads of tile t + 3 and the X
//     loads of tile t + 4 are issued, so a load has two to three tiles of MFMA time to land, and no
//     staging registers, no register -> LDS stores and no write bank conflicts remain.
//   * A direct load writes 64 lanes x 16 bytes to consecutive LDS addresses, so rows cannot be padded.
//     Bank conflicts of the operand reads are avoided by an XOR swizzle instead: the 16-byte chunk at
//     LDS position c of a row holds the chunk c ^ f(row) of that row, which each lane realises by
//     choosing its global source address; the reads apply the same XOR.
//       row-index-contiguous operand: stage[k][rows], f(k) = 2 * (k % 4); read with ds_read_b64_tr_b16
//           (a 16-lane group touches 4 k-rows x 32 bytes: 4 disjoint bank ranges)
//       k-contiguous operand:         stage[row][32], f(row) = (row / 4) % 4; read with ds_read_b128
//           (16 consecutive rows, one chunk each: 4 x 4 disjoint bank ranges)
//   * A single wavefront per SIMD issues at most one instruction every four cycles, eight per
//     32-cycle MFMA: the loop is unrolled over the four ring stages so that every LDS address is an
//     immediate, sources and destinations are running scalars, and loads of tiles beyond the K range
//     are not branched around but pointed at spare LDS.
//   * The texture path takes one 1 KiB load per 16 cycles and CU, and a wavefront whose load is not
//     accepted stalls with all its MFMAs behind it.  The four wavefronts run in lock step, so each
//     issues its loads in MFMA slots of its own: the path then sees one load per MFMA instead of
//     four at once.
//   * The compiler does not see these loads (inline assembly: it would otherwise wait for every
//     outstanding direct load before each LDS read), so the waits are placed by hand: loads complete
//     in issue order, and before the barrier that hands tile t + 1 to the readers each wavefront waits
//     until only the loads issued after those of tile t + 1 are outstanding.
//   * K offsets from tables (reduction modes that do not fuse into one stride): the 32 + 32 table
//     entries of a K tile are themselves loaded straight into LDS (one 4-byte load per lane, a private
//     ring of four 256-byte slots per wavefront) seven tiles ahead of the multiplication, read back
//     with ds_read_b32 once the same per-tile wait has covered them, and added to the lane's row
//     offset to give the source address of its 16 bytes.
//   * K tail: K may end 16 elements into a tile (one MFMA k-step).  That tile is loaded from K - 32,
//     so that no address leaves the tensor, and only its second k-step is multiplied.
//
// Restrictions (the dispatcher checks them): both operands gathered in 16-byte vectors, K a
// multiple of 16 and at least 32.
#pragma once
#include "contract_h.hpp"
#include "dma_lds.hpp"
#include "hd_addr.hpp"

namespace hiptk
{
    template <int BQ_, bool KAFF>
    struct HdGeom
    {
        static constexpr int BP = 256, BQ = BQ_, BK = 32, NS = 4;
        static constexpr int OPX   = BP * BK; // elements of X in one stage
        static constexpr int OPY   = BQ * BK;
        static constexpr int STAGE = OPX + OPY;
        static constexpr int NYL   = BQ / 64; // direct loads (1 KiB) of Y per wavefront and K tile; X: 4
        static constexpr int RING  = NS * STAGE * 2; // bytes
        static constexpr int EPI   = RING + 8192; // what the epilogue may use (it double-buffers its staging)
        static constexpr int SPARE = EPI; // 4 KiB per wave: where loads beyond the K range land
        static constexpr int KTAB  = SPARE + 16384; // table form: 4 slots x 256 bytes per wave
        static constexpr int LDS_BYTES = KTAB + (KAFF ? 0 : 4096);
        static_assert(BQ == 256 || BQ == 192, "wave tiles of 128 or 96 columns");
        static_assert(LDS_BYTES <= 160 * 1024, "LDS of one CU");
    };

    typedef const uint32_t __attribute__((address_space(3))) * lds_u32_cptr;

    // One operand's share of a wavefront's direct loads: BR / 64 loads of 1 KiB per K tile.
    template <bool KF, int BR, bool KAFF>
    struct HdLoader
    {
        static constexpr int NL = BR / 64;
        uint32_t     voff[NL]; // byte offsets of this lane's 16 bytes (affine K: relative to the tile's k origin)
        uint32_t     rowb[KAFF ? 1 : NL]; // table form: the row part of voff, in bytes
        lds_u32_cptr kent[(KAFF || KF) ? 1 : NL]; // table form: this lane's entry in slot 0 of the wave's table ring
        uint32_t     last; // table form: byte offset of the last vector the tables address

        // rtab: row offset table; r0: first row of the tile; kstride: element stride of k (affine form);
        // tab0: slot 0 of the wave's k-table ring; tabofs: first entry of this operand in a slot
        __device__ inline void init(const int32_t* rtab, int r0, int kstride, int wave, int lane, lds_u32_cptr tab0, int tabofs,
                                    uint32_t last_vec)
        {
            last = last_vec;
#pragma unroll
            for(int i = 0; i < NL; i++)
            {
                // the 16-byte slot of the operand stage this lane fills, and what belongs there
                const HdSlot sl      = hd_slot<KF, BR>((wave * NL + i) * 64 + lane);
                const int    rowpart = rtab[r0 + sl.row];
                const int    kidx    = sl.k;
                if constexpr(KAFF)
                    voff[i] = 2u * ((uint32_t)rowpart + (uint32_t)kidx * (uint32_t)kstride);
                else
                {
                    rowb[i] = 2u * (uint32_t)rowpart;
                    voff[i] = 0;
                    if(!KF || i == 0) // (k-contiguous: the chunk a lane fetches is the same for all its loads)
                        kent[KF ? 0 : i] = tab0 + tabofs + kidx;
                }
            }
        }

        // Table form: the offsets of the tile whose table entries are in ring slot S.
        // Two halves, so that the LDS latency passes between them.
        template <int S>
        __device__ inline void read_entries(uint32_t (&e)[NL]) const
        {
            if constexpr(!KAFF)
            {
#pragma unroll
                for(int i = 0; i < ((KF) ? 1 : NL); i++)
                    e[i] = kent[i][S * 64];
            }
        }
        // (clamped to the last vector the tables address: an entry that did not come out of LDS as it
        // went in must not become a request outside the tensor)
        __device__ inline void set_offsets(const uint32_t (&e)[NL], uint32_t (&out)[NL]) const
        {
            if constexpr(!KAFF)
            {
#pragma unroll
                for(int i = 0; i < NL; i++)
                {
                    const uint32_t o = rowb[i] + 2u * e[KF ? 0 : i];
                    out[i]           = o < last ? o : last;
                }
            }
        }
    };

    // MFMA operand fetch of the 32-row block i of a wave tile, k-substep ks (16 k), from a swizzled stage.
    template <bool KF, int BR>
    struct HdFrag
    {
        static constexpr int NB = BR / 64; // 32-row blocks per wave tile
        int base[KF ? 2 : NB]; // element offsets inside the operand stage

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
                for(int i = 0; i < NB; i++)
                {
                    const int r = wrow + i * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                    base[i]     = k * BR + ((((r >> 3) ^ sw) << 3) | (r & 7));
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
                const uint16_t* p  = opnd + base[i] + ks * 16 * BR;
                const short4_t  lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p));
                const short4_t  hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p + 4 * BR));
                const u32x2_t   l2 = __builtin_bit_cast(u32x2_t, lo);
                const u32x2_t   h2 = __builtin_bit_cast(u32x2_t, hi);
                return u32x4_t{l2[0], l2[1], h2[0], h2[1]};
            }
        }
    };

    template <typename Tr, bool XKF, bool YKF, int BQ, bool KAFF>
    __global__ void __launch_bounds__(256, 1) contract_hd_kernel(const KArgs a)
    {
        typedef HdGeom<BQ, KAFF> G;
        constexpr int BP = G::BP, BK = G::BK, NS = G::NS, NYL = G::NYL;
        constexpr int TP = 4, TQ = BQ / 64, WP = 2, WQ = 2, NM = TP * TQ;
        // loads a wavefront may have outstanding when tile t + 1 must have landed: the X loads of
        // tile t + 2 and everything issued for the tiles after it (table form: two table loads)
        constexpr int NWAIT = 8 + 2 * NYL + (KAFF ? 0 : 2);

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

        // This slice's K tiles: nt whole ones, and the 16-element tail when the slice ends at K
        const int     kt_begin = blockIdx.z * a.ktiles_per_split;
        const HdSlice sl       = hd_slice(a.K, kt_begin, a.ktiles_per_split);
        const int     nt = sl.nt, n_load = sl.n_load, kmax = sl.kmax, k00 = sl.k00, klast = sl.klast;
        const bool    half = sl.half != 0;

        typedef uint16_t __attribute__((address_space(3))) * lds_u16_ptr;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_u16_ptr)lds; // LDS byte address of the ring
        // this wave's share of an operand stage
        const uint32_t wdstx = lds0 + (uint32_t)wave * 4096u;
        const uint32_t wdsty = lds0 + G::OPX * 2 + (uint32_t)wave * (NYL * 1024u);
        // Loads of tiles beyond the K range are not skipped (the loop stays free of branches and
        // every wait sees the same number of younger loads): they re-read the last tile and land in
        // four spare KiB per wave behind the ring.
        const uint32_t wspare = lds0 + G::SPARE + (uint32_t)wave * 4096u;
        // table form: this wave's ring of k-table slots (64 entries: 32 of X, 32 of Y)
        const uint32_t     wtab = lds0 + G::KTAB + (uint32_t)wave * 1024u;
        const lds_u32_cptr tab0 = (lds_u32_cptr)((lds_u16_ptr)lds + G::KTAB / 2 + wave * 512);

        HdLoader<XKF, BP, KAFF> gx;
        HdLoader<YKF, BQ, KAFF> gy;
        gx.init(a.xp, p0, a.xk_stride, wave, lane, tab0, 0, a.x_last_vec);
        gy.init(a.yq, q0, a.yk_stride, wave, lane, tab0, 32, a.y_last_vec);
        HdFrag<XKF, BP> fx;
        HdFrag<YKF, BQ> fy;
        fx.init(wp * 128, lane);
        fy.init(wq * (BQ / 2), lane);

        // Affine form: the k origin of the next tile to be requested, per operand: a 32-bit byte offset
        // from the operand's base (offsets inside a tensor fit 31 bits of elements), kept in scalar
        // registers.  Tiles beyond the last one of the slice re-read the last one.
        const uint32_t xkb   = 2u * (uint32_t)a.xk_stride;
        const uint32_t ykb   = 2u * (uint32_t)a.yk_stride;
        int            xko = k00, yko = k00;
        // source of the next X / Y tile to be requested, its index, and where it goes
        const char* xsrc = (const char*)a.X + (KAFF ? (uint64_t)((uint32_t)k00 * xkb) : 0ull);
        const char* ysrc = (const char*)a.Y + (KAFF ? (uint64_t)((uint32_t)k00 * ykb) : 0ull);
        int         xu = 0, yu = 0;
        uint32_t    xdst = wdstx, ydst = wdsty;
        // after the loads of a tile have been issued: move on to the next tile; S = its ring stage
        auto x_next = [&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            xu++;
            if constexpr(KAFF)
            {
                xko  = hd_next_origin(xko, klast);
                xsrc = (const char*)a.X + (uint64_t)((uint32_t)xko * xkb);
            }
            xdst = xu < n_load ? wdstx + S * (G::STAGE * 2) : wspare;
        };
        auto y_next = [&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            yu++;
            if constexpr(KAFF)
            {
                yko  = hd_next_origin(yko, klast);
                ysrc = (const char*)a.Y + (uint64_t)((uint32_t)yko * ykb);
            }
            ydst = yu < n_load ? wdsty + S * (G::STAGE * 2) : wspare;
        };

        // Table form: lane L < 32 fetches xk[k + L], lane L >= 32 yk[k + L - 32], k the tile's origin;
        // both tables lie in one device allocation, so they are addressed from the lower of the two.
        const char* tsrc  = nullptr;
        uint32_t    tvoff = 0;
        int         tk    = kt_begin * BK; // origin of the next tile whose entries are requested (before clamping)
        if constexpr(!KAFF)
        {
            const char* const tx = (const char*)a.xk;
            const char* const ty = (const char*)a.yk;
            const char* const tb = tx < ty ? tx : ty;
            tvoff                = (uint32_t)((lane < 32 ? tx : ty) - tb) + 4u * (uint32_t)(lane & 31);
            tsrc                 = tb;
        }
        auto t_src = [&]() -> const char* {
            const int kc = tk < kmax ? tk : kmax;
            tk += BK;
            return tsrc + 4ull * (uint64_t)(uint32_t)kc;
        };

        f32x16_t acc[TP][TQ];
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int j = 0; j < TQ; j++)
#pragma unroll
                for(int r = 0; r < 16; r++)
                    acc[i][j][r] = 0.f;

        u32x4_t  xf[2][TP], yf[2][TQ];
        uint32_t xe[4], ye[NYL]; // table entries on their way from LDS to the offsets

        // One k-substep: NM MFMAs out of register set `slot`; the TP + TQ operand fetches `(nstage, nks)`
        // into the other set spread over its first MFMAs in the order the next substep needs them
        // (x0 y0 .. x1 ..); and the direct loads of X (ISX) or Y in the MFMA slots of this wave, each
        // with its M0 write one MFMA earlier.  Table form: the Y substep starts with the load of the
        // table entries of the tile seven ahead (into table slot TS), and each substep ends with the
        // offsets of the other operand's next tile (entries in table slot S).
        // sched_barrier(0) after every MFMA keeps the issue order as written.
        auto substep = [&](auto wv_c, auto slot_c, const uint16_t* nstage, auto nks_c, auto isx_c, auto s_c) {
            constexpr int  WV   = decltype(wv_c)::value;
            constexpr int  slot = decltype(slot_c)::value;
            constexpr int  nks  = decltype(nks_c)::value;
            constexpr bool ISX  = decltype(isx_c)::value;
            constexpr int  S    = decltype(s_c)::value;
            constexpr int  NL   = ISX ? 4 : NYL;
            constexpr int  SP   = NL * 4 <= NM ? 4 : NM / 4; // MFMA slots from one load of this wave to its next
            constexpr int  LS   = WV % SP; // slot of this wave's loads within each group
#pragma unroll
            for(int m = 0; m < NM; m++)
            {
                // fetch f goes before MFMA f
#pragma unroll
                for(int f = 0; f < TP + TQ; f++)
                    if(f == m)
                    {
                        if(f == 0)
                            xf[slot ^ 1][0] = fx.load(nstage, 0, nks);
                        else if(f <= TQ)
                            yf[slot ^ 1][f - 1] = fy.load(nstage + G::OPX, f - 1, nks);
                        else
                            xf[slot ^ 1][f - TQ] = fx.load(nstage, f - TQ, nks);
                    }
                if constexpr(!KAFF && !ISX)
                    if(m == 0)
                    {
                        dma_dst<((S + 3) & 3) * 256>(wtab);
                        dma_load1(tvoff, t_src());
                    }
                // M0 for the load that follows the next MFMA
                if((m % SP) == ((LS + SP - 1) % SP) && (LS != 0 || m != NM - 1))
                {
                    const int i = LS == 0 ? (m + 1) / SP : m / SP;
                    if(i == 0) dma_dst<0>(ISX ? xdst : ydst);
                    if(i == 1) dma_dst<1024>(ISX ? xdst : ydst);
                    if(i == 2) dma_dst<2048>(ISX ? xdst : ydst);
                    if(i == 3 && NL > 3) dma_dst<3072>(ISX ? xdst : ydst);
                }
                if(LS == 0 && m == 0)
                {
                    // (first slot of the substep: no earlier MFMA in it)
                    dma_dst<0>(ISX ? xdst : ydst);
                }
                if((m % SP) == LS && m / SP < NL)
                    dma_load(ISX ? gx.voff[m / SP] : gy.voff[m / SP], ISX ? xsrc : ysrc);
                if constexpr(!KAFF)
                {
                    // (the loads of this substep's operand are behind; the other operand's are in the
                    // substep that follows)
                    if(m == NM - 4)
                    {
                        if constexpr(ISX)
                            gy.template read_entries<S>(ye);
                        else
                            gx.template read_entries<S>(xe);
                    }
                    if(m == NM - 1)
                    {
                        if constexpr(ISX)
                            gy.set_offsets(ye, gy.voff);
                        else
                            gx.set_offsets(xe, gx.voff);
                    }
                }
                acc[m / TQ][m % TQ] = Tr::mfma(xf[slot][m / TQ], yf[slot][m % TQ], acc[m / TQ][m % TQ]);
                // (an MFMA has no side effect, so instruction selection may place it anywhere between its
                // operands and the first use of its result, before the scheduler ever sees the barrier
                // below: an empty ordered statement that reads the result keeps it here)
                asm volatile("" : : "a"(acc[m / TQ][m % TQ]));
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        typedef std::integral_constant<int, 2> I2;
        typedef std::integral_constant<int, 3> I3;

        // K tile t, whose ring stage is S = t % 4
        auto tile_step = [&](auto wv_c, auto s_c) {
            constexpr int   S   = decltype(s_c)::value;
            const uint16_t* cur = lds + S * G::STAGE;
            const uint16_t* nxt = lds + ((S + 1) & (NS - 1)) * G::STAGE;
            // substep 0: multiply k 0..15 of tile t, fetch k 16..31; the Y loads of tile t + 3
            // (table form: and the offsets of X of tile t + 4, whose entries are in table slot S)
            substep(wv_c, I0{}, cur, I1{}, std::false_type{}, s_c);
            y_next(s_c); // tile t + 4 shares tile t's stage
            // Every wave has issued its reads of tile t.  Tile t + 1 must have landed.
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(NWAIT));
            lds_barrier();
            __builtin_amdgcn_sched_barrier(0);
            // substep 1: multiply k 16..31 of tile t, fetch k 0..15 of tile t + 1 (beyond the last
            // tile: stale data, not used); the X loads of tile t + 4 go into the stage tile t has
            // just left (table form: and the offsets of Y of tile t + 4)
            substep(wv_c, I1{}, nxt, I0{}, std::true_type{}, s_c);
            x_next(std::integral_constant<int, (S + 1) & (NS - 1)>{}); // tile t + 5
        };

        auto main_loop = [&](auto wv_c) {
            // Table form: the entries of tiles 0..3 and the offsets of their loads; the entries of
            // tiles 4..6 are requested between the operand loads below, in the order the loop keeps.
            uint32_t pxv[KAFF ? 1 : NS][4], pyv[KAFF ? 1 : NS][NYL];
            if constexpr(!KAFF)
            {
#pragma unroll
                for(int u = 0; u < NS; u++)
                {
                    dma_dst_at(wtab, u * 256);
                    dma_load1(tvoff, t_src());
                }
                __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
#pragma unroll
                for(int u = 0; u < NS; u++)
                {
                    if(u == 0) { gx.template read_entries<0>(xe); gy.template read_entries<0>(ye); }
                    if(u == 1) { gx.template read_entries<1>(xe); gy.template read_entries<1>(ye); }
                    if(u == 2) { gx.template read_entries<2>(xe); gy.template read_entries<2>(ye); }
                    if(u == 3) { gx.template read_entries<3>(xe); gy.template read_entries<3>(ye); }
                    gx.set_offsets(xe, pxv[u]);
                    gy.set_offsets(ye, pyv[u]);
                }
                __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0); // the slots have been read
            }
            // prologue: tiles 0, 1, 2 and the X half of tile 3
#pragma unroll
            for(int t = 0; t < NS; t++)
            {
#pragma unroll
                for(int i = 0; i < 4; i++)
                {
                    dma_dst_at(xdst, i * 1024);
                    dma_load(KAFF ? gx.voff[i] : pxv[KAFF ? 0 : t][i], xsrc);
                }
                if(t == 0) x_next(I1{});
                if(t == 1) x_next(I2{});
                if(t == 2) x_next(I3{});
                if(t == 3) x_next(I0{});
                if(t < NS - 1)
                {
                    if constexpr(!KAFF)
                    {
                        // entries of tile 4 + t, in the place the loop gives them: in front of a tile's Y loads
                        dma_dst_at(wtab, t * 256);
                        dma_load1(tvoff, t_src());
                    }
#pragma unroll
                    for(int i = 0; i < NYL; i++)
                    {
                        dma_dst_at(ydst, i * 1024);
                        dma_load(KAFF ? gy.voff[i] : pyv[KAFF ? 0 : t][i], ysrc);
                    }
                    if(t == 0) y_next(I1{});
                    if(t == 1) y_next(I2{});
                    if(t == 2) y_next(I3{});
                }
            }
            if constexpr(!KAFF)
            {
#pragma unroll
                for(int i = 0; i < NYL; i++)
                    gy.voff[i] = pyv[KAFF ? 0 : NS - 1][i]; // tile 3's, issued in the first step
            }
            // tile 0 has landed (and the X loads of tile 1)
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(8 + 2 * NYL));
            lds_barrier();
#pragma unroll
            for(int i = 0; i < TP; i++)
                xf[0][i] = fx.load(lds, i, 0);
#pragma unroll
            for(int j = 0; j < TQ; j++)
                yf[0][j] = fy.load(lds + G::OPX, j, 0);
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
            if(half)
            {
                // the tail: tile nt was loaded from K - 32, its k 16..31 are the last 16 of K
                const uint16_t* st = lds + (nt & (NS - 1)) * G::STAGE;
#pragma unroll
                for(int i = 0; i < TP; i++)
                    xf[0][i] = fx.load(st, i, 1);
#pragma unroll
                for(int j = 0; j < TQ; j++)
                    yf[0][j] = fy.load(st + G::OPX, j, 1);
#pragma unroll
                for(int m = 0; m < NM; m++)
                    acc[m / TQ][m % TQ] = Tr::mfma(xf[0][m / TQ], yf[0][m % TQ], acc[m / TQ][m % TQ]);
            }
        };

        // One copy of the loop per wave position (the loop bodies differ in where the direct loads sit);
        // the epilogue is shared: the accumulators keep their registers through every copy of the loop
        // (an MFMA's result is tied to its addend), so the copies join without a move, and four waves
        // that run one copy of the epilogue fetch a quarter of the instructions (4096^3: 114.1 -> 112.1 us).
        auto run = [&](auto wv_c) {
            if(n_load > 0)
                main_loop(wv_c);
        };
        switch(wave)
        {
        case 0: run(I0{}); break;
        case 1: run(I1{}); break;
        case 2: run(I2{}); break;
        default: run(I3{}); break;
        }
        // the epilogue stages through LDS: every wave must be done reading operands
        lds_barrier();
        // (accumulators pinned in AGPRs: without it the compiler moved them to VGPRs and spilled)
#pragma unroll
        for(int i = 0; i < TP; i++)
#pragma unroll
            for(int j = 0; j < TQ; j++)
                asm volatile("" : "+a"(acc[i][j]));
        epilogue_h<Tr, WP, WQ, TP, TQ, G::EPI, true>(a, acc, lds, p0, q0, p_own, q_own);
        // the loads beyond the K range (into the spare KiB, and of table entries) must not outlive
        // the workgroup's LDS
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    }

    template <typename Tr, bool XKF, bool YKF, int BQ, bool KAFF>
    int launch_hd(const KArgs& a, hipStream_t stream)
    {
        typedef HdGeom<BQ, KAFF> G;
        if(a.K < G::BK || a.K % 16 != 0)
            return (int)hipErrorInvalidValue;
        if constexpr(!KAFF)
        {
            // the two k tables are addressed with 32-bit offsets from the lower one
            const uintptr_t tx = (uintptr_t)a.xk, ty = (uintptr_t)a.yk;
            if((tx < ty ? ty - tx : tx - ty) >= (1ull << 31))
                return (int)hipErrorInvalidValue;
        }
        auto                    kern = contract_hd_kernel<Tr, XKF, YKF, BQ, KAFF>;
        static const hipError_t attr = hipFuncSetAttribute(
            (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if(attr != hipSuccess)
            return (int)attr;
        dim3 grid(a.tiles_p * a.tiles_q, 1, a.split_k);
        hipLaunchKernelGGL(kern, grid, dim3(256), G::LDS_BYTES, stream, a);
        return (int)hipGetLastError();
    }
}

// Registry lines of the direct-load kernels: K a multiple of 16, at least 32.  (The table form is
// instantiated for the 256 x 192 tile only: beside 256 accumulator registers the 256 x 256 tile has
// no room for the table offsets, and spills in its main loop.)
#define HIPTK_HD_ENTRY(TR, ID, BQ, XKF, YKF, KAFF)                                                \
    {                                                                                             \
        TR::CLS, ID, XKF, YKF, 8, 8, KAFF, 256, BQ, 32, 256, hiptk::HdGeom<BQ, KAFF>::LDS_BYTES,  \
            #TR "_256x" #BQ "x32_x" #XKF "8_y" #YKF "8_kaff" #KAFF "_direct2x2",                  \
            &hiptk::launch_hd<hiptk::TR, XKF, YKF, BQ, KAFF>, 16                                  \
    }
#define HIPTK_HD_TILE(TR, ID, BQ, KAFF)                                                            \
    HIPTK_HD_ENTRY(TR, ID, BQ, true, true, KAFF), HIPTK_HD_ENTRY(TR, ID, BQ, true, false, KAFF),   \
        HIPTK_HD_ENTRY(TR, ID, BQ, false, true, KAFF), HIPTK_HD_ENTRY(TR, ID, BQ, false, false, KAFF)
