// Address arithmetic of the kernels that load their operand tiles straight into LDS
// (contract_hd.hpp), in functions that also compile for the host: a direct load has no bounds
// check and no mask, so which element every lane requests is checked exhaustively on the CPU
// (tests/cpp/hd_bounds.cpp) with the planner's own tables.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define HIPTK_HD_FN __host__ __device__ inline
#else
#define HIPTK_HD_FN inline
#endif

namespace hiptk
{
    constexpr int HD_BK = 32; // K tile of the direct-load kernels

    // The K tiles one workgroup reduces (split-K slice z = kt_begin / ktiles_per_split):
    // nt whole tiles of 32, then the 16-element tail when the slice ends at K (K % 32 == 16).
    // A tile is loaded whole; the tail tile is loaded from K - 32 (so that no address leaves the
    // tensor) and only its second half is multiplied.  Tiles requested beyond the last one repeat it.
    struct HdSlice
    {
        int nt; // whole tiles
        int half; // 1: a tail tile follows them
        int n_load; // tiles whose loads go to the ring (the others land in spare LDS)
        int kmax; // K - 32: the last origin a tile may have
        int k00; // origin of the slice's first tile
        int klast; // origin of its last tile
    };

    HIPTK_HD_FN HdSlice hd_slice(int K, int kt_begin, int ktiles_per_split)
    {
        HdSlice   s;
        const int kt_whole = K / HD_BK;
        const int kt_stop  = kt_begin + ktiles_per_split;
        s.nt               = (kt_stop < kt_whole ? kt_stop : kt_whole) - kt_begin;
        s.half             = ((K % HD_BK) != 0 && kt_stop > kt_whole) ? 1 : 0;
        s.n_load           = s.nt + s.half;
        s.kmax             = K - HD_BK;
        s.k00              = kt_begin * HD_BK < s.kmax ? kt_begin * HD_BK : s.kmax;
        s.klast            = s.half ? s.kmax : (kt_begin + s.nt - 1) * HD_BK;
        return s;
    }

    // origin of the tile requested after the one at ko
    HIPTK_HD_FN int hd_next_origin(int ko, int klast)
    {
        return ko + HD_BK < klast ? ko + HD_BK : klast;
    }

    // What the 16-byte slot s of an operand stage holds (a direct load fills slot 64 * j + lane
    // with lane's 16 bytes, j = which KiB of the stage): 8 consecutive elements starting at
    // (row, k) of the tile, along k for a k-contiguous operand (KF), along the row index otherwise.
    // The XOR is the bank swizzle the operand reads undo.
    struct HdSlot
    {
        int row, k;
    };

    // The 32/64-bit direct-load kernels (contract_wd.hpp): K tiles of bk, no tail (K is a multiple of
    // bk); tiles requested beyond the slice's last one repeat it.
    HIPTK_HD_FN int wd_next_origin(int ko, int klast, int bk)
    {
        return ko + bk < klast ? ko + bk : klast;
    }

    // ... their operand stages are tile[k][ROWS rows] of elements of 16 / V bytes, unpadded and
    // unswizzled (one element per lane and MFMA operand: consecutive lanes read consecutive rows):
    // the 16-byte slot s holds the V rows from `row` on at `k`.
    template <int V, int ROWS>
    HIPTK_HD_FN HdSlot wd_slot(int s)
    {
        HdSlot        o;
        constexpr int cpr = ROWS / V;
        o.k               = s / cpr;
        o.row             = V * (s % cpr);
        return o;
    }

    // The same kernels for operands that are contiguous along k: a 16-byte vector is V consecutive k of
    // one row, and a stage is tile[k / V][ROWS rows][V]: slot s holds row `row` from k on.  A lane of the
    // MFMA's k-slot j then reads one vector for V k-steps: the k-slots of a k-step are V apart in k instead
    // of adjacent, for both operands alike.
    template <int V, int ROWS>
    HIPTK_HD_FN HdSlot wd_slot_kf(int s)
    {
        HdSlot o;
        o.k   = V * (s / ROWS);
        o.row = s % ROWS;
        return o;
    }

    // A last K tile that holds only tail_k (< BK) k: does the vector at k-position `k` of the tile (V
    // consecutive k of a row if kf, else V rows at that k) lie inside K?  The others are loaded from 16
    // bytes of zeros instead, so the tile multiplies as a whole one.
    HIPTK_HD_FN bool wd_tail_inside(bool kf, int k, int v, int tail_k)
    {
        return kf ? k + v <= tail_k : k < tail_k;
    }

    // ... and where the four waves of a workgroup split a slice of n K tiles between them: wave w takes
    // `count` tiles from `first` on (none, for the last waves of a short slice).
    struct WdChunk
    {
        int first, count;
    };
    HIPTK_HD_FN WdChunk wd_wave_chunk(int n, int w)
    {
        const int per = (n + 3) / 4;
        WdChunk   c;
        c.first = w * per < n ? w * per : n;
        c.count = n - c.first < per ? n - c.first : per;
        return c;
    }

    template <bool KF, int BR>
    HIPTK_HD_FN HdSlot hd_slot(int s)
    {
        HdSlot o;
        if(KF)
        {
            // stage[row][32]: 4 chunks of 8 k per row
            o.row = s >> 2;
            o.k   = 8 * ((s & 3) ^ ((o.row >> 2) & 3));
        }
        else
        {
            // stage[k][BR]: BR / 8 chunks of 8 rows per k
            const int cpr = BR / 8;
            o.k           = s / cpr;
            o.row         = 8 * ((s % cpr) ^ (2 * (o.k & 3)));
        }
        return o;
    }
}
