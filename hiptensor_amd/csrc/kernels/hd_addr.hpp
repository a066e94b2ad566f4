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

    // ---- 16-bit kernel for operands that are both contiguous along k (contract_hk.hpp): K tiles of 64 ----
    // A stage is stage[row][64 k]: 128-byte rows, so that a direct load fetches whole 128-byte lines
    // (8 rows per KiB).  The 16-byte slot s holds the 8 k from `k` on of row `row`; the XOR puts the
    // 16 rows that 16 consecutive lanes of a ds_read_b128 touch into 16 disjoint bank ranges.
    constexpr int HK_BK = 64;

    // position (0 .. 7) in its row's 128 bytes of the 16-byte chunk that holds k = 8 * chunk .. + 7
    HIPTK_HD_FN int hk_chunk_pos(int row, int chunk)
    {
        return chunk ^ ((row >> 1) & 7);
    }

    template <int BR>
    HIPTK_HD_FN HdSlot hk_slot(int s)
    {
        HdSlot o;
        o.row = s >> 3;
        o.k   = 8 * hk_chunk_pos(o.row, s & 7); // (the XOR is its own inverse)
        return o;
    }

    // ... and for either kind of operand: a k-contiguous one as above, a row-contiguous one as
    // stage[k][BR] (64 k-rows), whose slot s holds the 8 rows from `row` on at `k`
    template <bool KF, int BR>
    HIPTK_HD_FN HdSlot hk_stage_slot(int s)
    {
        if(KF)
            return hk_slot<BR>(s);
        HdSlot        o;
        constexpr int cpr = BR / 8;
        o.k               = s / cpr;
        o.row             = 8 * ((s % cpr) ^ (2 * (o.k & 3)));
        return o;
    }

    // The K tiles one workgroup reduces: nt whole tiles of 64, then, when the slice ends at K and K is
    // not a multiple of 64, a tail tile of `tail` k-steps of 16: it is loaded whole from K - 64 (so
    // that no address leaves the tensor) and only its last `tail` k-steps are multiplied.  Tiles
    // requested beyond the last one repeat it.
    struct HkSlice
    {
        int nt, tail, n_load, kmax, k00, klast;
    };

    HIPTK_HD_FN HkSlice hk_slice(int K, int kt_begin, int ktiles_per_split)
    {
        HkSlice   s;
        const int kt_whole = K / HK_BK;
        const int kt_stop  = kt_begin + ktiles_per_split;
        s.nt               = (kt_stop < kt_whole ? kt_stop : kt_whole) - kt_begin;
        s.tail             = ((K % HK_BK) != 0 && kt_stop > kt_whole) ? (K % HK_BK) / 16 : 0;
        s.n_load           = s.nt + (s.tail ? 1 : 0);
        s.kmax             = K - HK_BK;
        s.k00              = kt_begin * HK_BK < s.kmax ? kt_begin * HK_BK : s.kmax;
        s.klast            = s.tail ? s.kmax : (kt_begin + s.nt - 1) * HK_BK;
        return s;
    }

    HIPTK_HD_FN int hk_next_origin(int ko, int klast)
    {
        return ko + HK_BK < klast ? ko + HK_BK : klast;
    }

    // The MFMA slot (0 .. 63, counted from the k-step in which a ring stage has become free) in front of
    // which wave `wave` issues its j-th direct load of the K tile that goes into that stage: one load
    // every `spacing` MFMAs, the waves staggered so that the texture path sees them one at a time.
    HIPTK_HD_FN constexpr int hk_load_slot(int wave, int j, int spacing)
    {
        return j * spacing + wave % spacing;
    }

    // position in its k-row of stage[k][rows] (row-contiguous operand) of the element of row `row`: the
    // 8-row chunks of a k-row are exchanged by c -> c ^ 2 (k % 4)
    HIPTK_HD_FN int hd_row_pos(int row, int k)
    {
        return (((row >> 3) ^ (2 * (k & 3))) << 3) | (row & 7);
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
    // A k-contiguous operand whose runs along k are one vector long has its neighbouring vectors elsewhere: where
    // those of consecutive rows follow one another in memory, the ring kernel (contract_hr.hpp) lays the stage out
    // chunk-major, stage[4 chunks of 8 k][rows][8]: a direct load's 64 lanes then cover 64 consecutive rows of one
    // chunk (4 lanes = 64 contiguous bytes, one access of the vector cache) instead of 16 rows x 4 chunks (4 lanes =
    // 4 places), and the MFMA operand read (16 lanes = 16 consecutive rows of one chunk = 256 contiguous bytes)
    // needs no swizzle.  `chunked` is that choice; it is a matter of speed only.
    template <bool KF, int BR>
    HIPTK_HD_FN HdSlot hr_slot(int s, bool chunked)
    {
        if(KF && chunked)
        {
            HdSlot o;
            o.row = s % BR;
            o.k   = 8 * (s / BR);
            return o;
        }
        return hd_slot<KF, BR>(s);
    }
    // element position in a k-contiguous operand's stage of the 8 k from 8 * chunk on of row `row`
    template <int BR>
    HIPTK_HD_FN int hr_chunk_elem(int row, int chunk, bool chunked)
    {
        return chunked ? (chunk * BR + row) * 8 : row * HD_BK + ((chunk ^ ((row >> 2) & 3)) << 3);
    }
}
