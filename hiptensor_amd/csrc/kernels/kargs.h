// Device-side argument block shared by every contraction kernel, and the launcher
// signature each kernel family exports to the dispatcher.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hiptk_kernels.h"

namespace hiptk
{
    struct KArgs
    {
        const void* X; // rows operand   (MFMA "A": register-varying output index p)
        const void* Y; // columns operand (MFMA "B": lane-varying output index q)
        const void* C;
        void*       D;
        void*       ws; // split-K partials, [split][P][Q] accumulator-typed
        const int32_t *xp, *xk, *yq, *yk, *cp, *cq, *dp, *dq;
        int32_t P, Q, K;
        int32_t ktiles_per_split; // K tiles (of BK) each z-slice reduces
        int32_t split_k;
        int32_t bilinear;
        int32_t tiles_p, tiles_q;
        int32_t xk_stride, yk_stride; // element stride of k when the K modes fused into one
        int32_t cd_affine; // 1: C / D offsets are p * stride + q * stride, no table lookups
        int32_t dp_stride, dq_stride, cp_stride, cq_stride;
        int32_t xp_stride, yq_stride; // with cd_affine: xp[p] = p * xp_stride, yq[q] = q * yq_stride (0: look them up)
        int32_t cd_vec; // contiguous elements along q shared by C and D
        // 1: a tile that would overhang P (Q) is moved back so that it ends at P (Q); it still
        // stores only the rows (columns) of its own range.  Lets vectors run along a contiguous
        // row (column) index whose extent is not a multiple of the vector.
        int32_t shift_p, shift_q;
        // byte offset of the last 16-byte vector of X / Y that the tables address (direct-load kernels, table form)
        uint32_t x_last_vec, y_last_vec;
        // 1: a k-contiguous X / Y is staged chunk-major by the kernels that can (the vectors of consecutive rows are
        // neighbours in memory; those of consecutive k are not)
        int32_t x_chunked, y_chunked;
        double   alpha[2], beta[2];
    };

    // Tile-level launcher: returns hipError_t as int.
    typedef int (*launch_fn)(const KArgs&, hipStream_t);

    struct KernelEntry
    {
        int32_t     cls, tile_id;
        int32_t     x_kfast, y_kfast, x_vec, y_vec;
        int32_t     k_affine; // 1: k offsets are k * stride, no table lookups
        int32_t     bp, bq, bk, threads, lds_bytes;
        const char* name;
        launch_fn   launch;
        int32_t     k_multiple; // 0: any K; else K must be a multiple of this and at least bk
        int32_t     mfma_k; // reduction depth of the MFMA instruction the tile is built on, where the selection tells tiles apart by it (else 0)
    };

    // Each kernel translation unit contributes its table.
    const KernelEntry* entries_f16_vec(int* count);
    const KernelEntry* entries_f16_aff(int* count);
    const KernelEntry* entries_bf16_aff(int* count);
    const KernelEntry* entries_f16_gen(int* count);
    const KernelEntry* entries_bf16_vec(int* count);
    const KernelEntry* entries_bf16_gen(int* count);
    const KernelEntry* entries_f16_hd(int* count);
    const KernelEntry* entries_f16_hd192(int* count);
    const KernelEntry* entries_f16_hd192_tab(int* count);
    const KernelEntry* entries_bf16_hd(int* count);
    const KernelEntry* entries_bf16_hd192(int* count);
    const KernelEntry* entries_bf16_hd192_tab(int* count);
    const KernelEntry* entries_f16_hk_kx(int* count);
    const KernelEntry* entries_f16_hk_rx(int* count);
    const KernelEntry* entries_bf16_hk_kx(int* count);
    const KernelEntry* entries_bf16_hk_rx(int* count);
    const KernelEntry* entries_f16_hr192_kx(int* count);
    const KernelEntry* entries_f16_hr192_rx(int* count);
    const KernelEntry* entries_bf16_hr192_kx(int* count);
    const KernelEntry* entries_bf16_hr192_rx(int* count);
    const KernelEntry* entries_f16_v4(int* count);
    const KernelEntry* entries_f16_v2(int* count);
    const KernelEntry* entries_bf16_v4(int* count);
    const KernelEntry* entries_bf16_v2(int* count);
    const KernelEntry* entries_f32(int* count);
    const KernelEntry* entries_f64(int* count);
    const KernelEntry* entries_c32(int* count);
    const KernelEntry* entries_c64(int* count);
    const KernelEntry* entries_f64_as_f32(int* count);
    const KernelEntry* entries_f32_as_f16(int* count);
    const KernelEntry* entries_f32_as_bf16(int* count);

    // XCD-aware mapping of the linear workgroup id to an output tile.  Workgroups are
    // handed to the 8 XCDs round-robin, so ids that are congruent mod 8 share an L2.
    // Give each XCD a contiguous band of the tile space and walk that band in
    // column-groups of GROUP rows so that the X rows / Y columns a band touches
    // stay resident in that XCD's L2.
    __device__ inline void tile_coords(int wg, int tiles_p, int tiles_q, int& tp, int& tq)
    {
        // XCD x runs the workgroups wg = x, x + 8, ...: base = total / 8 of them, one more for the
        // first total % 8 XCDs; give it the contiguous range of tiles that starts after its
        // predecessors' shares
        const int total = tiles_p * tiles_q;
        const int xcd = wg & 7, nth = wg >> 3;
        const int base = total >> 3, rem = total & 7;
        const int lin  = xcd * base + (xcd < rem ? xcd : rem) + nth;
        constexpr int GROUP = 4;
        const int     band  = GROUP * tiles_q;
        const int     g     = lin / band;
        const int     first = g * GROUP;
        const int     rows  = (tiles_p - first) < GROUP ? (tiles_p - first) : GROUP;
        const int     r     = lin - g * band;
        tp                  = first + r % rows;
        tq                  = r / rows;
    }
}
