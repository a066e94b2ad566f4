// Host-side check of the direct-load contraction kernels' addressing (kernels/hd_addr.hpp, the
// functions the kernels themselves call): a direct load has no bounds check and no mask, so for a
// list of problems planned by the library's own planner this program walks every 16-byte request
// of every lane, K tile, split-K slice and (sampled) output tile and checks that it
//   * reads table entries inside the padded tables,
//   * starts a multiple of 16 bytes from the tensor's base and ends inside the tensor's span,
//   * covers 8 elements that are contiguous in memory (the planner's vector promise),
// that the 16-byte slots of a stage tile it exactly once, that a k-contiguous operand's chunk is
// the same for all of a lane's loads (the table form reads one entry per lane for them), and that
// the K tiles of all slices multiply every k exactly once.  The same for the 32/64-bit direct-load
// kernels (64 x 64 tile, vectors of 16 / sizeof(element) rows, byte offsets that must fit 32 bits).
// Exit code 0 and "ok" on success.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "../../hiptensor_amd/csrc/host/planner.hpp"
#include "../../hiptensor_amd/csrc/kernels/hd_addr.hpp"
#include "../../include/hiptk_kernels.h"

using namespace hipta;
using hiptk::hd_next_origin;
using hiptk::hd_slice;
using hiptk::hd_slot;
using hiptk::HdSlice;
using hiptk::HdSlot;
using hiptk::hk_chunk_pos;
using hiptk::hk_next_origin;
using hiptk::hk_slice;
using hiptk::hd_row_pos;
using hiptk::hk_stage_slot;
using hiptk::hr_chunk_elem;
using hiptk::hr_slot;
using hiptk::HkSlice;
using hiptk::wd_next_origin;
using hiptk::wd_slot;
using hiptk::wd_slot_kf;
using hiptk::wd_tail_inside;
using hiptk::wd_wave_chunk;
using hiptk::WdChunk;

static int g_fail = 0;
#define CHECK(cond, ...)                                                  \
    do                                                                    \
    {                                                                     \
        if(!(cond))                                                       \
        {                                                                 \
            if(g_fail < 20)                                               \
            {                                                             \
                std::printf("FAIL %s:%d %s: ", __FILE__, __LINE__, #cond); \
                std::printf(__VA_ARGS__);                                 \
                std::printf("\n");                                        \
            }                                                             \
            g_fail++;                                                     \
        }                                                                 \
    } while(0)

struct Case
{
    std::string                              name;
    std::vector<int32_t>                     mA, mB, mD; // modes as listed
    std::vector<std::pair<int32_t, int64_t>> ext;
    std::vector<int32_t>                     oA, oB, oD; // storage order, fastest first (empty: as listed)
    int64_t                                  padD = 0; // elements added after D's fastest mode
    bool                                     bilinear = false;
};

static int64_t extent(const Case& c, int32_t m)
{
    for(auto& e : c.ext)
        if(e.first == m)
            return e.second;
    return 0;
}

static int g_dtype = 2; // HIP_R_16F

static TensorIn tensor(const Case& c, const std::vector<int32_t>& modes, std::vector<int32_t> order, int64_t pad)
{
    if(order.empty())
        order = modes;
    TensorIn t;
    t.dtype = g_dtype;
    t.mode  = modes;
    t.len.resize(modes.size());
    t.stride.resize(modes.size());
    int64_t s = 1;
    for(size_t i = 0; i < order.size(); i++)
    {
        const size_t at = std::find(modes.begin(), modes.end(), order[i]) - modes.begin();
        t.len[at]       = extent(c, order[i]);
        t.stride[at]    = s;
        s *= t.len[at];
        if(i == 0)
            s += pad;
    }
    t.align = 256;
    return t;
}

// The kernels compute their operands' row offsets where the planner says the rows of X and the columns of Y are one mode
// each: what they compute must be what the tables hold.
static int check_computed_rows(const Case& c, const GemmView& v)
{
    if(!v.cd_affine)
        return 0;
    if(v.xp_stride)
        for(int64_t r = 0; r < v.P; r++)
            CHECK(v.xp[(size_t)r] == r * v.xp_stride, "%s xp[%lld] is not %lld x the row stride", c.name.c_str(), (long long)r, (long long)r);
    if(v.yq_stride)
        for(int64_t r = 0; r < v.Q; r++)
            CHECK(v.yq[(size_t)r] == r * v.yq_stride, "%s yq[%lld] is not %lld x the column stride", c.name.c_str(), (long long)r, (long long)r);
    return v.xp_stride && v.yq_stride;
}

template <bool KF, int BR>
static void check_operand(const char* what, const Case& c, const GemmView& v, bool is_x, int r0, const std::vector<int>& origins,
                          bool affine, bool ring = false) // ring: the kernel on 16 x 16 x 32 MFMAs (contract_hr.hpp), table form only
{
    const bool chunked = ring && KF && (is_x ? v.x_rows_adjacent : v.y_rows_adjacent) != 0;
    const std::vector<int32_t>& rtab    = is_x ? v.xp : v.yq;
    const std::vector<int32_t>& ktab    = is_x ? v.xk : v.yk;
    const int64_t               kstride = is_x ? v.xk_stride : v.yk_stride;
    const int64_t               nrows   = is_x ? v.P : v.Q;
    const int64_t               span    = (is_x != v.swapped) ? v.spanA : v.spanB;
    std::vector<int>            seen(BR * 32 / 8, 0);
    constexpr int               NL = BR / 64;
    for(int wave = 0; wave < 4; wave++)
        for(int lane = 0; lane < 64; lane++)
        {
            int k_first = -1;
            for(int i = 0; i < NL; i++)
            {
                const int    s  = (wave * NL + i) * 64 + lane;
                const HdSlot sl = ring ? hr_slot<KF, BR>(s, chunked) : hd_slot<KF, BR>(s);
                CHECK(sl.row >= 0 && sl.row + (KF ? 1 : 8) <= BR && sl.k >= 0 && sl.k + (KF ? 8 : 1) <= 32, "%s %s slot %d -> row %d k %d",
                      c.name.c_str(), what, s, sl.row, sl.k);
                seen[KF ? sl.row * 4 + sl.k / 8 : sl.k * (BR / 8) + sl.row / 8]++;
                if(ring) // the LDS elements 8 s .. 8 s + 7 are where the operand reads look for this vector
                    CHECK(8 * s == (KF ? hr_chunk_elem<BR>(sl.row, sl.k / 8, chunked) : sl.k * BR + hd_row_pos(sl.row, sl.k)),
                          "%s %s slot %d is not where the readers look", c.name.c_str(), what, s);
                if(KF && !ring)
                {
                    CHECK(k_first < 0 || k_first == sl.k, "%s %s lane %d: chunk differs between its loads", c.name.c_str(), what, lane);
                    k_first = sl.k;
                }
                CHECK((size_t)(r0 + sl.row) < rtab.size(), "%s %s row table index %d of %zu", c.name.c_str(), what, r0 + sl.row, rtab.size());
                const int64_t rowpart = rtab[(size_t)(r0 + sl.row)];
                for(int o : origins)
                {
                    CHECK(o >= 0 && (size_t)(o + sl.k + 7) < ktab.size(), "%s %s k table index %d", c.name.c_str(), what, o + sl.k);
                    const int64_t off = rowpart + (affine ? (int64_t)(o + sl.k) * kstride : (int64_t)ktab[(size_t)(o + sl.k)]);
                    CHECK(off >= 0 && off + 8 <= span, "%s %s r0 %d slot %d origin %d: elements %lld..+8 of %lld", c.name.c_str(), what, r0, s, o,
                          (long long)off, (long long)span);
                    // (the table form clamps every request to the last vector the tables address)
                    CHECK(off <= (is_x ? v.x_max_off : v.y_max_off) - 7, "%s %s offset %lld beyond the last vector", c.name.c_str(), what, (long long)off);
                    CHECK(off % 8 == 0, "%s %s r0 %d slot %d origin %d: offset %lld not a multiple of 8", c.name.c_str(), what, r0, s, o,
                          (long long)off);
                    // the 8 elements are the tile's (row, k .. k + 7) or (row .. row + 7, k)
                    if(KF)
                    {
                        for(int j = 1; j < 8 && o + sl.k + j < v.K; j++)
                            CHECK(ktab[(size_t)(o + sl.k + j)] - ktab[(size_t)(o + sl.k)] == j, "%s %s k run broken at %d", c.name.c_str(), what,
                                  o + sl.k);
                    }
                    else
                    {
                        for(int j = 1; j < 8 && r0 + sl.row + j < nrows; j++)
                            CHECK(rtab[(size_t)(r0 + sl.row + j)] - rowpart == j, "%s %s row run broken at %d", c.name.c_str(), what,
                                  r0 + sl.row);
                    }
                    if(affine)
                        CHECK(o + sl.k >= v.K || ktab[(size_t)(o + sl.k)] == (int64_t)(o + sl.k) * kstride, "%s %s affine k offset", c.name.c_str(), what);
                }
            }
        }
    for(size_t i = 0; i < seen.size(); i++)
        CHECK(seen[i] == 1, "%s %s chunk %zu filled %d times", c.name.c_str(), what, i, seen[i]);
    if(ring && KF)
    {
        // operand read of v_mfma_f32_16x16x32: lane l reads the 16 bytes of chunk l / 16 of row (block's first) + l % 16;
        // 16 consecutive lanes must touch 16 different 16-byte groups of the 64 banks
        for(int b = 0; b < BR / 16; b++)
            for(int g = 0; g < 4; g++)
            {
                int groups = 0;
                for(int l = 0; l < 16; l++)
                    groups |= 1 << ((hr_chunk_elem<BR>(16 * b + l, g, chunked) / 8) % 16);
                CHECK(groups == 0xFFFF, "%s %s block %d chunk %d: bank groups %x", c.name.c_str(), what, b, g, groups);
            }
    }
    if(ring && !KF)
    {
        // a transposing read: lane g of a 16-lane group points at the rows 4 (g % 4) .. + 3 of k-row g / 4: 8 contiguous bytes,
        // and the group's 16 words in 16 different 8-byte bank pairs
        for(int b = 0; b < BR / 16; b++)
            for(int grp = 0; grp < 8; grp++)
            {
                unsigned long long pairs = 0;
                for(int g = 0; g < 16; g++)
                {
                    const int k = 8 * (grp & 3) + 4 * (grp >> 2) + (g >> 2), r = 16 * b + 4 * (g & 3);
                    CHECK(hd_row_pos(r + 3, k) == hd_row_pos(r, k) + 3, "%s %s rows %d..+3 at k %d are not contiguous in LDS", c.name.c_str(), what, r, k);
                    pairs |= 1ull << (((k * BR + hd_row_pos(r, k)) / 4) % 32);
                }
                CHECK(__builtin_popcountll(pairs) == 16, "%s %s block %d group %d: transposing read touches %d bank pairs", c.name.c_str(), what, b, grp,
                      __builtin_popcountll(pairs));
            }
    }
}

template <int BQ>
static long check_tile_size(const Case& c, const GemmView& v, bool ring = false)
{
    long      walked = 0;
    const int K      = (int)v.K;
    const int tiles_p = (int)((v.P + 255) / 256), tiles_q = (int)((v.Q + BQ - 1) / BQ);
    const int ktiles  = (K + 31) / 32;
    for(int want = 1; want <= 5; want++)
    {
        int split = std::min(want, ktiles);
        int per   = (ktiles + split - 1) / split;
        split     = (ktiles + per - 1) / per;
        std::vector<int> covered((size_t)K, 0);
        std::vector<int> origins; // every origin any slice requests, affine or table form
        for(int z = 0; z < split; z++)
        {
            const HdSlice sl = hd_slice(K, z * per, per);
            CHECK(sl.nt >= 0 && sl.n_load >= 1, "%s K %d slice %d/%d: nt %d n_load %d", c.name.c_str(), K, z, split, sl.nt, sl.n_load);
            for(int u = 0; u < sl.nt; u++)
                for(int k = 0; k < 32; k++)
                    covered[(size_t)((z * per + u) * 32 + k)]++;
            if(sl.half)
                for(int k = K - 16; k < K; k++)
                    covered[(size_t)k]++;
            // affine form: running origin; table form: clamped tile index (both as the kernel steps them)
            int ko = sl.k00, tk = z * per * 32;
            for(int u = 0; u < sl.n_load + 12; u++)
            {
                const int to = std::min(tk, sl.kmax);
                CHECK(ko >= 0 && ko <= K - 32 && to >= 0 && to <= K - 32, "%s origin out of range", c.name.c_str());
                if(u < sl.nt)
                    CHECK(ko == (z * per + u) * 32 && to == ko, "%s whole tile %d origin %d / %d", c.name.c_str(), u, ko, to);
                else if(u == sl.nt && sl.half)
                    CHECK(ko == K - 32 && to == K - 32, "%s tail tile origin %d / %d", c.name.c_str(), ko, to);
                origins.push_back(ko);
                origins.push_back(to);
                ko = hd_next_origin(ko, sl.klast);
                tk += 32;
            }
        }
        for(int k = 0; k < K; k++)
            CHECK(covered[(size_t)k] == 1, "%s K %d split %d: k %d multiplied %d times", c.name.c_str(), K, split, k, covered[(size_t)k]);
        std::sort(origins.begin(), origins.end());
        origins.erase(std::unique(origins.begin(), origins.end()), origins.end());
        // sampled output tiles: the corners and the middle
        std::vector<int> tps = {0, tiles_p / 2, tiles_p - 1}, tqs = {0, tiles_q / 2, tiles_q - 1};
        for(int tp : tps)
            for(int tq : tqs)
            {
                const int p_own = tp * 256, q_own = tq * BQ;
                const int p0 = (v.shift_p && p_own + 256 > v.P) ? (int)v.P - 256 : p_own;
                const int q0 = (v.shift_q && q_own + BQ > v.Q) ? (int)v.Q - BQ : q_own;
                const bool affine = !ring && v.k_affine != 0;
                if(v.x_kfast)
                    check_operand<true, 256>("X", c, v, true, p0, origins, affine, ring);
                else
                    check_operand<false, 256>("X", c, v, true, p0, origins, affine, ring);
                if(v.y_kfast)
                    check_operand<true, BQ>("Y", c, v, false, q0, origins, affine, ring);
                else
                    check_operand<false, BQ>("Y", c, v, false, q0, origins, affine, ring);
                walked += (long)origins.size() * (256 + BQ) * 4;
            }
        if(want > 1 && split == 1)
            break;
    }
    return walked;
}

// ---- the 16-bit kernels on 16 x 16 x 32 MFMAs: K tiles of 64, stage[row][64] (k-contiguous operand) or stage[k][rows]
// (row-contiguous), 8 loads per wave and operand ----
template <bool KF, int BR>
static void check_hk_operand(const char* what, const Case& c, const GemmView& v, bool is_x, int r0, const std::vector<int>& origins, bool affine)
{
    const std::vector<int32_t>& rtab    = is_x ? v.xp : v.yq;
    const std::vector<int32_t>& ktab    = is_x ? v.xk : v.yk;
    const int64_t               kstride = is_x ? v.xk_stride : v.yk_stride;
    const int64_t               nrows   = is_x ? v.P : v.Q;
    const int64_t               span    = (is_x != v.swapped) ? v.spanA : v.spanB;
    std::vector<int>            seen(BR * 8, 0);
    constexpr int               NL = BR / 32;
    for(int wave = 0; wave < 4; wave++)
        for(int lane = 0; lane < 64; lane++)
            for(int i = 0; i < NL; i++)
            {
                const int    s  = (wave * NL + i) * 64 + lane;
                const HdSlot sl = hk_stage_slot<KF, BR>(s);
                if(KF)
                {
                    CHECK(sl.row >= 0 && sl.row < BR && sl.k >= 0 && sl.k + 8 <= 64 && sl.k % 8 == 0, "%s %s slot %d -> row %d k %d", c.name.c_str(), what, s,
                          sl.row, sl.k);
                    // the LDS bytes 16 s .. 16 s + 15 of a stage laid out [row][8 chunks] are where the readers look for this chunk
                    CHECK(s == sl.row * 8 + hk_chunk_pos(sl.row, sl.k / 8), "%s %s slot %d is not where the readers look", c.name.c_str(), what, s);
                    seen[(size_t)(sl.row * 8 + sl.k / 8)]++;
                }
                else
                {
                    CHECK(sl.row >= 0 && sl.row + 8 <= BR && sl.row % 8 == 0 && sl.k >= 0 && sl.k < 64, "%s %s slot %d -> row %d k %d", c.name.c_str(), what, s,
                          sl.row, sl.k);
                    // the LDS elements 8 s .. 8 s + 7 of a stage laid out [k][BR] are where the readers look for these 8 rows
                    CHECK(8 * s == sl.k * BR + hd_row_pos(sl.row, sl.k), "%s %s slot %d is not where the readers look", c.name.c_str(), what, s);
                    seen[(size_t)(sl.k * (BR / 8) + sl.row / 8)]++;
                }
                CHECK((size_t)(r0 + sl.row) < rtab.size(), "%s %s row table index %d of %zu", c.name.c_str(), what, r0 + sl.row, rtab.size());
                const int64_t rowpart = rtab[(size_t)(r0 + sl.row)];
                for(int j = 1; !KF && j < 8 && r0 + sl.row + j < nrows; j++)
                    CHECK(rtab[(size_t)(r0 + sl.row + j)] - rowpart == j, "%s %s row run broken at %d", c.name.c_str(), what, r0 + sl.row);
                const uint64_t lanepart = 2ull * ((uint64_t)rowpart + (affine ? (uint64_t)sl.k * (uint64_t)kstride : 0ull));
                CHECK(lanepart <= 0xFFFFFFFFull, "%s %s lane offset overflows 32 bits", c.name.c_str(), what);
                for(int o : origins)
                {
                    CHECK(o >= 0 && o + sl.k + (KF ? 8 : 1) <= v.K, "%s %s k %d of %lld", c.name.c_str(), what, o + sl.k, (long long)v.K);
                    // one k stride: origin in the scalar base; tables: the entry of the vector's first k, added to the row part
                    const uint64_t origin = 2ull * (affine ? (uint64_t)o * (uint64_t)kstride : (uint64_t)ktab[(size_t)(o + sl.k)]);
                    CHECK(origin <= 0xFFFFFFFFull, "%s %s origin overflows 32 bits", c.name.c_str(), what);
                    const int64_t off = rowpart + (affine ? (int64_t)(o + sl.k) * kstride : (int64_t)ktab[(size_t)(o + sl.k)]);
                    CHECK((uint64_t)off * 2 == lanepart + origin, "%s %s address parts", c.name.c_str(), what);
                    CHECK(off <= (is_x ? v.x_max_off : v.y_max_off) - 7, "%s %s offset %lld beyond the last vector", c.name.c_str(), what, (long long)off);
                    CHECK(off >= 0 && off + 8 <= span, "%s %s r0 %d slot %d origin %d: elements %lld..+8 of %lld", c.name.c_str(), what, r0, s, o,
                          (long long)off, (long long)span);
                    CHECK(off % 8 == 0, "%s %s r0 %d slot %d origin %d: offset %lld not a multiple of 8", c.name.c_str(), what, r0, s, o, (long long)off);
                    for(int j = 0; j < (KF ? 8 : 1); j++)
                        CHECK(affine ? (ktab[(size_t)(o + sl.k + j)] == (int64_t)(o + sl.k + j) * kstride && (!KF || j == 0 || kstride == 1))
                                     : (ktab[(size_t)(o + sl.k + j)] - ktab[(size_t)(o + sl.k)] == j),
                              "%s %s k run broken at %d", c.name.c_str(), what, o + sl.k);
                }
            }
    for(size_t i = 0; i < seen.size(); i++)
        CHECK(seen[i] == 1, "%s %s chunk %zu filled %d times", c.name.c_str(), what, i, seen[i]);
    if(KF)
    {
        // the operand reads: lane l of k-step ks reads chunk 4 ks + l / 16 of row (wave row) + 16 b + l % 16; 16 consecutive
        // lanes must touch 16 different 16-byte bank groups (a row is 128 bytes = half of the 64 banks)
        for(int ks = 0; ks < 2; ks++)
            for(int g = 0; g < 4; g++)
            {
                int groups = 0;
                for(int l = 16 * g; l < 16 * g + 16; l++)
                    groups |= 1 << (((l & 15) & 1) * 8 + hk_chunk_pos(l & 15, 4 * ks + (l >> 4)));
                CHECK(groups == 0xFFFF, "%s %s k-step %d lanes %d..: bank groups %x", c.name.c_str(), what, ks, 16 * g, groups);
            }
    }
    else
    {
        // a transposing read: lane g of a 16-lane group points at the 4 consecutive rows 4 (g % 4) .. + 3 of k-row g / 4; they must be
        // 8 contiguous bytes, and the group's 16 words must lie in 16 different 8-byte bank pairs (4 k-rows x 32 bytes)
        for(int b = 0; b < BR / 32; b++)
            for(int grp = 0; grp < 4; grp++)
            {
                unsigned long long pairs = 0;
                for(int g = 0; g < 16; g++)
                {
                    const int k = 8 * grp + (g >> 2), r = 16 * b + 4 * (g & 3);
                    CHECK(hd_row_pos(r + 3, k) == hd_row_pos(r, k) + 3, "%s %s rows %d..+3 at k %d are not contiguous in LDS", c.name.c_str(), what, r, k);
                    pairs |= 1ull << (((k * BR + hd_row_pos(r, k)) / 4) % 32);
                }
                CHECK(__builtin_popcountll(pairs) == 16, "%s %s block %d group %d: transposing read touches %d bank pairs", c.name.c_str(), what, b, grp,
                      __builtin_popcountll(pairs));
            }
    }
}

template <int BQ>
static long check_hk_tile(const Case& c, const GemmView& v, bool affine) // affine: the kernel multiplies a k stride (else it reads the tables)
{
    long       walked = 0;
    const int  K      = (int)v.K;
    const int  tiles_p = (int)((v.P + 255) / 256), tiles_q = (int)((v.Q + BQ - 1) / BQ);
    const int ktiles  = (K + 63) / 64;
    for(int want = 1; want <= 5; want++)
    {
        int split = std::min(want, ktiles);
        int per   = (ktiles + split - 1) / split;
        split     = (ktiles + per - 1) / per;
        std::vector<int> covered((size_t)K, 0);
        std::vector<int> origins;
        for(int z = 0; z < split; z++)
        {
            const HkSlice sl = hk_slice(K, z * per, per);
            CHECK(sl.nt >= 0 && sl.n_load >= 1 && sl.tail >= 0 && sl.tail <= 3, "%s K %d slice %d/%d: nt %d tail %d", c.name.c_str(), K, z, split, sl.nt, sl.tail);
            for(int u = 0; u < sl.nt; u++)
                for(int k = 0; k < 64; k++)
                    covered[(size_t)((z * per + u) * 64 + k)]++;
            // the tail tile is loaded from K - 64 and its last `tail` k-steps are multiplied
            for(int k = K - 16 * sl.tail; k < K; k++)
                covered[(size_t)k]++;
            // one k stride: a running origin that stops at the slice's last tile; tables: the tile index, clamped to K - 64
            int ko = sl.k00, tk = z * per * 64;
            for(int u = 0; u < sl.n_load + 8; u++)
            {
                const int to = std::min(tk, sl.kmax);
                CHECK(ko >= 0 && ko <= K - 64 && to >= 0 && to <= K - 64, "%s origin %d / %d out of range", c.name.c_str(), ko, to);
                if(u < sl.nt)
                    CHECK(ko == (z * per + u) * 64 && to == ko, "%s whole tile %d origin %d / %d", c.name.c_str(), u, ko, to);
                else if(sl.tail)
                    CHECK(ko == K - 64 && (u > sl.nt || to == K - 64), "%s tail tile origin %d / %d", c.name.c_str(), ko, to);
                else
                    CHECK(ko == (z * per + sl.nt - 1) * 64, "%s tile %d beyond the slice at %d", c.name.c_str(), u, ko);
                origins.push_back(affine ? ko : to);
                ko = hk_next_origin(ko, sl.klast);
                tk += 64;
            }
        }
        for(int k = 0; k < K; k++)
            CHECK(covered[(size_t)k] == 1, "%s K %d split %d: k %d multiplied %d times", c.name.c_str(), K, split, k, covered[(size_t)k]);
        std::sort(origins.begin(), origins.end());
        origins.erase(std::unique(origins.begin(), origins.end()), origins.end());
        for(int tp : {0, tiles_p / 2, tiles_p - 1})
            for(int tq : {0, tiles_q / 2, tiles_q - 1})
            {
                const int p_own = tp * 256, q_own = tq * BQ;
                const int p0 = (v.shift_p && p_own + 256 > v.P) ? (int)v.P - 256 : p_own;
                const int q0 = (v.shift_q && q_own + BQ > v.Q) ? (int)v.Q - BQ : q_own;
                if(v.x_kfast)
                    check_hk_operand<true, 256>("X", c, v, true, p0, origins, affine);
                else
                    check_hk_operand<false, 256>("X", c, v, true, p0, origins, affine);
                if(v.y_kfast)
                    check_hk_operand<true, BQ>("Y", c, v, false, q0, origins, affine);
                else
                    check_hk_operand<false, BQ>("Y", c, v, false, q0, origins, affine);
                walked += (long)origins.size() * (256 + BQ) * 8;
            }
        if(want > 1 && split == 1)
            break;
    }
    return walked;
}

// ---- the 32/64-bit kernels: V rows per 16-byte vector, K tiles of BK, NLW loads per wave and operand; tiles of
// ROWS x ROWS whose four waves share the stages (ROWS = 64), or load all of them each (ROWS = 32: the waves split K) ----
template <int V, int ROWS, bool KF>
static void check_wide_operand(const char* what, const Case& c, const GemmView& v, bool is_x, int r0, int BK, int NLW,
                               const std::vector<int>& origins)
{
    constexpr bool WK = ROWS == 32;
    const std::vector<int32_t>& rtab    = is_x ? v.xp : v.yq;
    const std::vector<int32_t>& ktab    = is_x ? v.xk : v.yk;
    const int64_t               kstride = is_x ? v.xk_stride : v.yk_stride;
    const int64_t               nrows   = is_x ? v.P : v.Q;
    const int64_t               span    = (is_x != v.swapped) ? v.spanA : v.spanB;
    const int64_t               es      = 16 / V;
    std::vector<int>            seen((size_t)BK * ROWS / V, 0);
    CHECK((WK ? 1 : 4) * NLW * 64 == BK * ROWS / V, "%s %s: %d loads do not tile a stage", c.name.c_str(), what, NLW * 64);
    for(int wave = 0; wave < 4; wave++)
        for(int lane = 0; lane < 64; lane++)
            for(int i = 0; i < NLW; i++)
            {
                const int    s  = ((WK ? 0 : wave * NLW) + i) * 64 + lane;
                const HdSlot sl = KF ? wd_slot_kf<V, ROWS>(s) : wd_slot<V, ROWS>(s);
                if(KF)
                {
                    CHECK(sl.row >= 0 && sl.row < ROWS && sl.k >= 0 && sl.k + V <= BK && sl.k % V == 0, "%s %s slot %d -> row %d k %d", c.name.c_str(),
                          what, s, sl.row, sl.k);
                    // the LDS bytes 16 s .. 16 s + 15 of a stage laid out [k / V][ROWS][V] are exactly these V k of this row
                    CHECK((int64_t)16 * s == (((int64_t)sl.k / V) * ROWS + sl.row) * 16, "%s %s slot %d is not where the readers look", c.name.c_str(), what, s);
                    seen[(size_t)((sl.k / V) * ROWS + sl.row)]++;
                }
                else
                {
                    CHECK(sl.row >= 0 && sl.row + V <= ROWS && sl.row % V == 0 && sl.k >= 0 && sl.k < BK, "%s %s slot %d -> row %d k %d", c.name.c_str(),
                          what, s, sl.row, sl.k);
                    // the LDS bytes 16 s .. 16 s + 15 of a stage laid out [k][ROWS] are exactly these V rows at this k
                    CHECK((int64_t)16 * s == ((int64_t)sl.k * ROWS + sl.row) * es, "%s %s slot %d is not where the readers look", c.name.c_str(), what, s);
                    seen[(size_t)(sl.k * (ROWS / V) + sl.row / V)]++;
                }
                CHECK((size_t)(r0 + sl.row) < rtab.size(), "%s %s row table index %d of %zu", c.name.c_str(), what, r0 + sl.row, rtab.size());
                const int64_t rowpart = rtab[(size_t)(r0 + sl.row)];
                for(int j = 1; !KF && j < V && r0 + sl.row + j < nrows; j++)
                    CHECK(rtab[(size_t)(r0 + sl.row + j)] - rowpart == j, "%s %s row run broken at %d", c.name.c_str(), what, r0 + sl.row);
                // the lane's part of the address, as the kernel computes it in 32 bits
                const uint64_t lanepart = (uint64_t)es * ((uint64_t)rowpart + (uint64_t)sl.k * (uint64_t)kstride);
                CHECK(lanepart <= 0xFFFFFFFFull, "%s %s lane offset overflows 32 bits", c.name.c_str(), what);
                for(int o : origins)
                {
                    const int tail_k = (int)(v.K % BK);
                    if(tail_k && o == (int)(v.K / BK) * BK)
                    {
                        // the short last tile: a vector is requested only if it lies inside K (else 16 bytes of zeros are)
                        const bool in = wd_tail_inside(KF, sl.k, V, tail_k);
                        CHECK(in == (o + sl.k + (KF ? V - 1 : 0) < v.K), "%s %s short tile: slot k %d of %d kept %d", c.name.c_str(), what, sl.k, tail_k, (int)in);
                        CHECK(KF || !in || o + sl.k < v.K, "%s %s short tile row beyond K", c.name.c_str(), what);
                        if(!in)
                            continue;
                    }
                    CHECK(o >= 0 && o + sl.k + (KF ? V - 1 : 0) < v.K, "%s %s k %d of %lld", c.name.c_str(), what, o + sl.k, (long long)v.K);
                    for(int j = 1; KF && j < V; j++)
                        CHECK(ktab[(size_t)(o + sl.k + j)] - ktab[(size_t)(o + sl.k)] == j, "%s %s k run broken at %d", c.name.c_str(), what, o + sl.k);
                    const uint64_t origin = (uint64_t)es * (uint64_t)o * (uint64_t)kstride;
                    CHECK(origin <= 0xFFFFFFFFull, "%s %s origin overflows 32 bits", c.name.c_str(), what);
                    const int64_t off = rowpart + (int64_t)(o + sl.k) * kstride;
                    CHECK((uint64_t)off * es == lanepart + origin, "%s %s address parts", c.name.c_str(), what);
                    CHECK(off >= 0 && off + V <= span, "%s %s r0 %d slot %d origin %d: elements %lld..+%d of %lld", c.name.c_str(), what, r0, s, o,
                          (long long)off, V, (long long)span);
                    CHECK(off % V == 0, "%s %s r0 %d slot %d origin %d: offset %lld not a multiple of %d", c.name.c_str(), what, r0, s, o,
                          (long long)off, V);
                    CHECK(ktab[(size_t)(o + sl.k)] == (int64_t)(o + sl.k) * kstride, "%s %s affine k offset", c.name.c_str(), what);
                }
            }
    for(size_t i = 0; i < seen.size(); i++)
        CHECK(seen[i] == (WK ? 4 : 1), "%s %s vector %zu filled %d times", c.name.c_str(), what, i, seen[i]);
}

template <int V, int ROWS>
static long check_wide_tile(const Case& c, const GemmView& v, int BK, int NLW)
{
    constexpr bool WK = ROWS == 32;
    long      walked = 0;
    const int K      = (int)v.K;
    const int tiles_p = (int)((v.P + ROWS - 1) / ROWS), tiles_q = (int)((v.Q + ROWS - 1) / ROWS);
    const int ktiles  = (K + BK - 1) / BK; // the last one may be short
    CHECK(K >= BK, "%s K %d offered to K tiles of %d", c.name.c_str(), K, BK);
    for(int want = 1; want <= 7; want++)
    {
        int split = std::min(want, ktiles);
        int per   = (ktiles + split - 1) / split;
        split     = (ktiles + per - 1) / per;
        std::vector<int> covered((size_t)K, 0);
        std::vector<int> origins;
        for(int z = 0; z < split; z++)
          for(int wave = 0; wave < (WK ? 4 : 1); wave++)
          {
            // as the kernel: the slice's (or, of it, the wave's) tiles, then repeats of the last one (a ring of up to 8 stages)
            int kt_begin = z * per;
            int nt       = std::min(kt_begin + per, ktiles) - kt_begin;
            CHECK(nt >= 1, "%s K %d slice %d/%d is empty", c.name.c_str(), K, z, split);
            if(WK)
            {
                const WdChunk ch = wd_wave_chunk(nt, wave);
                CHECK(ch.first >= 0 && ch.count >= 0 && ch.first + ch.count <= nt, "%s wave %d chunk %d + %d of %d", c.name.c_str(), wave, ch.first, ch.count, nt);
                kt_begin += ch.first;
                nt = ch.count;
                if(nt == 0)
                    continue; // the kernel requests nothing then
            }
            const int klast = (kt_begin + nt - 1) * BK;
            int       ko    = kt_begin * BK;
            for(int u = 0; u < nt + 12; u++)
            {
                CHECK(ko >= 0 && ko < K && (ko + BK <= K || ko == (K / BK) * BK), "%s origin %d out of range", c.name.c_str(), ko);
                if(u < nt)
                {
                    CHECK(ko == (kt_begin + u) * BK, "%s tile %d origin %d", c.name.c_str(), u, ko);
                    for(int k = 0; k < BK && ko + k < K; k++)
                        covered[(size_t)(ko + k)]++;
                }
                else
                    CHECK(ko == klast, "%s tile %d beyond the slice at %d, not at its last one %d", c.name.c_str(), u, ko, klast);
                origins.push_back(ko);
                ko = wd_next_origin(ko, klast, BK);
            }
          }
        for(int k = 0; k < K; k++)
            CHECK(covered[(size_t)k] == 1, "%s K %d split %d: k %d multiplied %d times", c.name.c_str(), K, split, k, covered[(size_t)k]);
        std::sort(origins.begin(), origins.end());
        origins.erase(std::unique(origins.begin(), origins.end()), origins.end());
        for(int tp : {0, tiles_p / 2, tiles_p - 1})
            for(int tq : {0, tiles_q / 2, tiles_q - 1})
            {
                if(v.x_kfast)
                    check_wide_operand<V, ROWS, true>("X", c, v, true, tp * ROWS, BK, NLW, origins);
                else
                    check_wide_operand<V, ROWS, false>("X", c, v, true, tp * ROWS, BK, NLW, origins);
                if(v.y_kfast)
                    check_wide_operand<V, ROWS, true>("Y", c, v, false, tq * ROWS, BK, NLW, origins);
                else
                    check_wide_operand<V, ROWS, false>("Y", c, v, false, tq * ROWS, BK, NLW, origins);
                walked += (long)origins.size() * 2 * BK * ROWS / V;
            }
        if(want > 1 && split == 1)
            break;
    }
    return walked;
}

struct WideTile
{
    const char* type;
    int         dtype, compute, elem_bytes, tile, bk, rows;
};

int main()
{
    std::vector<Case> cases;
    auto rank4 = [&](const char* name, std::vector<int32_t> mA, std::vector<int32_t> mB, std::vector<int32_t> mD, int64_t m0, int64_t m1,
                     int64_t n0, int64_t n1, int64_t k0, int64_t k1) {
        Case c;
        c.name = name;
        c.mA = mA, c.mB = mB, c.mD = mD;
        c.ext = {{0, m0}, {1, m1}, {10, n0}, {11, n1}, {20, k0}, {21, k1}};
        cases.push_back(c);
    };
    for(auto kk : std::vector<std::pair<int, int>>{{16, 3}, {16, 13}, {32, 1}, {32, 5}, {32, 11}, {16, 2}})
    {
        const std::string t = "k" + std::to_string(kk.first * kk.second);
        rank4((t + "_rowfast").c_str(), {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 40, 9, 24, 13, kk.first, kk.second);
        rank4((t + "_kfast").c_str(), {20, 21, 0, 1}, {20, 21, 10, 11}, {10, 11, 0, 1}, 40, 9, 24, 13, kk.first, kk.second);
        rank4((t + "_mixed").c_str(), {0, 1, 20, 21}, {20, 21, 10, 11}, {10, 11, 0, 1}, 40, 9, 24, 13, kk.first, kk.second);
        rank4((t + "_mixed2").c_str(), {20, 21, 0, 1}, {10, 11, 20, 21}, {0, 1, 10, 11}, 40, 9, 24, 13, kk.first, kk.second);
    }
    // K in tiles of 64 with every tail (0, 16, 32, 48 beyond a tile) and one tile only, every operand layout
    for(auto kk : std::vector<std::pair<int, int>>{{16, 4}, {16, 5}, {16, 7}, {16, 8}, {16, 11}, {16, 14}, {16, 21}})
    {
        const std::string t = "k" + std::to_string(kk.first * kk.second);
        rank4((t + "_kfast64").c_str(), {20, 21, 0, 1}, {20, 21, 10, 11}, {10, 11, 0, 1}, 40, 9, 24, 13, kk.first, kk.second);
        rank4((t + "_rowfast64").c_str(), {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 40, 9, 24, 13, kk.first, kk.second);
        rank4((t + "_mixed64").c_str(), {0, 1, 20, 21}, {20, 21, 10, 11}, {10, 11, 0, 1}, 40, 9, 24, 13, kk.first, kk.second);
    }
    // 4096^3 (benchmark configuration 2) and its row-major form
    rank4("cfg2", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 64, 64, 64, 64, 64, 64);
    rank4("cfg2_rowmajor", {21, 20, 1, 0}, {21, 20, 11, 10}, {11, 10, 1, 0}, 64, 64, 64, 64, 64, 64);
    // rows that are one ragged run (tiles moved back), K modes in different orders (tables), odd leading strides
    rank4("ragged_rowfast", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 15, 19, 17, 21, 16, 9);
    rank4("ktable_rowfast", {0, 1, 20, 21}, {10, 11, 21, 20}, {0, 1, 10, 11}, 40, 9, 24, 13, 16, 27);
    {
        // three K modes, the outer two in different orders in A and B
        for(int form = 0; form < 4; form++)
        {
            Case c;
            c.name = std::string("ktab3_") + (form == 0 ? "rowfast" : form == 1 ? "kfast" : form == 2 ? "mixed" : "mixed2");
            c.ext  = {{0, 40}, {1, 9}, {10, 24}, {11, 13}, {20, 16}, {21, 3}, {22, 5}};
            const bool akf = form == 1 || form == 3, bkf = form == 1 || form == 2;
            c.mA = akf ? std::vector<int32_t>{20, 21, 22, 0, 1} : std::vector<int32_t>{0, 1, 20, 21, 22};
            c.mB = bkf ? std::vector<int32_t>{20, 22, 21, 10, 11} : std::vector<int32_t>{10, 11, 20, 22, 21};
            c.mD = {0, 1, 10, 11};
            cases.push_back(c);
        }
    }
    {
        // benchmark configuration 5 (rank 6, A and B stored permuted, D padded) at full and at reduced size
        for(int small = 0; small < 3; small++)
        {
            Case c;
            c.name = small == 0 ? "cfg5" : small == 1 ? "cfg5_small_k400" : "cfg5_small_k320";
            if(small == 0)
                c.ext = {{0, 32}, {1, 7}, {2, 24}, {10, 24}, {11, 9}, {12, 32}, {20, 17}, {21, 8}, {22, 30}};
            else
                c.ext = {{0, 32}, {1, 7}, {2, 8}, {10, 24}, {11, 2}, {12, 32}, {20, small == 1 ? 5 : 4}, {21, 8}, {22, 10}};
            c.mA = {0, 1, 2, 20, 21, 22}, c.mB = {10, 11, 12, 20, 21, 22}, c.mD = {0, 1, 2, 10, 11, 12};
            c.oA = {21, 0, 20, 2, 1, 22}, c.oB = {12, 20, 10, 22, 21, 11};
            c.padD = 8, c.bilinear = true;
            cases.push_back(c);
        }
    }
    long walked = 0;
    int  offered = 0, offered_hk = 0, offered_ring = 0, offered_ring_chunked = 0, computed_rows = 0;
    for(const Case& c : cases)
    {
        ProblemIn in;
        in.A = tensor(c, c.mA, c.oA, 0);
        in.B = tensor(c, c.mB, c.oB, 0);
        in.D = tensor(c, c.mD, c.oD, c.padD);
        in.bilinear = c.bilinear;
        if(c.bilinear)
            in.C = in.D;
        in.compute = 4; // HIPTENSOR_COMPUTE_32F
        GemmView    v;
        std::string why;
        const PlanStatus st = build_view(in, v, why);
        CHECK(st == PlanStatus::OK, "%s: %s", c.name.c_str(), why.c_str());
        if(st != PlanStatus::OK)
            continue;
        // is a direct-load tile offered for it?  (tile ids 9: 256 x 256, 10: 256 x 192; on 16 x 16 x 32 MFMAs: 11: 256 x 256 in
        // K tiles of 64, one k stride per operand; 12: 256 x 192 in K tiles of 32 through a ring of four stages, k offsets from tables)
        for(int tile : {9, 10, 11, 12})
        {
            hiptk_problem_t p{};
            p.cls = v.cls, p.tile_id = tile, p.x_kfast = v.x_kfast, p.y_kfast = v.y_kfast, p.x_vec = v.x_vec, p.y_vec = v.y_vec;
            p.k_affine = v.k_affine, p.P = v.P, p.Q = v.Q, p.K = v.K, p.shift_p = v.shift_p, p.shift_q = v.shift_q;
            p.xy_aligned = v.xy_aligned, p.x_max_off = (int32_t)v.x_max_off, p.y_max_off = (int32_t)v.y_max_off;
            p.x_rows_adjacent = v.x_rows_adjacent, p.y_rows_adjacent = v.y_rows_adjacent;
            const bool avail = hiptk_kernel_available(&p) != 0;
            std::printf("%-22s P %5lld Q %5lld K %5lld xkf %d ykf %d vec %d/%d kaff %d shift %d/%d aligned %d tile %2d: %s\n", c.name.c_str(),
                        (long long)v.P, (long long)v.Q, (long long)v.K, v.x_kfast, v.y_kfast, v.x_vec, v.y_vec, v.k_affine, v.shift_p, v.shift_q,
                        v.xy_aligned, tile, avail ? "offered" : "not offered");
            if(!avail)
                continue;
            CHECK(v.x_vec == 8 && v.y_vec == 8 && v.K % 16 == 0 && v.K >= 32 && v.xy_aligned, "%s offered outside its restrictions", c.name.c_str());
            if(tile == 11)
            {
                computed_rows += check_computed_rows(c, v);
                CHECK(v.k_affine && v.K >= 64, "%s offered the K-tile-of-64 kernel outside its restrictions", c.name.c_str());
                offered_hk++;
                walked += check_hk_tile<256>(c, v, true);
                continue;
            }
            if(tile == 12)
            {
                offered_ring++;
                offered_ring_chunked += (v.x_kfast && v.x_rows_adjacent) || (v.y_kfast && v.y_rows_adjacent);
                walked += check_tile_size<192>(c, v, true);
                continue;
            }
            offered++;
            walked += tile == 9 ? check_tile_size<256>(c, v) : check_tile_size<192>(c, v);
        }
    }
    CHECK(offered >= 40, "only %d (case, tile) pairs were offered a direct-load kernel", offered);
    CHECK(offered_hk >= 15, "only %d cases were offered the kernel with K tiles of 64", offered_hk);
    CHECK(computed_rows >= 10, "only %d cases of the K-tile-of-64 kernel have computed row offsets", computed_rows);
    CHECK(offered_ring >= 20, "only %d cases were offered the ring kernel", offered_ring);
    CHECK(offered_ring_chunked >= 3, "only %d cases of the ring kernel stage an operand chunk-major", offered_ring_chunked);
    std::printf("offered: %d (K tiles of 32), %d (K tiles of 64), %d (ring; %d chunk-major)\n", offered, offered_hk, offered_ring, offered_ring_chunked);

    // ---- 32/64-bit classes ----
    // benchmark configurations 1 (256^3), 3 (1920^2 x 768), 4 (1024^2 x 512) and a tensor of 2^32 bytes and more
    rank4("cfg1", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 16, 16, 16, 16, 16, 16);
    rank4("cfg3", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 48, 40, 48, 40, 32, 24);
    rank4("cfg4", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 32, 32, 32, 32, 32, 16);
    rank4("k8_rowfast", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 40, 9, 24, 13, 8, 1);
    rank4("k24_rowfast", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 42, 9, 25, 13, 8, 3);
    // odd row counts under k-contiguous operands: tiles overhang, C / D may ask for moved-back tiles, which these kernels do not do
    rank4("ragged_kfast", {20, 21, 0, 1}, {20, 21, 10, 11}, {10, 11, 0, 1}, 15, 19, 17, 21, 16, 9);
    // K that ends inside a K tile: 100 = 6 x 16 + 4 = 12 x 8 + 4, 42 (not even a multiple of the f32 vector: row-contiguous only)
    rank4("k100_rowfast", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 40, 9, 24, 13, 20, 5);
    rank4("k100_kfast", {20, 21, 0, 1}, {20, 21, 10, 11}, {10, 11, 0, 1}, 40, 9, 24, 13, 20, 5);
    rank4("k100_mixed", {0, 1, 20, 21}, {20, 21, 10, 11}, {10, 11, 0, 1}, 40, 9, 24, 13, 20, 5);
    rank4("k42_rowfast", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 40, 9, 24, 13, 6, 7);
    rank4("k42_kfast", {20, 21, 0, 1}, {20, 21, 10, 11}, {10, 11, 0, 1}, 40, 9, 24, 13, 6, 7);
    rank4("big_rowfast", {0, 1, 20, 21}, {10, 11, 20, 21}, {0, 1, 10, 11}, 8192, 16, 64, 1, 64, 64);
    const WideTile wide[] = {{"f32", 0, 4, 4, 2, 16, 64}, {"f64", 1, 16, 8, 2, 8, 64}, {"c32", 4, 2048, 8, 2, 8, 64},
                             {"f32", 0, 4, 4, 3, 16, 32}, {"f64", 1, 16, 8, 3, 8, 32}, {"c32", 4, 2048, 8, 3, 8, 32},
                             {"c64", 5, 4096, 16, 3, 8, 64}, {"c64", 5, 4096, 16, 4, 8, 32}};
    int offered_wide = 0, refused_big = 0, offered_kf = 0, offered_mixed = 0;
    for(const WideTile& w : wide)
        for(const Case& c : cases)
        {
            g_dtype = w.dtype;
            ProblemIn in;
            in.A = tensor(c, c.mA, c.oA, 0);
            in.B = tensor(c, c.mB, c.oB, 0);
            in.D = tensor(c, c.mD, c.oD, c.padD);
            in.bilinear = c.bilinear;
            if(c.bilinear)
                in.C = in.D;
            in.compute = w.compute;
            GemmView    v;
            std::string why;
            const PlanStatus st = build_view(in, v, why);
            CHECK(st == PlanStatus::OK, "%s %s: %s", w.type, c.name.c_str(), why.c_str());
            if(st != PlanStatus::OK)
                continue;
            hiptk_problem_t p{};
            p.cls = v.cls, p.tile_id = w.tile, p.x_kfast = v.x_kfast, p.y_kfast = v.y_kfast, p.x_vec = v.x_vec, p.y_vec = v.y_vec;
            p.k_affine = v.k_affine, p.P = v.P, p.Q = v.Q, p.K = v.K, p.shift_p = v.shift_p, p.shift_q = v.shift_q;
            p.xy_aligned = v.xy_aligned, p.x_max_off = (int32_t)v.x_max_off, p.y_max_off = (int32_t)v.y_max_off;
            const bool avail = hiptk_kernel_available(&p) != 0;
            std::printf("%s %-22s P %5lld Q %5lld K %5lld xkf %d ykf %d vec %d/%d kaff %d shift %d/%d aligned %d tile %2d: %s\n", w.type,
                        c.name.c_str(), (long long)v.P, (long long)v.Q, (long long)v.K, v.x_kfast, v.y_kfast, v.x_vec, v.y_vec, v.k_affine,
                        v.shift_p, v.shift_q, v.xy_aligned, w.tile, avail ? "offered" : "not offered");
            const bool big = (std::max(v.x_max_off, v.y_max_off) + 16 / w.elem_bytes) * (int64_t)w.elem_bytes > 0xFFFFFFFFll;
            if(c.name == "big_rowfast" && big)
            {
                CHECK(!avail, "%s %s: offered although byte offsets pass 2^32", w.type, c.name.c_str());
                refused_big++;
            }
            if(!avail)
                continue;
            const int V = 16 / w.elem_bytes;
            CHECK(v.x_vec == V && v.y_vec == V && v.k_affine && v.K >= w.bk && (!(v.x_kfast || v.y_kfast) || v.K % V == 0) && v.xy_aligned
                      && (v.x_kfast || !v.shift_p) && (v.y_kfast || !v.shift_q),
                  "%s %s offered outside its restrictions", w.type, c.name.c_str());
            offered_wide++;
            const int nlw = w.bk * w.rows * w.elem_bytes / (w.rows == 32 ? 1024 : 4096);
            offered_kf += (v.x_kfast || v.y_kfast) ? 1 : 0;
            offered_mixed += (v.x_kfast != v.y_kfast) ? 1 : 0;
            if(w.rows == 64)
                walked += V == 4   ? check_wide_tile<4, 64>(c, v, w.bk, nlw)
                          : V == 2 ? check_wide_tile<2, 64>(c, v, w.bk, nlw)
                                   : check_wide_tile<1, 64>(c, v, w.bk, nlw);
            else
                walked += V == 4   ? check_wide_tile<4, 32>(c, v, w.bk, nlw)
                          : V == 2 ? check_wide_tile<2, 32>(c, v, w.bk, nlw)
                                   : check_wide_tile<1, 32>(c, v, w.bk, nlw);
        }
    g_dtype = 2;
    CHECK(offered_mixed >= 30, "only %d mixed (case, type, tile) triples were offered a 32/64-bit direct-load kernel", offered_mixed);
    CHECK(offered_kf >= 30, "only %d k-contiguous (case, type, tile) triples were offered a 32/64-bit direct-load kernel", offered_kf);
    CHECK(offered_wide >= 60, "only %d (case, type, tile) triples were offered a 32/64-bit direct-load kernel", offered_wide);
    CHECK(refused_big >= 2, "the tensor past 2^32 bytes was not exercised (%d)", refused_big);
    std::printf("%s: %d + %d problems x tiles, %ld requests walked, %d failures\n", g_fail ? "FAILED" : "ok", offered, offered_wide, walked,
                g_fail);
    return g_fail ? 1 : 0;
}
