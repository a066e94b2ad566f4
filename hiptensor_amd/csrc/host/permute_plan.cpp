#include "permute_plan.hpp"

#include <algorithm>
#include <cstring>

namespace hipta
{
    namespace
    {
        struct Tile
        {
            int ti, tj;
        };
        // the kernel layer's tile shapes (elements): square, long along i, long along j
        constexpr Tile TILES4[4] = {{64, 64}, {256, 16}, {16, 256}, {128, 128}};
        constexpr Tile TILES2[4] = {{128, 128}, {512, 32}, {32, 512}, {256, 128}};

        bool alignedTo(const void* p, int64_t bytes)
        {
            return (reinterpret_cast<uintptr_t>(p) % (uintptr_t)bytes) == 0;
        }

        // Largest vector (elements) not above cap that divides `extent` and every stride in
        // `others`, and that the address is aligned for.
        int pickVec(int elem_bytes, int cap, int64_t extent, const std::vector<int64_t>& others, const void* p, bool copy)
        {
            const int cands4[] = {4, 2, 1}, cands2[] = {8, 2, 1}, candsCopy2[] = {8, 4, 2, 1};
            const int* c;
            int        n;
            if(elem_bytes == 4)
                c = cands4, n = 3;
            else if(copy)
                c = candsCopy2, n = 4;
            else
                c = cands2, n = 3;
            for(int k = 0; k < n; ++k)
            {
                const int v = c[k];
                if(v > cap || extent % v != 0 || !alignedTo(p, (int64_t)v * elem_bytes))
                    continue;
                bool ok = true;
                for(int64_t s : others)
                    ok = ok && (s % v == 0);
                if(ok)
                    return v;
            }
            return 1;
        }

        // Share of a tile grid's lanes that fall inside the extents.
        double coverage(int64_t e, int t)
        {
            const int64_t tiles = (e + t - 1) / t;
            return (double)e / (double)(tiles * t);
        }

        int pickTile(int elem_bytes, int64_t e_i, int64_t e_j, const int order[3])
        {
            const Tile* ts   = elem_bytes == 4 ? TILES4 : TILES2;
            int         best = order[0];
            double      bc   = -1.0;
            for(int k = 0; k < 3; ++k)
            {
                const int    t = order[k];
                const double c = coverage(e_i, ts[t].ti) * coverage(e_j, ts[t].tj);
                if(c > bc + 1e-9)
                    bc = c, best = t;
            }
            return best;
        }
    }

    PermuteStatus plan_permutation(const PermuteIn& in, const PermuteTuning& tune, hiptk_permute_t& out)
    {
        std::memset(&out, 0, sizeof(out));
        const size_t rank = in.lenA.size();
        if(in.lenB.size() != rank || in.modeA.size() != rank || in.modeB.size() != rank)
            return PermuteStatus::BAD_RANK;

        // position of each B mode in A; every label once on both sides, lengths agree
        std::vector<int> posInA(rank, -1);
        std::vector<bool> used(rank, false);
        for(size_t k = 0; k < rank; ++k)
        {
            for(size_t i = 0; i < rank; ++i)
                if(in.modeA[i] == in.modeB[k] && !used[i])
                {
                    posInA[k] = (int)i;
                    break;
                }
            if(posInA[k] < 0 || in.lenB[k] != in.lenA[posInA[k]])
                return PermuteStatus::BAD_MODES;
            used[posInA[k]] = true;
        }
        int64_t count = 1;
        for(size_t i = 0; i < rank; ++i)
        {
            if(in.lenA[i] < 0)
                return PermuteStatus::BAD_MODES;
            if(in.lenA[i] == 0)
                return PermuteStatus::EMPTY;
            count *= in.lenA[i];
            if(count >= (int64_t(1) << 31))
                return PermuteStatus::TOO_LARGE;
        }

        // packed strides, first listed mode fastest; B's stride carried to A's order
        std::vector<int64_t> bInA(rank, 0);
        {
            int64_t s = 1;
            for(size_t k = 0; k < rank; ++k)
            {
                bInA[posInA[k]] = s;
                s *= in.lenB[k];
            }
        }
        // drop extent-1 modes, fuse neighbours of A that are neighbours in B in the same order
        std::vector<int64_t> ext, as, bs;
        {
            int64_t s = 1;
            for(size_t i = 0; i < rank; ++i)
            {
                const int64_t e = in.lenA[i];
                if(e != 1)
                {
                    if(!ext.empty() && bInA[i] == bs.back() * ext.back())
                        ext.back() *= e;
                    else
                    {
                        ext.push_back(e);
                        as.push_back(s);
                        bs.push_back(bInA[i]);
                    }
                }
                s *= e;
            }
            if(ext.empty())
            {
                ext.push_back(1);
                as.push_back(1);
                bs.push_back(1);
            }
        }
        const int r    = (int)ext.size();
        if(r > HIPTK_PERM_MAX_RANK)
            return PermuteStatus::BAD_RANK; // more modes left after fusion than the kernels index
        out.elem_bytes = in.elem_bytes;
        out.rank       = r;
        for(int d = 0; d < r; ++d)
        {
            out.extent[d]   = (int32_t)ext[d];
            out.a_stride[d] = (int32_t)as[d];
            out.b_stride[d] = (int32_t)bs[d];
        }
        out.vec_r = out.vec_w = 1;
        out.group             = tune.group >= 0 ? tune.group : 1;
        const int cap         = std::max(1, tune.max_vec);

        if(r == 1)
        {
            out.kernel = HIPTK_PERM_COPY;
            const int v = std::min(pickVec(in.elem_bytes, cap, ext[0], {}, in.A, true),
                                   pickVec(in.elem_bytes, cap, ext[0], {}, in.B, true));
            out.vec_r = out.vec_w = v;
            return PermuteStatus::OK;
        }

        int jB = 0; // B's fastest mode
        for(int d = 0; d < r; ++d)
            if(bs[d] == 1)
                jB = d;

        // layout-admissible kernels: TILED needs differing fastest modes, ROWS a shared one,
        // STRIP a tile mode of at most 64 elements whose partner follows it directly in memory
        const bool shared = jB == 0;
        const bool stripJ = !shared && ext[jB] <= 64 && ext[jB] <= ext[0] && bs[0] == ext[jB]; // short j, B holds i right after it
        const bool stripI = !shared && ext[0] <= 64 && jB == 1 && !stripJ; // short i, A holds j right after it
        // Many short modes: no single mode gives a long run.  A tile row then spans A's two
        // fastest modes and a tile column B's two fastest modes, where those are free.
        // Fills `out` and returns true when that kernel applies (force: even where the plain
        // tiles would cover the extents well).
        auto tryGrouped = [&](bool force, bool anySize) -> bool {
            if(shared)
                return false;
            const int64_t target = 128; // elements per tile row / column aimed at
            // a side whose fastest mode is short takes a chunk of the next mode along; a long one
            // is tiled by itself
            int mi2 = (ext[0] <= target && r > 1 && jB != 1) ? 1 : -1;
            int mj2 = -1;
            if(ext[jB] <= target)
                for(int d = 1; d < r; ++d)
                    if(bs[d] == ext[jB])
                        mj2 = d;
            if(mi2 != -1 && mi2 == mj2) // both sides want mode 1: the side with the shorter run gets it
                (ext[jB] < ext[0] ? mi2 : mj2) = -1;
            const int    order[] = {0, 1, 2};
            const int    st      = pickTile(in.elem_bytes, ext[0], ext[jB], order);
            const Tile*  ts      = in.elem_bytes == 4 ? TILES4 : TILES2;
            const double cov     = coverage(ext[0], ts[st].ti) * coverage(ext[jB], ts[st].tj);
            if(cov >= 0.7 && !force)
                return false;
            std::vector<int64_t> aOth(as.begin() + 1, as.end()), bOth;
            for(int d = 0; d < r; ++d)
                if(d != jB)
                    bOth.push_back(bs[d]);
            int vr = pickVec(in.elem_bytes, cap, ext[0], aOth, in.A, false);
            int vw = pickVec(in.elem_bytes, cap, ext[jB], bOth, in.B, false);
            int64_t wi = std::min<int64_t>(ext[0], target), wj = std::min<int64_t>(ext[jB], target);
            int64_t ci = mi2 == -1 ? 1 : std::max<int64_t>(1, std::min<int64_t>(ext[mi2], target / ext[0]));
            int64_t cj = mj2 == -1 ? 1 : std::max<int64_t>(1, std::min<int64_t>(ext[mj2], target / ext[jB]));
            auto ldsBytes = [&]() { return (wj * cj) * (wi * ci + 2) * in.elem_bytes; };
            while(ldsBytes() > 56 * 1024)
            {
                // shrink the longer side: first its chunk, then (a tiled side) its width
                const bool iSide = wi * ci >= wj * cj;
                int64_t&   c     = iSide ? ci : cj;
                int64_t&   w     = iSide ? wi : wj;
                const int  v     = iSide ? vr : vw;
                if(c > 1)
                    c -= 1;
                else if(w > 2 * v && w > 16)
                    w = (w / 2 + v - 1) / v * v;
                else
                    return false;
            }
            // a small problem needs more workgroups than long runs: halve the larger side of the
            // tile until there are two workgroups per compute unit (256 of them) or the tile is small
            auto groups = [&]() {
                int64_t g = ((ext[0] + wi - 1) / wi) * ((ext[jB] + wj - 1) / wj);
                for(int d = 1; d < r; ++d)
                {
                    if(d == jB)
                        continue;
                    g *= d == mi2 ? (ext[d] + ci - 1) / ci : d == mj2 ? (ext[d] + cj - 1) / cj : ext[d];
                }
                return g;
            };
            while(groups() < 512 && wi * ci * wj * cj >= 2 * 2048)
            {
                const bool iSide = wi * ci >= wj * cj;
                int64_t&   c     = iSide ? ci : cj;
                int64_t&   w     = iSide ? wi : wj;
                const int  v     = iSide ? vr : vw;
                if(c > 1)
                    c = (c + 1) / 2;
                else if(w > 2 * v && w > 16)
                    w = (w / 2 + v - 1) / v * v;
                else
                    break;
            }
            while(vr > 1 && (wi * ci / vr < 2 || wi % vr != 0))
                vr = vr == 8 ? 2 : vr / 2;
            while(vw > 1 && (wj * cj / vw < 2 || wj % vw != 0))
                vw = vw == 8 ? 2 : vw / 2;
            if(wi < 2 || wj < 2 || wi * ci / vr < 2 || wj * cj / vw < 2)
                return false;
            if(wi * ci * wj * cj < 1536 && !anySize)
                return false; // tiles of a few hundred elements: one thread per element does better
                              // (192-element tiles: 459 against 1910 GB/s; 1890-element tiles: 1590 against 1190)
            out.kernel  = HIPTK_PERM_GROUPED;
            out.mode_i  = 0;
            out.mode_j  = jB;
            out.mode_i2 = mi2;
            out.mode_j2 = mj2;
            out.chunk_i = (int32_t)ci;
            out.chunk_j = (int32_t)cj;
            out.width_i = (int32_t)wi;
            out.width_j = (int32_t)wj;
            out.vec_r   = vr;
            out.vec_w   = vw;
            return true;
        };
        // A short shared fastest mode (interleaved channels): tiles of that mode times a chunk of
        // A's next mode times a chunk of B's next mode, so that both sides see long runs.
        auto tryShared = [&](bool force) -> bool {
            if(!shared || r < 3 || ext[0] > 128)
                return false;
            if(ext[0] * in.elem_bytes >= 64 && !force)
                return false; // from 64-byte runs on, plain rows do as well or better (measured)
            const int mi2 = 1;
            int       mj2 = -1;
            for(int d = 1; d < r; ++d)
                if(bs[d] == ext[0])
                    mj2 = d;
            if(mj2 == -1 || mj2 == mi2)
                return false;
            const int64_t target = 512 / in.elem_bytes; // elements per run aimed at
            int64_t       ci = std::max<int64_t>(1, std::min<int64_t>(ext[mi2], target / ext[0]));
            int64_t       cj = std::max<int64_t>(1, std::min<int64_t>(ext[mj2], target / ext[0]));
            auto ldsBytes = [&]() { return cj * (ext[0] * ci + 2) * in.elem_bytes; };
            while(ldsBytes() > 56 * 1024 && cj > 1)
                cj -= 1;
            if(ldsBytes() > 56 * 1024)
                return false;
            std::vector<int64_t> aOth(as.begin() + 1, as.end()), bOth(bs.begin() + 1, bs.end());
            int v = std::min(pickVec(in.elem_bytes, cap, ext[0], aOth, in.A, false), pickVec(in.elem_bytes, cap, ext[0], bOth, in.B, false));
            while(v > 1 && (ext[0] * ci / v < 2 || ext[0] * cj / v < 2))
                v = v == 8 ? 2 : v / 2;
            if(ext[0] * ci / v < 2 || ext[0] * cj / v < 2)
                return false;
            out.kernel  = HIPTK_PERM_SHARED;
            out.mode_i  = 0;
            out.mode_j  = 0;
            out.mode_i2 = mi2;
            out.mode_j2 = mj2;
            out.chunk_i = (int32_t)ci;
            out.chunk_j = (int32_t)cj;
            out.vec_r = out.vec_w = v;
            return true;
        };
        out.mode_i2 = out.mode_j2 = -1;
        out.chunk_i = out.chunk_j = 1;
        int        kernel;
        if(tune.kernel == HIPTK_PERM_GROUPED && (tryGrouped(true, true) || tryShared(true)))
            return PermuteStatus::OK;
        if(tune.kernel == HIPTK_PERM_GATHER)
            kernel = HIPTK_PERM_GATHER;
        else if(tune.kernel == HIPTK_PERM_STRIP && (stripJ || stripI))
            kernel = HIPTK_PERM_STRIP;
        else if(tune.kernel == HIPTK_PERM_TILED || tune.kernel == HIPTK_PERM_ROWS)
            kernel = shared ? HIPTK_PERM_ROWS : HIPTK_PERM_TILED;
        else if(count <= 16384)
            kernel = HIPTK_PERM_GATHER; // a launch's worth of latency either way
        else if((stripJ && ext[0] >= 64) || (stripI && ext[jB] >= 64))
            kernel = HIPTK_PERM_STRIP;
        else if(shared && tune.tile < 0 && tryShared(false))
            return PermuteStatus::OK;
        else if(shared)
            kernel = ext[0] >= 16 ? HIPTK_PERM_ROWS : HIPTK_PERM_GATHER;
        else if(tune.tile < 0 && tryGrouped(ext[0] < 16 || ext[jB] < 16, false)) // (the plain tiles need 16 and more)
            return PermuteStatus::OK;
        else
            kernel = (ext[0] >= 16 && ext[jB] >= 16) ? HIPTK_PERM_TILED : HIPTK_PERM_GATHER;
        out.kernel = kernel;
        if(kernel == HIPTK_PERM_GATHER)
            return PermuteStatus::OK;

        out.mode_i = 0;
        if(kernel == HIPTK_PERM_STRIP)
        {
            out.mode_j = jB;
            out.tile   = stripJ ? 0 : 1;
            const int64_t        run = ext[0] * ext[jB];
            std::vector<int64_t> linOthers, rowOthers;
            for(int d = 1; d < r; ++d)
            {
                if(d != jB)
                    linOthers.push_back(stripJ ? bs[d] : as[d]);
                if(stripJ || d != jB)
                    rowOthers.push_back(stripJ ? as[d] : bs[d]);
            }
            if(!stripJ)
                rowOthers.push_back(bs[0]);
            if(stripJ)
            {
                out.vec_r = pickVec(in.elem_bytes, cap, ext[0], rowOthers, in.A, false);
                out.vec_w = pickVec(in.elem_bytes, cap, run, linOthers, in.B, false);
            }
            else
            {
                out.vec_r = pickVec(in.elem_bytes, cap, run, linOthers, in.A, false);
                out.vec_w = pickVec(in.elem_bytes, cap, ext[jB], rowOthers, in.B, false);
            }
            return PermuteStatus::OK;
        }
        std::vector<int64_t> aOthers(as.begin() + 1, as.end());
        const int            vr = pickVec(in.elem_bytes, cap, ext[0], aOthers, in.A, false);
        if(kernel == HIPTK_PERM_TILED)
        {
            out.mode_j = jB;
            std::vector<int64_t> bOthers;
            for(int d = 0; d < r; ++d)
                if(d != jB)
                    bOthers.push_back(bs[d]);
            out.vec_r         = vr;
            out.vec_w         = pickVec(in.elem_bytes, cap, ext[jB], bOthers, in.B, false);
            const int order[] = {0, 1, 2};
            out.tile          = tune.tile >= 0 && tune.tile <= 3 ? tune.tile : pickTile(in.elem_bytes, ext[0], ext[jB], order);
            // The 64 KiB tile doubles the contiguous run (on both sides for f32: 512 bytes; on A's
            // side for f16), which HBM rewards as long as the tile grid does not lose much more
            // of it at the edges.
            if(tune.tile < 0)
            {
                const Tile*  ts   = in.elem_bytes == 4 ? TILES4 : TILES2;
                const double cur  = coverage(ext[0], ts[out.tile].ti) * coverage(ext[jB], ts[out.tile].tj);
                const double big  = coverage(ext[0], ts[3].ti) * coverage(ext[jB], ts[3].tj);
                if(big >= 0.9 * cur)
                    out.tile = 3;
            }
        }
        else
        {
            // second tile mode: the one B walks next, so that stores sweep B in order
            int mj = 1;
            for(int d = 1; d < r; ++d)
                if(bs[d] < bs[mj])
                    mj = d;
            out.mode_j = mj;
            std::vector<int64_t> bOthers(bs.begin() + 1, bs.end());
            const int            vw = pickVec(in.elem_bytes, cap, ext[0], bOthers, in.B, false);
            out.vec_r = out.vec_w = std::min(vr, vw);
            const int order[]     = {1, 0, 2};
            out.tile              = tune.tile >= 0 && tune.tile <= 2 ? tune.tile : pickTile(in.elem_bytes, ext[0], ext[mj], order);
        }
        return PermuteStatus::OK;
    }
}
