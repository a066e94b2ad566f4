#include "planner.hpp"

#include <algorithm>
#include <cstdio>

#include "hiptk_kernels.h"

namespace hipta
{
    namespace
    {
        // hipDataType values (hip/library_types.h)
        enum
        {
            DT_R32F  = 0,
            DT_R64F  = 1,
            DT_R16F  = 2,
            DT_C32F  = 4,
            DT_C64F  = 5,
            DT_R16BF = 14
        };
        // hiptensorComputeType_t values
        enum
        {
            CT_16F  = 1,
            CT_32F  = 4,
            CT_64F  = 16,
            CT_16BF = 1024,
            CT_C32F = 2048,
            CT_C64F = 4096
        };

        int find_mode(const std::vector<int32_t>& modes, int32_t m)
        {
            for(size_t i = 0; i < modes.size(); i++)
                if(modes[i] == m)
                    return (int)i;
            return -1;
        }

        bool has_repeats(const std::vector<int32_t>& modes)
        {
            for(size_t i = 0; i < modes.size(); i++)
                for(size_t j = i + 1; j < modes.size(); j++)
                    if(modes[i] == modes[j])
                        return true;
            return false;
        }

        enum Group
        {
            GP,
            GQ,
            GK
        };

        // Merge dims i and i+1 (i is faster) when every tensor that carries them steps
        // through both with one stride.
        void fuse(std::vector<Dim>& d, Group g, bool bilinear)
        {
            size_t i = 0;
            while(i + 1 < d.size())
            {
                const Dim& a = d[i];
                const Dim& b = d[i + 1];
                bool       ok;
                if(g == GK)
                    ok = b.sx == a.sx * a.len && b.sy == a.sy * a.len;
                else
                {
                    ok = (g == GP ? b.sx == a.sx * a.len : b.sy == a.sy * a.len)
                         && b.sd == a.sd * a.len && (!bilinear || b.sc == a.sc * a.len);
                }
                if(ok)
                {
                    d[i].len *= b.len;
                    d.erase(d.begin() + (long)i + 1);
                }
                else
                    i++;
            }
        }

        // (the per-tensor check in build_view has already ruled out products that overflow)
        int64_t extent(const std::vector<Dim>& d)
        {
            int64_t e = 1;
            for(const Dim& x : d)
                e *= x.len;
            return e;
        }

        template <typename Get>
        bool make_table(const std::vector<Dim>& d, int64_t n, size_t padded, Get get, std::vector<int32_t>& out, int64_t& maxoff)
        {
            out.assign(padded, 0);
            std::vector<int64_t> idx(d.size(), 0);
            int64_t              off = 0;
            maxoff                   = 0;
            for(int64_t i = 0; i < n; i++)
            {
                if(off > 0x7FFFFFFFll)
                    return false;
                out[(size_t)i] = (int32_t)off;
                maxoff         = std::max(maxoff, off);
                // odometer increment, fastest dim first
                for(size_t k = 0; k < d.size(); k++)
                {
                    off += get(d[k]);
                    if(++idx[k] < d[k].len)
                        break;
                    off -= get(d[k]) * d[k].len;
                    idx[k] = 0;
                }
            }
            return true;
        }

        // Extent from which a sole row / column dim may carry vectors although it is not a multiple
        // of them: the smallest tile of every class with vector kernels (64 x 64) then fits and can
        // be moved back; larger tiles are offered only where they fit (hiptk_kernel_available).
        constexpr int64_t RAGGED_MIN = 64;

        // Widest power-of-two vector (<= maxv elements) along a contiguous leading dim.  Vectors
        // must not straddle the end of that dim's run: its length is a multiple of the vector, or
        // (`sole`: it is its group's only dim, at least RAGGED_MIN long) the kernels move the last
        // tile back so that every vector of it lies inside; *ragged says that this is relied on.
        // Neither the base address nor the other strides need to be multiples of the vector:
        // global memory takes vector loads and stores at any element-aligned address on this
        // target (the compiler itself emits them for under-aligned types).
        int vector_width(int64_t lead_len, bool sole, int maxv, bool* ragged, int64_t ragged_min = RAGGED_MIN)
        {
            if(ragged)
                *ragged = false;
            for(int v = maxv; v > 1; v /= 2)
            {
                if(lead_len % v == 0)
                    return v;
                if(ragged && sole && lead_len >= ragged_min)
                {
                    *ragged = true;
                    return v;
                }
            }
            return 1;
        }
    }

    int64_t span_elems(const std::vector<int64_t>& len, const std::vector<int64_t>& stride)
    {
        int64_t e = 1;
        for(size_t i = 0; i < len.size(); i++)
        {
            if(len[i] <= 0)
                return 0;
            e += (len[i] - 1) * (i < stride.size() ? stride[i] : 0);
        }
        return e;
    }

    int kernel_class(int typeA, int typeB, int typeC, int typeD, bool bilinear, int compute)
    {
        if(typeA != typeB || typeA != typeD || (bilinear && typeC != typeA))
            return -1;
        switch(typeA)
        {
        case DT_R16F: return compute == CT_32F ? HIPTK_F16 : -1;
        case DT_R16BF: return compute == CT_32F ? HIPTK_BF16 : -1;
        case DT_R32F:
            if(compute == CT_32F)
                return HIPTK_F32;
            if(compute == CT_16F)
                return HIPTK_F32_AS_F16;
            if(compute == CT_16BF)
                return HIPTK_F32_AS_BF16;
            return -1;
        case DT_R64F:
            if(compute == CT_64F)
                return HIPTK_F64;
            if(compute == CT_32F)
                return HIPTK_F64_AS_F32;
            return -1;
        case DT_C32F: return compute == CT_C32F ? HIPTK_C32 : -1;
        case DT_C64F: return compute == CT_C64F ? HIPTK_C64 : -1;
        default: return -1;
        }
    }

    int class_elem_bytes(int cls)
    {
        switch(cls)
        {
        case HIPTK_F16:
        case HIPTK_BF16: return 2;
        case HIPTK_F32:
        case HIPTK_F32_AS_F16:
        case HIPTK_F32_AS_BF16: return 4;
        case HIPTK_F64:
        case HIPTK_F64_AS_F32:
        case HIPTK_C32: return 8;
        case HIPTK_C64: return 16;
        default: return 0;
        }
    }

    int class_max_vec(int cls)
    {
        const int b = class_elem_bytes(cls);
        return b ? 16 / b : 1;
    }

    PlanStatus build_view(const ProblemIn& in, GemmView& v, std::string& why)
    {
        v          = GemmView();
        v.bilinear = in.bilinear;
        v.cls      = kernel_class(in.A.dtype, in.B.dtype, in.C.dtype, in.D.dtype, in.bilinear, in.compute);
        if(v.cls < 0)
        {
            why = "no kernel class for this combination of data types and compute type";
            return PlanStatus::UNSUPPORTED_TYPES;
        }
        v.elem_bytes = class_elem_bytes(v.cls);

        const TensorIn &A = in.A, &B = in.B, &C = in.C, &D = in.D;
        if(A.len.size() != A.mode.size() || A.len.size() != A.stride.size()
           || B.len.size() != B.mode.size() || B.len.size() != B.stride.size()
           || D.len.size() != D.mode.size() || D.len.size() != D.stride.size()
           || (in.bilinear && (C.len.size() != D.len.size() || C.stride.size() != D.len.size())))
        {
            why = "rank of a tensor descriptor does not match its mode list";
            return PlanStatus::INVALID;
        }
        if(has_repeats(A.mode) || has_repeats(B.mode) || has_repeats(D.mode))
        {
            why = "a mode label appears twice in one tensor";
            return PlanStatus::UNSUPPORTED_SHAPE;
        }
        for(const TensorIn* t : {&A, &B, &D})
            for(int64_t l : t->len)
                if(l <= 0)
                {
                    why = "a mode has extent 0";
                    return PlanStatus::UNSUPPORTED_SHAPE;
                }

        // Strides: the kernels address with unsigned 32-bit element offsets from each tensor's
        // base, so a negative stride would reach outside the tensor; D must not map two indices
        // of a mode onto one element (several work-items would write it).  Extents whose product
        // overflows cannot be a tensor of fewer than 2^31 elements either.
        for(const TensorIn* t : {&A, &B, &D, &C})
        {
            if(t == &C && !in.bilinear)
                continue;
            int64_t total = 1;
            for(size_t i = 0; i < t->len.size(); i++)
            {
                if(t->stride[i] < 0)
                {
                    why = "a stride is negative";
                    return PlanStatus::INVALID;
                }
                if(t == &D && t->stride[i] == 0 && t->len[i] > 1)
                {
                    why = "a mode of D of extent > 1 has stride 0";
                    return PlanStatus::INVALID;
                }
                if(__builtin_mul_overflow(total, t->len[i], &total))
                {
                    why = "a tensor's extents overflow 64 bits";
                    return PlanStatus::UNSUPPORTED_SHAPE;
                }
            }
        }

        // ---- classify modes: M = D and A, N = D and B, K = A and B ----
        struct Raw
        {
            int64_t len, sa, sb, sc, sd;
        };
        std::vector<Raw> M, N, K;
        for(size_t i = 0; i < D.mode.size(); i++)
        {
            const int ia = find_mode(A.mode, D.mode[i]);
            const int ib = find_mode(B.mode, D.mode[i]);
            if(ia >= 0 && ib >= 0)
            {
                why = "a mode appears in A, B and D (batch modes are not part of this path)";
                return PlanStatus::UNSUPPORTED_SHAPE;
            }
            if(ia < 0 && ib < 0)
            {
                why = "a mode of D appears in neither A nor B";
                return PlanStatus::INVALID;
            }
            const int64_t len = ia >= 0 ? A.len[(size_t)ia] : B.len[(size_t)ib];
            if(len != D.len[i] || (in.bilinear && C.len[i] != D.len[i]))
            {
                why = "extent of an output mode differs between tensors";
                return PlanStatus::INVALID;
            }
            Raw r{len, 0, 0, in.bilinear ? C.stride[i] : 0, D.stride[i]};
            if(ia >= 0)
            {
                r.sa = A.stride[(size_t)ia];
                M.push_back(r);
            }
            else
            {
                r.sb = B.stride[(size_t)ib];
                N.push_back(r);
            }
        }
        for(size_t i = 0; i < A.mode.size(); i++)
        {
            const int ib = find_mode(B.mode, A.mode[i]);
            if(ib < 0 || find_mode(D.mode, A.mode[i]) >= 0)
                continue; // modes held by A alone are read at index 0, as the reference does
            if(A.len[i] != B.len[(size_t)ib])
            {
                why = "extent of a contracted mode differs between A and B";
                return PlanStatus::INVALID;
            }
            K.push_back(Raw{A.len[i], A.stride[i], B.stride[(size_t)ib], 0, 0});
        }

        // ---- orientation: q must be the index D is contiguous in ----
        auto min_sd = [](const std::vector<Raw>& g) {
            int64_t best = INT64_MAX;
            for(const Raw& r : g)
                if(r.len > 1)
                    best = std::min(best, r.sd);
            return best;
        };
        v.swapped = min_sd(M) < min_sd(N);

        const std::vector<Raw>& Pg = v.swapped ? N : M;
        const std::vector<Raw>& Qg = v.swapped ? M : N;
        for(const Raw& r : Pg)
            if(r.len > 1)
                v.pdims.push_back(Dim{r.len, v.swapped ? r.sb : r.sa, 0, r.sc, r.sd});
        for(const Raw& r : Qg)
            if(r.len > 1)
                v.qdims.push_back(Dim{r.len, 0, v.swapped ? r.sa : r.sb, r.sc, r.sd});
        for(const Raw& r : K)
            if(r.len > 1)
                v.kdims.push_back(Dim{r.len, v.swapped ? r.sb : r.sa, v.swapped ? r.sa : r.sb, 0, 0});

        // ---- order (fastest first) and fuse ----
        std::stable_sort(v.qdims.begin(), v.qdims.end(), [](const Dim& a, const Dim& b) {
            return a.sd != b.sd ? a.sd < b.sd : a.sy < b.sy;
        });
        std::stable_sort(v.pdims.begin(), v.pdims.end(), [](const Dim& a, const Dim& b) {
            return a.sx != b.sx ? a.sx < b.sx : a.sd < b.sd;
        });
        {
            // K order follows the operand that is contiguous along a K mode; X wins a tie.
            bool x_has = false, y_has = false;
            for(const Dim& d : v.kdims)
            {
                x_has |= d.sx == 1;
                y_has |= d.sy == 1;
            }
            const bool by_y = !x_has && y_has;
            std::stable_sort(v.kdims.begin(), v.kdims.end(), [by_y](const Dim& a, const Dim& b) {
                const int64_t ka = by_y ? a.sy : a.sx, kb = by_y ? b.sy : b.sx;
                return ka != kb ? ka < kb : (by_y ? a.sx < b.sx : a.sy < b.sy);
            });
        }
        fuse(v.pdims, GP, in.bilinear);
        fuse(v.qdims, GQ, in.bilinear);
        fuse(v.kdims, GK, in.bilinear);
        v.P = extent(v.pdims);
        v.Q = extent(v.qdims);
        v.K = extent(v.kdims);
        // every folded extent gets an int32 offset table on the host and on the device
        if(v.P > (1ll << 28) || v.Q > (1ll << 28) || v.K > (1ll << 28))
        {
            why = "a folded extent exceeds 2^28 (offset tables would not fit)";
            return PlanStatus::UNSUPPORTED_SHAPE;
        }

        if(v.kdims.size() <= 1)
        {
            v.k_affine  = 1;
            v.xk_stride = v.kdims.empty() ? 0 : v.kdims[0].sx;
            v.yk_stride = v.kdims.empty() ? 0 : v.kdims[0].sy;
            if(v.xk_stride > 0x7FFFFFFFll || v.yk_stride > 0x7FFFFFFFll)
                v.k_affine = 0;
        }

        if(v.pdims.size() <= 1 && v.qdims.size() <= 1)
        {
            v.cd_affine = 1;
            v.dp_stride = v.pdims.empty() ? 0 : v.pdims[0].sd;
            v.cp_stride = v.pdims.empty() ? 0 : v.pdims[0].sc;
            v.dq_stride = v.qdims.empty() ? 0 : v.qdims[0].sd;
            v.cq_stride = v.qdims.empty() ? 0 : v.qdims[0].sc;
            v.xp_stride = v.pdims.empty() ? 0 : v.pdims[0].sx;
            v.yq_stride = v.qdims.empty() ? 0 : v.qdims[0].sy;
            for(int64_t st : {v.dp_stride, v.dq_stride, v.cp_stride, v.cq_stride})
                if(st > 0x7FFFFFFFll)
                    v.cd_affine = 0;
            if(v.xp_stride > 0x7FFFFFFFll || v.yq_stride > 0x7FFFFFFFll || !v.cd_affine)
                v.xp_stride = v.yq_stride = 0;
        }

        // ---- gather direction and vector width per operand ----
        const int maxv = class_max_vec(v.cls);
        // f32 (4 elements in 16 bytes): the register-staged kernels also gather both operands in pairs
        const bool half_vectors = v.cls == HIPTK_F32;
        auto pick = [&](bool use_x, const std::vector<Dim>& rows, int& kfast, int& vec, bool& ragged) {
            int  vk = 1, vr = 1;
            bool rr = false;
            // (a ragged K needs no flag: the kernels' last K tile handles a straddling vector)
            bool kr = false;
            if(!v.kdims.empty() && (use_x ? v.kdims[0].sx : v.kdims[0].sy) == 1)
                vk = vector_width(v.kdims[0].len, v.kdims.size() == 1, maxv, &kr, 2 * maxv);
            if(!rows.empty() && (use_x ? rows[0].sx : rows[0].sy) == 1)
                vr = vector_width(rows[0].len, rows.size() == 1, maxv, &rr);
            // the wide classes are instantiated for full-width vectors and for scalars; f32 also for
            // 8-byte vectors and the 16-bit classes for 8- and 4-byte vectors (narrowed jointly below)
            if(maxv != 8 && !half_vectors)
            {
                if(vk < maxv)
                    vk = 1;
                if(vr < maxv)
                    vr = 1;
            }
            if(vr > vk)
            {
                kfast  = 0;
                vec    = vr;
                ragged = rr;
            }
            else
            {
                kfast  = 1;
                vec    = vk;
                ragged = false;
            }
        };
        bool xRagged = false, yRagged = false, cdRagged = false;
        pick(true, v.pdims, v.x_kfast, v.x_vec, xRagged);
        pick(false, v.qdims, v.y_kfast, v.y_vec, yRagged);
        if(maxv == 8 && !(v.x_vec == 8 && v.y_vec == 8))
        {
            // 16-bit kernels exist for (8,8), (4,4), (2,2), (1,8), (8,1) and (1,1) elements per
            // vector of (X, Y): narrow the pair to the widest of those both operands admit.  A
            // narrower vector along the same direction is always valid.
            if(v.x_vec >= 2 && v.y_vec >= 2)
                v.x_vec = v.y_vec = std::min(v.x_vec, v.y_vec);
            else
            {
                // scalar gathers are staged k-fast
                if(v.x_vec < 8)
                {
                    v.x_vec   = 1;
                    v.x_kfast = 1;
                    xRagged   = false;
                }
                if(v.y_vec < 8)
                {
                    v.y_vec   = 1;
                    v.y_kfast = 1;
                    yRagged   = false;
                }
            }
        }
        if(half_vectors && !(v.x_vec == maxv && v.y_vec == maxv) && !(v.x_vec == 1 && v.y_vec == 1))
        {
            // f32 kernels exist for (4,4), (4,1), (1,4), (1,1) and (2,2) elements per vector of (X, Y)
            if(v.x_vec >= 2 && v.y_vec >= 2)
                v.x_vec = v.y_vec = 2;
            else
            {
                // scalar gathers are staged k-fast
                if(v.x_vec < maxv)
                {
                    v.x_vec   = 1;
                    v.x_kfast = 1;
                    xRagged   = false;
                }
                if(v.y_vec < maxv)
                {
                    v.y_vec   = 1;
                    v.y_kfast = 1;
                    yRagged   = false;
                }
            }
        }
        v.cd_vec = 1;
        if(!v.qdims.empty() && v.qdims[0].sd == 1 && (!in.bilinear || v.qdims[0].sc == 1))
            v.cd_vec = vector_width(v.qdims[0].len, v.qdims.size() == 1, maxv, &cdRagged);
        v.shift_p = xRagged ? 1 : 0;
        v.shift_q = (yRagged || cdRagged) ? 1 : 0;

        // ---- offset tables ----
        // Row / column tables cover every index a tile may overhang to: the largest tile edge is
        // 256 and need not divide 256 (192-wide tiles), so one extra 256 beyond the rounded
        // extent; the pad value 0 is the offset of row 0, a valid element.  The k tables get
        // the same: the kernels read k offsets up to three K tiles ahead.
        auto padded = [](int64_t n) { return (size_t)((n + 255) / 256 * 256 + 256); };
        int64_t mxp, mxk, myq, myk, mcp, mcq, mdp, mdq;
        bool    ok = true;
        ok &= make_table(v.pdims, v.P, padded(v.P), [](const Dim& d) { return d.sx; }, v.xp, mxp);
        ok &= make_table(v.kdims, v.K, padded(v.K), [](const Dim& d) { return d.sx; }, v.xk, mxk);
        ok &= make_table(v.qdims, v.Q, padded(v.Q), [](const Dim& d) { return d.sy; }, v.yq, myq);
        ok &= make_table(v.kdims, v.K, padded(v.K), [](const Dim& d) { return d.sy; }, v.yk, myk);
        ok &= make_table(v.pdims, v.P, padded(v.P), [](const Dim& d) { return d.sd; }, v.dp, mdp);
        ok &= make_table(v.qdims, v.Q, padded(v.Q), [](const Dim& d) { return d.sd; }, v.dq, mdq);
        if(in.bilinear)
        {
            ok &= make_table(v.pdims, v.P, padded(v.P), [](const Dim& d) { return d.sc; }, v.cp, mcp);
            ok &= make_table(v.qdims, v.Q, padded(v.Q), [](const Dim& d) { return d.sc; }, v.cq, mcq);
        }
        else
            mcp = mcq = 0;
        const int64_t lim = 0x7FFFFFFFll;
        if(!ok || mxp + mxk > lim || myq + myk > lim || mcp + mcq > lim || mdp + mdq > lim)
        {
            why = "a tensor spans more than 2^31 elements";
            return PlanStatus::UNSUPPORTED_SHAPE;
        }

        v.x_max_off = mxp + mxk;
        v.y_max_off = myq + myk;
        // 16-byte vectors that start on 16-byte multiples of the tensor's base
        {
            const int want = v.elem_bytes >= 1 && v.elem_bytes <= 16 ? 16 / v.elem_bytes : 0;
            auto aligned = [want](const std::vector<int32_t>& rows, int64_t nrows, const std::vector<int32_t>& ks, int64_t nk,
                                  bool kfast, int vec, bool shifted) {
                if(want == 0 || vec != want || (!kfast && shifted))
                    return false;
                for(int64_t r = 0; r < nrows; r += kfast ? 1 : vec)
                    if(rows[(size_t)r] % vec != 0)
                        return false;
                for(int64_t k = 0; k < nk; k += kfast ? vec : 1)
                    if(ks[(size_t)k] % vec != 0)
                        return false;
                return true;
            };
            v.xy_aligned = (aligned(v.xp, v.P, v.xk, v.K, v.x_kfast != 0, v.x_vec, v.shift_p != 0)
                            && aligned(v.yq, v.Q, v.yk, v.K, v.y_kfast != 0, v.y_vec, v.shift_q != 0))
                               ? 1
                               : 0;
        }

        // k-contiguous operand: which neighbour of a vector is its neighbour in memory too, the next row's or the next
        // vector of its own row?
        {
            auto rows_adjacent = [](const std::vector<int32_t>& rows, int64_t nrows, const std::vector<int32_t>& ks, int64_t nk, bool kfast, int vec) {
                if(!kfast || vec < 2 || nrows < 2)
                    return 0;
                int64_t by_row = 0, by_k = 0, k_pairs = 0;
                for(int64_t r = 0; r + 1 < nrows; r++)
                    by_row += (int64_t)rows[(size_t)r + 1] - rows[(size_t)r] == vec;
                for(int64_t k = 0; k + vec < nk; k += vec, k_pairs++)
                    by_k += (int64_t)ks[(size_t)(k + vec)] - ks[(size_t)k] == vec;
                // (as fractions of the pairs there are)
                return by_row * (k_pairs > 0 ? k_pairs : 1) > by_k * (nrows - 1) ? 1 : 0;
            };
            v.x_rows_adjacent = rows_adjacent(v.xp, v.P, v.xk, v.K, v.x_kfast != 0, v.x_vec);
            v.y_rows_adjacent = rows_adjacent(v.yq, v.Q, v.yk, v.K, v.y_kfast != 0, v.y_vec);
        }

        v.spanA = span_elems(A.len, A.stride);
        v.spanB = span_elems(B.len, B.stride);
        v.spanD = span_elems(D.len, D.stride);
        v.spanC = in.bilinear ? span_elems(C.len, C.stride) : 0;
        return PlanStatus::OK;
    }
}
