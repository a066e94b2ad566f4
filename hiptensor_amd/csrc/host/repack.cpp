#include "repack.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <limits>

#include "permute_plan.hpp"

namespace hipta
{
    namespace
    {
        struct ModeRef
        {
            int32_t label;
            int64_t len, stride;
        };

        int find_label(const std::vector<int32_t>& modes, int32_t label)
        {
            for(size_t i = 0; i < modes.size(); i++)
                if(modes[i] == label)
                    return (int)i;
            return -1;
        }

        // The modes of `t` longer than one element, fastest first; false unless they tile the
        // tensor's memory without gaps (the permutation kernels read a packed source).
        bool dense_modes(const TensorIn& t, std::vector<ModeRef>& out)
        {
            out.clear();
            for(size_t i = 0; i < t.mode.size(); i++)
                if(t.len[i] > 1)
                    out.push_back(ModeRef{t.mode[i], t.len[i], t.stride[i]});
            std::stable_sort(out.begin(), out.end(), [](const ModeRef& a, const ModeRef& b) { return a.stride < b.stride; });
            int64_t run = 1;
            for(const ModeRef& m : out)
            {
                if(m.stride != run)
                    return false;
                run *= m.len;
            }
            return true;
        }

        uint64_t round_up(uint64_t n, uint64_t a)
        {
            return (n + a - 1) / a * a;
        }

        // label no caller's mode list is likely to hold: the 4-byte words of a wider element
        constexpr int32_t WORD_LABEL = std::numeric_limits<int32_t>::min() + 7;

        // Plans the move of operand `t` (modes in `src`, fastest first) into a packed copy whose
        // modes run in `order` (fastest first).  False when the permutation kernels do not take it.
        bool plan_pack(const TensorIn& t, const std::vector<ModeRef>& src, const std::vector<ModeRef>& order, int elem_bytes, PackedOperand& po, TensorIn& packed)
        {
            PermuteIn pin;
            pin.elem_bytes = elem_bytes >= 4 ? 4 : 2;
            const int words = elem_bytes / pin.elem_bytes; // a wider element moves as 2 or 4 words
            if(words > 1)
            {
                pin.lenA.push_back(words);
                pin.modeA.push_back(WORD_LABEL);
                pin.lenB.push_back(words);
                pin.modeB.push_back(WORD_LABEL);
            }
            int64_t count = 1;
            for(const ModeRef& m : src)
            {
                if(m.label == WORD_LABEL)
                    return false;
                pin.lenA.push_back(m.len);
                pin.modeA.push_back(m.label);
                count *= m.len;
            }
            for(const ModeRef& m : order)
            {
                pin.lenB.push_back(m.len);
                pin.modeB.push_back(m.label);
            }
            // only the alignment of the two addresses enters the plan: the source is aligned as
            // its descriptor promised, the copy starts at a 256-byte boundary
            const uintptr_t alignA = std::max<uintptr_t>(t.align ? t.align : (uintptr_t)elem_bytes, (uintptr_t)pin.elem_bytes);
            pin.A                  = reinterpret_cast<const void*>(alignA);
            pin.B                  = reinterpret_cast<const void*>((uintptr_t)PACK_ALIGN);
            if(plan_permutation(pin, PermuteTuning{}, po.perm) != PermuteStatus::OK)
                return false;
            if(po.perm.rank < 2)
                return false; // already in that order: nothing a copy would change
            po.perm.alpha = 1.0f;
            po.perm.op_a  = HIPTK_PERM_OP_RAW;
            po.perm.op_b  = 0;
            po.on         = true;
            const double raw = (double)count * elem_bytes;
            po.bytes         = round_up((uint64_t)raw, PACK_ALIGN);
            // read once, written once, plus a launch.  Measured on operands of 10-20 MB with runs of
            // 15 elements: the element-wise fallback moves 1.2 (2-byte) to 2.0 TB/s (4-byte), the
            // tile kernels 1.6-3.2 TB/s (5-6 TB/s on large tensors with long runs)
            const double rate = po.perm.kernel == HIPTK_PERM_GATHER ? (pin.elem_bytes == 2 ? 1.2e6 : 2.0e6) : 2.5e6; // bytes / us
            po.est_us         = 2.0 * raw / rate + 3.0;

            packed       = t;
            packed.align = (uint32_t)PACK_ALIGN;
            packed.len.clear();
            packed.stride.clear();
            packed.mode.clear();
            int64_t run = 1;
            for(const ModeRef& m : order)
            {
                packed.mode.push_back(m.label);
                packed.len.push_back(m.len);
                packed.stride.push_back(run);
                run *= m.len;
            }
            for(size_t i = 0; i < t.mode.size(); i++)
                if(t.len[i] == 1)
                {
                    packed.mode.push_back(t.mode[i]);
                    packed.len.push_back(1);
                    packed.stride.push_back(run);
                }
            return true;
        }

        struct OperandModes
        {
            bool                 eligible = false;
            std::vector<ModeRef> src; // as stored, fastest first
            std::vector<ModeRef> outer, inner; // free modes (also in D), contracted modes (also in the other operand)
        };

        OperandModes classify(const TensorIn& t, const TensorIn& other, const TensorIn& D)
        {
            OperandModes o;
            if(!dense_modes(t, o.src) || o.src.size() < 2)
                return o;
            for(const ModeRef& m : o.src)
            {
                const bool inD = find_label(D.mode, m.label) >= 0, inO = find_label(other.mode, m.label) >= 0;
                if(inD == inO)
                    return o; // a mode held by this operand alone is read at index 0: not a dense source
                (inD ? o.outer : o.inner).push_back(m);
            }
            o.eligible = true;
            return o;
        }

        int64_t stride_in(const TensorIn& t, int32_t label)
        {
            const int i = find_label(t.mode, label);
            return i < 0 ? 0 : t.stride[(size_t)i];
        }

        void sort_by(std::vector<ModeRef>& ms, const TensorIn& ref)
        {
            std::stable_sort(ms.begin(), ms.end(), [&ref](const ModeRef& a, const ModeRef& b) {
                return stride_in(ref, a.label) < stride_in(ref, b.label);
            });
        }
    }

    RepackMode repack_mode_from_env()
    {
        const char* e = std::getenv("HIPTENSOR_AMD_REPACK");
        if(e && (!std::strcmp(e, "0") || !std::strcmp(e, "off")))
            return RepackMode::OFF;
        if(e && (!std::strcmp(e, "1") || !std::strcmp(e, "force")))
            return RepackMode::FORCE;
        return std::getenv("HIPTENSOR_AMD_FORCE_KERNEL") ? RepackMode::OFF : RepackMode::AUTO;
    }

    PlanStatus plan_contraction(const ProblemIn&                    in,
                                const std::vector<const Solution*>& candidates,
                                uint64_t                            max_ws,
                                uint64_t                            split_cap,
                                const DeviceModel&                  dev,
                                RepackMode                          mode,
                                ContractionPlanChoice&              out,
                                std::string&                        why)
    {
        out         = ContractionPlanChoice();
        out.problem = in;
        if(PlanStatus st = build_view(in, out.view, why); st != PlanStatus::OK)
            return st;
        out.ranked = rank_choices(candidates, out.view, std::min(max_ws, split_cap), dev);
        if(mode == RepackMode::OFF || out.ranked.empty())
            return PlanStatus::OK;
        const int maxv = class_max_vec(out.view.cls);
        if(maxv <= 1 || max_ws <= PACK_ALIGN)
            return PlanStatus::OK;
        if(mode == RepackMode::AUTO && std::min(out.view.x_vec, out.view.y_vec) >= maxv)
            return PlanStatus::OK; // both operands already arrive in whole vectors

        const OperandModes ma = classify(in.A, in.B, in.D), mb = classify(in.B, in.A, in.D);
        if(!ma.eligible && !mb.eligible)
            return PlanStatus::OK;
        const int    es        = out.view.elem_bytes;
        const double base_us   = out.ranked.front().est_us;
        double       best_us   = 0.0;
        bool         have_best = false;
        ContractionPlanChoice best;
        // 0: as it lies, 1: packed with its free modes fastest, 2: packed with the contracted modes fastest
        for(int ca = 0; ca < 3; ca++)
            for(int cb = 0; cb < 3; cb++)
            {
                if((ca == 0 && cb == 0) || (ca && !ma.eligible) || (cb && !mb.eligible))
                    continue;
                ContractionPlanChoice alt;
                alt.problem = in;
                // the contracted modes run in one order in both copies, so that they fuse: the order
                // of the operand that stays, else A's
                const TensorIn& kref = ca == 0 ? in.A : cb == 0 ? in.B : in.A;
                bool            ok   = true;
                for(int side = 0; side < 2 && ok; side++)
                {
                    const int c = side == 0 ? ca : cb;
                    if(!c)
                        continue;
                    const OperandModes&  m     = side == 0 ? ma : mb;
                    std::vector<ModeRef> outer = m.outer, inner = m.inner, order;
                    sort_by(outer, in.D);
                    sort_by(inner, kref);
                    const std::vector<ModeRef>& first = c == 1 ? outer : inner;
                    const std::vector<ModeRef>& then  = c == 1 ? inner : outer;
                    order.insert(order.end(), first.begin(), first.end());
                    order.insert(order.end(), then.begin(), then.end());
                    ok = plan_pack(side == 0 ? in.A : in.B, m.src, order, es, side == 0 ? alt.a : alt.b, side == 0 ? alt.problem.A : alt.problem.B);
                }
                if(!ok)
                    continue;
                alt.b.offset   = alt.a.on ? alt.a.bytes : 0;
                alt.pack_bytes = PACK_ALIGN + (alt.a.on ? alt.a.bytes : 0) + (alt.b.on ? alt.b.bytes : 0);
                if(alt.pack_bytes > max_ws)
                    continue;
                std::string ignored;
                if(build_view(alt.problem, alt.view, ignored) != PlanStatus::OK)
                    continue;
                alt.ranked = rank_choices(candidates, alt.view, std::min(max_ws - alt.pack_bytes, split_cap), dev);
                if(alt.ranked.empty())
                    continue;
                double us = alt.ranked.front().est_us + alt.a.est_us + alt.b.est_us;
                if(mode == RepackMode::FORCE)
                    us -= 1e9 * ((alt.a.on ? 1 : 0) + (alt.b.on ? 1 : 0)); // as many copies as the layouts admit
                if(!have_best || us < best_us)
                {
                    best      = std::move(alt);
                    best_us   = us;
                    have_best = true;
                }
            }
        // a packed plan has to promise a clear gain: the estimates are good to about ten percent
        if(have_best && (mode == RepackMode::FORCE || best_us < 0.9 * base_us))
            out = std::move(best);
        return PlanStatus::OK;
    }
}
