// Kernel registry and selection.
//
// A Solution is one kernel family: an element class (f16, bf16, f32, f64, complex ...)
// at one workgroup tile.  The layout / vector variant inside a family is fixed by the
// planner, not chosen here.  The registry is what hiptensorInitContractionFind hands
// out as candidates (reference: ContractionSolutionInstances / ContractionSolutionRegistry,
// library/src/contraction/contraction_solution_registry.cpp:55-282), and choose() takes
// the place of both bruteForceModel and the "actor-critic" lookup tables
// (library/src/contraction/contraction_selection.cpp:44-195, 197-2214) with an
// analytic cost model of tiles over the device's compute units.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "hiptk_kernels.h"
#include "planner.hpp"

namespace hipta
{
    struct Solution
    {
        uint64_t    uid; // stable id: hash of (class, tile shape)
        int         cls, tile_id;
        int         bp, bq, bk, threads, lds_bytes;
        bool        direct; // operand tiles go from global memory straight into LDS
        int         mfma_k; // 32: a 16-bit tile on v_mfma_f32_16x16x32 (else 0)
        std::string name;
    };

    struct DeviceModel
    {
        int    cus        = 256;
        double clock_ghz  = 2.4;
        double hbm_gbs    = 8000.0;
        int    lds_per_cu = 163840;
    };

    struct Choice
    {
        const Solution* sol      = nullptr;
        int             split_k  = 1;
        double          est_us   = 0.0;
        uint64_t        ws_bytes = 0;
    };

    class SolutionRegistry
    {
    public:
        static const SolutionRegistry& get();
        const std::vector<Solution>&   all() const { return mAll; }
        std::vector<const Solution*>   forClass(int cls) const;
        const Solution*                byUid(uint64_t uid) const;

    private:
        SolutionRegistry();
        std::vector<Solution> mAll;
    };

    // Is there a kernel of this family for the view's layout / vector combination?
    bool solution_fits(const Solution& s, const GemmView& v);

    // Estimated run time in microseconds of `s` on `v` with `split` K slices.
    double estimate_us(const Solution& s, const GemmView& v, int split, const DeviceModel& dev);

    // Ranks (solution, split) pairs among `candidates` (restricted to the view's class)
    // by estimate; `max_ws` bounds the workspace split-K may use.  Best first.
    std::vector<Choice> rank_choices(const std::vector<const Solution*>& candidates,
                                     const GemmView&                     v,
                                     uint64_t                            max_ws,
                                     const DeviceModel&                  dev);

    // MFMA flop per clock per CU of a class (dense peak), for estimates and reports.
    double class_flops_per_clk_cu(int cls);
    // real flops per (p, q, k) triple: 2, or 8 for the complex classes
    double class_flops_per_mac(int cls);
    int    class_acc_bytes(int cls);
}
