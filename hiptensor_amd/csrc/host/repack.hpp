// Packed copies of contraction operands.
//
// An operand whose modes are interleaved so that neither its row index nor its reduction
// index has contiguous runs of a whole vector can only be gathered element by element, which
// costs the matrix kernels a factor of two to four.  Where the caller grants workspace, the
// plan may instead first move such an operand into a packed copy (the permutation kernels
// move it at memory speed, a few percent of the contraction's time) and contract the copy
// with the vector kernels.  The reference has no such step (its kernels read every layout
// through Composable Kernel's descriptors, library/src/contraction/contraction_solution_impl.hpp:
// 80-203); the decision is the cost model's and the result is the same contraction.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "hiptk_kernels.h"
#include "planner.hpp"
#include "solution.hpp"

namespace hipta
{
    struct PackedOperand
    {
        bool            on = false;
        hiptk_permute_t perm{}; // operand as given -> packed copy (a raw move)
        uint64_t        bytes  = 0; // size of the copy, a multiple of 256
        uint64_t        offset = 0; // where it sits in the (256-byte aligned) workspace
        double          est_us = 0.0;
    };

    enum class RepackMode
    {
        OFF, // contract the operands where they lie
        AUTO, // pack where the cost model expects a clear gain
        FORCE // pack wherever the layout admits it (tests)
    };

    struct ContractionPlanChoice
    {
        ProblemIn           problem; // A / B replaced by the layout of their packed copies
        GemmView            view;
        std::vector<Choice> ranked; // kernel choices for `view`, best first
        PackedOperand       a, b;
        uint64_t            pack_bytes = 0; // workspace taken by the copies (incl. alignment slack)
    };

    // Slack added to the workspace so that the copies can start at a 256-byte boundary.
    constexpr uint64_t PACK_ALIGN = 256;

    // Builds the GEMM view of `in` and ranks kernels for it; with mode != OFF also weighs the
    // alternatives in which A, B or both are first packed (row-fast or reduction-fast), within
    // `max_ws` bytes of workspace (`split_cap` bounds the part split-K may take).
    PlanStatus plan_contraction(const ProblemIn&                    in,
                                const std::vector<const Solution*>& candidates,
                                uint64_t                            max_ws,
                                uint64_t                            split_cap,
                                const DeviceModel&                  dev,
                                RepackMode                          mode,
                                ContractionPlanChoice&              out,
                                std::string&                        why);

    // HIPTENSOR_AMD_REPACK = 0 | off, 1 | force, auto (default).  A kernel pinned through
    // HIPTENSOR_AMD_FORCE_KERNEL keeps the operands where they lie unless packing is forced too.
    RepackMode repack_mode_from_env();
}
