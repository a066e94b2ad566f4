// Host-side planning of a tensor permutation: checks the two mode lists against each other,
// fuses modes that stay adjacent, and picks the kernel, tile shape and vector widths.
// Pure host logic (no HIP calls), so it can be exercised without a device.
//
// Layout rule of the reference (library/src/permutation/permutation_solution_impl.hpp:117-132):
// both tensors are packed with their first listed mode fastest, whatever strides the
// descriptors hold.
#pragma once
#include <cstdint>
#include <vector>

#include "hiptk_kernels.h"

namespace hipta
{
    struct PermuteIn
    {
        int                  elem_bytes = 4; // 2: f16, 4: f32
        std::vector<int64_t> lenA, lenB;
        std::vector<int32_t> modeA, modeB;
        const void*          A = nullptr; // only the alignment of the two addresses is used
        const void*          B = nullptr;
    };

    enum class PermuteStatus
    {
        OK,
        EMPTY, // an extent is zero: nothing to do
        BAD_RANK, // ranks differ, or more than HIPTK_PERM_MAX_RANK modes are left after fusion
        BAD_MODES, // modeB is not a reordering of modeA, or a length disagrees
        TOO_LARGE // 2^31 elements or more
    };

    // Preferences a test or an experiment can impose (environment, see permutation.cpp).
    struct PermuteTuning
    {
        int kernel  = -1; // HIPTK_PERM_* to use wherever the layout admits it, -1: automatic
        int tile    = -1; // 0..2, -1: automatic
        int max_vec = 8; // cap on elements per load / store
        int group   = -1; // tiles per band of the workgroup order, -1: automatic
    };

    // Fills `out` (alpha and the operators are left for the caller); out.rank is the number of
    // modes left after extent-1 modes were dropped and neighbours fused.
    PermuteStatus plan_permutation(const PermuteIn& in, const PermuteTuning& tune, hiptk_permute_t& out);
}
