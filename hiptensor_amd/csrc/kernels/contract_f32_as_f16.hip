// f32 tensors contracted with f16 arithmetic: operands are rounded to f16 as they are staged
// into LDS, products accumulate in f32, results are f32.  16-byte gathers (4 elements) or
// scalar gathers; k offsets always from the tables.
#include "contract_h.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HP_TILE_VV(TraitsF32AsF16, 0, 128, 128, 64, 2, 4, 4, false),
        HIPTK_H_TILE_VV(TraitsF32AsF16, 1, 64, 64, 64, 2, 2, 4, false),
        HIPTK_H_TILE_V1V(TraitsF32AsF16, 2, 128, 128, 32, 2, 2, 4),
        HIPTK_H_TILE_V1V(TraitsF32AsF16, 3, 64, 64, 32, 2, 2, 4),
        HIPTK_H_TILE_VV(TraitsF32AsF16, 4, 256, 256, 64, 2, 4, 4, false),
    };

    const KernelEntry* entries_f32_as_f16(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
