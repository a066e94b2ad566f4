// bf16 kernels for problems in which an operand has no contiguous run of 8 elements
// (scalar gather).
#include "contract_h.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_H_TILE_V1(TraitsBF16, 3, 128, 128, 32, 2, 2),
        HIPTK_H_TILE_V1(TraitsBF16, 4, 64, 64, 32, 2, 2),
    };

    const KernelEntry* entries_bf16_gen(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
