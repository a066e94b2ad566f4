// bf16 kernels that load their operand tiles straight into LDS: 256 x 256 tile, affine K.
#include "contract_hd.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HD_TILE(TraitsBF16, 9, 256, true),
    };

    const KernelEntry* entries_bf16_hd(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
