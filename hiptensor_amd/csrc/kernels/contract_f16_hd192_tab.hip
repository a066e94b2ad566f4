// f16 kernels that load their operand tiles straight into LDS: 256 x 192 tile, K offsets from tables.
#include "contract_hd.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HD_TILE(TraitsF16, 10, 192, false),
    };

    const KernelEntry* entries_f16_hd192_tab(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
