// f16 kernels that load their operand tiles straight into LDS: 256 x 256 tile, K offsets from tables.
#include "contract_hd.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HD_TILE(TraitsF16, 9, 256, false),
    };

    const KernelEntry* entries_f16_hd_tab(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
