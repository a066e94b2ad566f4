// f16 kernels whose operands are gathered as 4-byte vectors (2 elements): problems whose
// contiguous runs or alignment do not admit the full 16 bytes.  Table-driven k offsets.
#include "contract_h.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HP_TILE_VV(TraitsF16, 1, 128, 128, 64, 2, 4, 2, false),
        HIPTK_H_TILE_VV(TraitsF16, 2, 64, 64, 64, 2, 2, 2, false),
    };

    const KernelEntry* entries_f16_v2(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
