// bf16 kernels whose operands are gathered as 8-byte vectors (4 elements): problems whose
// contiguous runs or alignment do not admit the full 16 bytes.  Table-driven k offsets.
#include "contract_h.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_H_TILE_VV(TraitsBF16, 0, 256, 256, 64, 2, 4, 4, false),
        HIPTK_HP_TILE_VV(TraitsBF16, 1, 128, 128, 64, 2, 4, 4, false),
        HIPTK_H_TILE_VV(TraitsBF16, 2, 64, 64, 64, 2, 2, 4, false),
    };

    const KernelEntry* entries_bf16_v4(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
