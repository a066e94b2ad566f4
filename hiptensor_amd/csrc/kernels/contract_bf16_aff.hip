// bf16 kernels whose two operands are both gathered as 16-byte vectors and whose K modes
// fused into one stride per operand (k offsets are a multiply).
#include "contract_h.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_H_TILE_V8(TraitsBF16, 0, 256, 256, 64, 2, 4, true),
        HIPTK_H_TILE_V8(TraitsBF16, 1, 128, 128, 64, 2, 2, true),
        HIPTK_H_TILE_V8(TraitsBF16, 2, 64, 64, 64, 2, 2, true),
    };

    const KernelEntry* entries_bf16_aff(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
