// bf16 kernels whose two operands are both gathered as 16-byte vectors, k offsets from
// the tables (several K modes that do not fuse).
#include "contract_h.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HP_TILE_V8(TraitsBF16, 0, 256, 256, 64, 2, 4, false),
        HIPTK_HP_TILE_V8(TraitsBF16, 1, 128, 128, 64, 2, 4, false),
        HIPTK_H_TILE_V8(TraitsBF16, 2, 64, 64, 64, 2, 2, false),
        HIPTK_HP_TILE_V8(TraitsBF16, 5, 256, 128, 64, 4, 2, false),
        HIPTK_HP_TILE_V8(TraitsBF16, 6, 128, 256, 64, 2, 4, false),
        // 256 x 192: the 24 row vectors of a 192-row tile do not divide the workgroup, so only
        // the variants whose column operand is contiguous along k are built
        HIPTK_HP_ENTRY(TraitsBF16, 7, 256, 192, 64, 4, 2, true, true, 8, 8, false),
        HIPTK_HP_ENTRY(TraitsBF16, 7, 256, 192, 64, 4, 2, false, true, 8, 8, false),
        // 256 x 256 on four wavefronts (one per SIMD, wave tile 128 x 128, accumulators in AGPRs)
        HIPTK_HP_TILE_V8(TraitsBF16, 8, 256, 256, 64, 2, 2, false),
    };

    const KernelEntry* entries_bf16_vec(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
