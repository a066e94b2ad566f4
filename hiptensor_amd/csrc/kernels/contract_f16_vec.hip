// f16 kernels whose two operands are both gathered as 16-byte vectors, k offsets from
// the tables (several K modes that do not fuse).
#include "contract_h.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_H_TILE_V8(TraitsF16, 0, 256, 256, 64, 2, 4, false),
        HIPTK_H_TILE_V8(TraitsF16, 1, 128, 128, 64, 2, 2, false),
        HIPTK_H_TILE_V8(TraitsF16, 2, 64, 64, 64, 2, 2, false),
    };

    const KernelEntry* entries_f16_vec(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
