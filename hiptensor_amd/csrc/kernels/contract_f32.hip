// f32 kernels (v_mfma_f32_32x32x2_f32).
#include "contract_wd.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_W_TILE(WTraitsF32, 0, 128, 128, 16, 2, 4),
        HIPTK_W_TILE(WTraitsF32, 1, 64, 64, 16, 2, 2),
        HIPTK_W_TILE_HALF(WTraitsF32, 0, 128, 128, 16, 2, 4),
        HIPTK_W_TILE_HALF(WTraitsF32, 1, 64, 64, 16, 2, 2),
        HIPTK_WD_ENTRY(WTraitsF32, 2, 16, 4),
        HIPTK_WK_ENTRY(WTraitsF32, 3, 16, 4),
        HIPTK_WD_ENTRY_KF(WTraitsF32, 2, 16, 4, 1, 1),
        HIPTK_WK_ENTRY_KF(WTraitsF32, 3, 16, 4, 1, 1),
        HIPTK_WD_ENTRY_KF(WTraitsF32, 2, 16, 4, 1, 0),
        HIPTK_WK_ENTRY_KF(WTraitsF32, 3, 16, 4, 1, 0),
        HIPTK_WD_ENTRY_KF(WTraitsF32, 2, 16, 4, 0, 1),
        HIPTK_WK_ENTRY_KF(WTraitsF32, 3, 16, 4, 0, 1),
    };

    const KernelEntry* entries_f32(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
