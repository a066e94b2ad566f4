// f64 kernels (v_mfma_f64_16x16x4_f64).
#include "contract_wd.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_W_TILE(WTraitsF64, 0, 128, 128, 16, 2, 4),
        HIPTK_W_TILE(WTraitsF64, 1, 64, 64, 16, 4, 2),
        HIPTK_WD_ENTRY(WTraitsF64, 2, 8, 4),
        HIPTK_WK_ENTRY(WTraitsF64, 3, 8, 4),
        HIPTK_WD_ENTRY_KF(WTraitsF64, 2, 8, 4, 1, 1),
        HIPTK_WK_ENTRY_KF(WTraitsF64, 3, 8, 4, 1, 1),
        HIPTK_WD_ENTRY_KF(WTraitsF64, 2, 8, 4, 1, 0),
        HIPTK_WK_ENTRY_KF(WTraitsF64, 3, 8, 4, 1, 0),
        HIPTK_WD_ENTRY_KF(WTraitsF64, 2, 8, 4, 0, 1),
        HIPTK_WK_ENTRY_KF(WTraitsF64, 3, 8, 4, 0, 1),
    };

    const KernelEntry* entries_f64(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
