// complex f32 kernels (two v_mfma_f32_32x32x2_f32 per complex k).
#include "contract_wd.hpp"

namespace hiptk
{
    // (the 64 x 64 direct-load tile keeps a ring of 8 K tiles here: its 230 registers a lane leave a CU two
    // workgroups whatever the LDS, and with a ring of 4 the same two cover less: 2048^2 x 1024 240 -> 291 us)
    static const KernelEntry k_entries[] = {
        HIPTK_W_TILE(WTraitsC32, 0, 128, 128, 8, 2, 4),
        HIPTK_W_TILE(WTraitsC32, 1, 64, 64, 8, 2, 2),
        HIPTK_WD_ENTRY(WTraitsC32, 2, 8, 8),
        HIPTK_WK_ENTRY(WTraitsC32, 3, 8, 4),
        HIPTK_WD_ENTRY_KF(WTraitsC32, 2, 8, 8, 1, 1),
        HIPTK_WK_ENTRY_KF(WTraitsC32, 3, 8, 4, 1, 1),
        HIPTK_WD_ENTRY_KF(WTraitsC32, 2, 8, 8, 1, 0),
        HIPTK_WK_ENTRY_KF(WTraitsC32, 3, 8, 4, 1, 0),
        HIPTK_WD_ENTRY_KF(WTraitsC32, 2, 8, 8, 0, 1),
        HIPTK_WK_ENTRY_KF(WTraitsC32, 3, 8, 4, 0, 1),
    };

    const KernelEntry* entries_c32(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
