// complex f64 kernels (two v_mfma_f64_16x16x4_f64 per two complex k).
#include "contract_wd.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        // (K tiles of 16 on the 64 x 64 tile: 2048^2 x 1024 527 against 555 us with 8, 1920^2 x 768 406 against 432;
        // on the 32 x 32 tile they pay on short problems only: 512^3 26.6 against 31.2 us, 1920^2 x 768 391 against 375)
        HIPTK_W_TILE(WTraitsC64, 0, 64, 64, 16, 4, 2),
        HIPTK_W_TILE(WTraitsC64, 1, 32, 32, 8, 2, 2),
        HIPTK_W_TILE(WTraitsC64, 2, 32, 32, 16, 2, 2),
        // (one element per 16-byte vector: every layout with one K stride is "k-contiguous, vectors of one")
        HIPTK_WD_ENTRY_KF(WTraitsC64, 3, 8, 4, 1, 1),
        HIPTK_WK_ENTRY_KF(WTraitsC64, 4, 8, 4, 1, 1),
    };

    const KernelEntry* entries_c64(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
