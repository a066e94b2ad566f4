// complex f64 kernels (two v_mfma_f64_16x16x4_f64 per two complex k).
#include "contract_w.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_W_TILE(WTraitsC64, 0, 64, 64, 8, 4, 2),
        HIPTK_W_TILE(WTraitsC64, 1, 32, 32, 8, 2, 2),
        HIPTK_W_TILE(WTraitsC64, 2, 128, 128, 8, 2, 4),
    };

    const KernelEntry* entries_c64(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
