// bf16 kernels on v_mfma_f32_16x16x32 with operand tiles loaded straight into LDS in K tiles of 64: 256 x 256 tile, X k-contiguous.
#include "contract_hk.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HK_ENTRY(TraitsBF16, 11, 256, true, true, 2, 2, 4),
        HIPTK_HK_ENTRY(TraitsBF16, 11, 256, true, false, 2, 2, 4),
    };

    const KernelEntry* entries_bf16_hk_kx(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
