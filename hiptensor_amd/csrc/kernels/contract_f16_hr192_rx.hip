// f16 kernels on v_mfma_f32_16x16x32 with operand tiles loaded straight into a ring of four LDS stages in K tiles of 32:
// 256 x 192 tile, k offsets from tables, X row-contiguous.
#include "contract_hr.hpp"

namespace hiptk
{
    static const KernelEntry k_entries[] = {
        HIPTK_HR_ENTRY(TraitsF16, 12, 192, false, true),
        HIPTK_HR_ENTRY(TraitsF16, 12, 192, false, false),
    };

    const KernelEntry* entries_f16_hr192_rx(int* count)
    {
        *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
        return k_entries;
    }
}
