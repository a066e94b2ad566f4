"""Host-side behaviour of hiptensorPermutation that needs no device: argument checks in the
reference's order (library/src/permutation/hiptensor_permutation.cpp:77-155, 173-189), mode
fusion and kernel choice of the planner."""
import ctypes as C

import pytest

import perm_cases
from hiptensor_amd import api
from hiptensor_amd import workloads as wl


def _descs(h, lens, perm, dtype=api.HIP_R_32F, dtypeB=None):
    modes = list(range(100, 100 + len(lens)))
    dA = api.check(api.hiptensorInitTensorDescriptor(h, lens, None, dtype), "dA")
    dB = api.check(api.hiptensorInitTensorDescriptor(h, [lens[p] for p in perm], None, dtype if dtypeB is None else dtypeB), "dB")
    return dA, modes, dB, [modes[p] for p in perm]


def test_null_arguments_are_not_initialized(host_handle):
    dA, mA, dB, mB = _descs(host_handle, [4, 5], [1, 0])
    one = C.c_float(1.0)
    good = [host_handle, one, 256, dA, mA, 512, dB, mB]
    for i in range(len(good)):
        args = list(good)
        args[i] = None
        st = api.hiptensorPermutation(*args, api.HIP_R_32F, None)
        assert st == api.HIPTENSOR_STATUS_NOT_INITIALIZED, i


def test_type_checks_in_reference_order(host_handle):
    one = C.c_float(1.0)
    # data type other than f16 / f32: NOT_SUPPORTED, before the A/B mismatch check
    dA, mA, dB, mB = _descs(host_handle, [4, 5], [1, 0], api.HIP_R_64F, api.HIP_R_32F)
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB, mB, api.HIP_R_32F, None) == api.HIPTENSOR_STATUS_NOT_SUPPORTED
    dA, mA, dB, mB = _descs(host_handle, [4, 5], [1, 0], api.HIP_R_16BF)
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB, mB, api.HIP_R_32F, None) == api.HIPTENSOR_STATUS_NOT_SUPPORTED
    # A and B of different types: INVALID_VALUE
    dA, mA, dB, mB = _descs(host_handle, [4, 5], [1, 0], api.HIP_R_32F, api.HIP_R_16F)
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB, mB, api.HIP_R_32F, None) == api.HIPTENSOR_STATUS_INVALID_VALUE
    # scalar type other than f16 / f32: NOT_SUPPORTED
    dA, mA, dB, mB = _descs(host_handle, [4, 5], [1, 0])
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB, mB, api.HIP_R_64F, None) == api.HIPTENSOR_STATUS_NOT_SUPPORTED


@pytest.mark.parametrize("lens", [[7], [2, 2, 2, 2, 2, 2, 2]])
def test_ranks_without_an_instance_report_internal_error(host_handle, lens):
    dA, mA, dB, mB = _descs(host_handle, lens, list(range(len(lens))))
    st = api.hiptensorPermutation(host_handle, C.c_float(1.0), 256, dA, mA, 512, dB, mB, api.HIP_R_32F, None)
    assert st == api.HIPTENSOR_STATUS_INTERNAL_ERROR


def test_inconsistent_modes_or_lengths_are_invalid(host_handle):
    one = C.c_float(1.0)
    dA, mA, dB, mB = _descs(host_handle, [4, 5, 6], [2, 0, 1])
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB, [mB[0], mB[1], 999], api.HIP_R_32F, None) == api.HIPTENSOR_STATUS_INVALID_VALUE
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB, [mB[0], mB[0], mB[2]], api.HIP_R_32F, None) == api.HIPTENSOR_STATUS_INVALID_VALUE
    # lengths of B not those of A's modes
    dB2 = api.check(api.hiptensorInitTensorDescriptor(host_handle, [6, 4, 7], None, api.HIP_R_32F), "dB2")
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB2, mB, api.HIP_R_32F, None) == api.HIPTENSOR_STATUS_INVALID_VALUE
    # different rank
    dB3 = api.check(api.hiptensorInitTensorDescriptor(host_handle, [6, 4], None, api.HIP_R_32F), "dB3")
    assert api.hiptensorPermutation(host_handle, one, 256, dA, mA, 512, dB3, mB[:2], api.HIP_R_32F, None) == api.HIPTENSOR_STATUS_INVALID_VALUE


def test_too_many_elements_not_supported(host_handle):
    dA, mA, dB, mB = _descs(host_handle, [1 << 16, 1 << 15], [1, 0])
    assert api.permutationInfo(dA, mA, dB, mB)[0] == api.HIPTENSOR_STATUS_NOT_SUPPORTED


def test_a_handle_without_device_refuses_to_execute(host_handle):
    dA, mA, dB, mB = _descs(host_handle, [4, 5], [1, 0])
    st = api.hiptensorPermutation(host_handle, C.c_float(1.0), 256, dA, mA, 512, dB, mB, api.HIP_R_32F, None)
    assert st == api.HIPTENSOR_STATUS_ARCH_MISMATCH


def _info(h, dtype, lens, perm, A=0, B=0):
    p = wl.Permutation(h, wl.permutation(dtype, lens, perm))
    out = p.info(A, B)
    p.close()
    return out


def test_fusion_and_kernel_choice(host_handle):
    h = host_handle
    # identity order: everything fuses, vector copy
    i = _info(h, "f32", [64, 64, 64], [0, 1, 2])
    assert (i["fused_rank"], i["kernel"], i["vec_r"], i["extent"]) == (1, api.PERM_COPY, 4, [64 ** 3])
    # extent-1 modes vanish, neighbours that stay neighbours fuse
    i = _info(h, "f32", [8, 1, 16, 32, 64], [3, 4, 0, 1, 2])
    assert i["fused_rank"] == 2 and i["extent"] == [8 * 16, 32 * 64] and i["b_stride"] == [32 * 64, 1]
    assert i["kernel"] == api.PERM_TILED and (i["mode_i"], i["mode_j"]) == (0, 1) and (i["vec_r"], i["vec_w"]) == (4, 4)
    # the sample program's shape: 33 is odd, so loads are scalar; stores run along 34 * 35
    i = _info(h, "f32", [33, 32, 34, 35], [2, 3, 1, 0])
    assert i["kernel"] == api.PERM_GROUPED and i["extent"] == [33, 32, 34 * 35] and (i["vec_r"], i["vec_w"]) == (1, 2)
    assert i["kernel_name"] == "permute_grouped_f32_33x64_r1_w2"  # a small tensor: tiles shrunk until 512 workgroups
    # shared fastest mode
    i = _info(h, "f16", [512, 24, 96], [0, 2, 1])
    assert i["kernel"] == api.PERM_ROWS and i["vec_r"] == i["vec_w"] == 8 and i["mode_j"] == 2
    # ... a short one (interleaved channels): tiles of it times chunks of A's and B's next modes
    i = _info(h, "f32", [4, 512, 512, 8], [0, 2, 1, 3])
    assert i["kernel"] == api.PERM_SHARED and i["kernel_name"] == "permute_shared_f32_4x32x32_v4"
    # short fastest mode, tiny tensors: one thread per element
    assert _info(h, "f32", [3, 5, 7, 9, 11], [0, 4, 2, 3, 1])["kernel"] == api.PERM_GATHER
    assert _info(h, "f32", [5, 2, 3, 4], [3, 2, 1, 0])["kernel"] == api.PERM_GATHER
    # a short tile mode whose partner follows it in memory: strips
    i = _info(h, "f32", [512, 512, 3, 16], [2, 0, 1, 3])
    assert i["kernel"] == api.PERM_STRIP and i["tile"] == 0 and i["extent"][:2] == [512 * 512, 3] and (i["vec_r"], i["vec_w"]) == (4, 4)
    i = _info(h, "f16", [3, 512, 512, 16], [1, 2, 0, 3])
    assert i["kernel"] == api.PERM_STRIP and i["tile"] == 1 and (i["vec_r"], i["vec_w"]) == (8, 8)
    # ... when the partner is elsewhere in memory, grouped tiles take B's next mode along instead
    i = _info(h, "f32", [512, 3, 512, 16], [1, 3, 0, 2])
    assert i["kernel"] == api.PERM_GROUPED and i["kernel_name"] == "permute_grouped_f32_128x48_r4_w1"
    # many short modes: rows span A's two fastest modes, columns B's two fastest
    i = _info(h, "f32", [16] * 6, [5, 4, 3, 2, 1, 0])
    assert i["kernel"] == api.PERM_GROUPED and i["kernel_name"] == "permute_grouped_f32_112x112_r4_w4"
    assert _info(h, "f16", [16] * 6, [5, 4, 3, 2, 1, 0])["kernel_name"] == "permute_grouped_f16_128x128_r8_w8"
    # all extents one
    i = _info(h, "f16", [1, 1, 1], [2, 0, 1])
    assert (i["fused_rank"], i["kernel"], i["extent"]) == (1, api.PERM_COPY, [1])
    # a zero extent: nothing to launch
    assert _info(h, "f32", [4, 0, 3], [2, 0, 1])["empty"] == 1


def test_vector_width_follows_pointer_alignment(host_handle):
    h = host_handle
    assert _info(h, "f32", [256, 192], [1, 0], A=0x1000, B=0x2000)["vec_r"] == 4
    i = _info(h, "f32", [256, 192], [1, 0], A=0x1008, B=0x2004)
    assert (i["vec_r"], i["vec_w"]) == (2, 1)
    i = _info(h, "f16", [256, 192], [1, 0], A=0x1004, B=0x2010)
    assert (i["vec_r"], i["vec_w"]) == (2, 8)
    assert _info(h, "f16", [64, 64, 64], [0, 1, 2], A=0x1008, B=0x2000)["vec_r"] == 4


def test_every_validation_case_plans(host_handle):
    for rank in (2, 3, 4, 5, 6):
        for w in perm_cases.validation(rank, thin=36):
            p = wl.Permutation(host_handle, w)
            i = p.info()
            p.close()
            assert i["kernel_name"], w["name"]
