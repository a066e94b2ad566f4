"""The C++ API as a drop-in: programs written against <hiptensor/hiptensor.hpp> build against
this repository's headers and link against libhiptensor_amd.so."""
import os
import subprocess

import pytest

from hiptensor_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin", "dropin_contraction")
BIN_PERM = os.path.join(ROOT, "tests", "cpp", "bin", "dropin_permutation")
REF_SAMPLES = "/root/reference/samples"
HIPCC = "/opt/rocm/bin/hipcc"


def build_dropin():
    os.makedirs(os.path.dirname(BIN), exist_ok=True)
    for out in (BIN, BIN_PERM):
        src = os.path.join(ROOT, "tests", "cpp", os.path.basename(out) + ".cpp")
        subprocess.run([HIPCC, "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"), src, "-o", out,
                        "-L" + os.path.dirname(_lib.LIB_PATH), "-lhiptensor_amd",
                        "-Wl,-rpath,$ORIGIN/../../../hiptensor_amd/lib"], check=True, capture_output=True)


def test_dropin_program_builds_and_links():
    build_dropin()
    assert os.path.exists(BIN) and os.path.exists(BIN_PERM)


def test_internal_headers_build_and_hold_their_values(tmp_path):
    """<hiptensor/internal/{types,config}.hpp> (element type names, numeric_limits of the 16-bit
    types, maxExactInteger, convert, __half host operators, inserters) compile together with the
    public header and compute what their names promise (a host-only program)."""
    src = os.path.join(ROOT, "tests", "cpp", "internal_headers.cpp")
    out = tmp_path / "internal_headers"
    subprocess.run([HIPCC, "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"), src, "-o", str(out),
                    "-L" + os.path.dirname(_lib.LIB_PATH), "-lhiptensor_amd",
                    "-Wl,-rpath," + os.path.dirname(_lib.LIB_PATH)], check=True, capture_output=True)
    r = subprocess.run([str(out)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and r.stdout.startswith("ok"), (r.stdout, r.stderr)


@pytest.mark.skipif(not os.path.isdir(REF_SAMPLES), reason="reference tree not mounted")
@pytest.mark.parametrize("sample", [
    "simple_bilinear_contraction_f32_f32_f32_f32_compute_f32",
    "simple_bilinear_contraction_f16_f16_f16_f16_compute_f16",
    "simple_scale_contraction_cf32_cf32_cf32_compute_cf32",
    "simple_scale_contraction_bf16_bf16_bf16_compute_bf16",
])
def test_reference_samples_compile_unchanged(sample, tmp_path):
    """The reference's own sample programs, compiled where they lie, against these headers and
    this library (they are not run: they refuse every architecture but gfx908 .. gfx942)."""
    src = os.path.join(REF_SAMPLES, "01_contraction", sample + ".cpp")
    out = tmp_path / sample
    subprocess.run([HIPCC, "-std=c++17", "-O0", "-I" + os.path.join(ROOT, "include"), "-I" + REF_SAMPLES, src,
                    "-o", str(out), "-L" + os.path.dirname(_lib.LIB_PATH), "-lhiptensor_amd"],
                   check=True, capture_output=True)
    assert out.exists()


@pytest.mark.skipif(not os.path.isdir(REF_SAMPLES), reason="reference tree not mounted")
def test_reference_permutation_sample_compiles_unchanged(tmp_path):
    """samples/02_permutation/permutation.cpp against these headers and this library."""
    src = os.path.join(REF_SAMPLES, "02_permutation", "permutation.cpp")
    out = tmp_path / "permutation"
    subprocess.run([HIPCC, "-std=c++17", "-O0", "-I" + os.path.join(ROOT, "include"), "-I" + REF_SAMPLES, src,
                    "-o", str(out), "-L" + os.path.dirname(_lib.LIB_PATH), "-lhiptensor_amd"],
                   check=True, capture_output=True)
    assert out.exists()


@pytest.mark.gpu
def test_dropin_program_runs():
    assert os.path.exists(BIN), "tests/cpp/bin/dropin_contraction is not built (build() makes it)"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0 and "dropin_contraction: ok" in r.stdout


@pytest.mark.gpu
def test_dropin_permutation_program_runs():
    assert os.path.exists(BIN_PERM), "tests/cpp/bin/dropin_permutation is not built (build() makes it)"
    r = subprocess.run([BIN_PERM], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0 and "dropin_permutation: ok" in r.stdout


def test_direct_load_kernels_request_only_what_exists(tmp_path):
    """tests/cpp/hd_bounds.cpp: every 16-byte request of the kernels that load operand tiles straight
    into LDS, walked on the host with the planner's own tables and the kernels' own address functions
    (kernels/hd_addr.hpp), lies inside its tensor, is 16-byte aligned and contiguous; every stage
    slot is filled once; every k is multiplied once (K tails, split-K slices, table-driven K)."""
    src = os.path.join(ROOT, "tests", "cpp", "hd_bounds.cpp")
    out = tmp_path / "hd_bounds"
    subprocess.run(["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"), "-isystem", "/opt/rocm/include",
                    "-D__HIP_PLATFORM_AMD__", src, "-o", str(out), "-L" + os.path.dirname(_lib.LIB_PATH), "-lhiptensor_amd",
                    "-Wl,-rpath," + os.path.dirname(_lib.LIB_PATH)], check=True, capture_output=True)
    r = subprocess.run([str(out)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().splitlines()[-1].startswith("ok"), (r.stdout[-2000:], r.stderr)
