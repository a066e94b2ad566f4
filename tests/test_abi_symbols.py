"""The shared library loads and exports every entry point the headers under include/ declare:
the kernel-layer C ABI, the flat C ABI, and the C++ functions of <hiptensor/hiptensor.hpp>."""
import os
import re
import subprocess

from hiptensor_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def c_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(hipt\w+|hiptensor\w+)\s*\(", text)) - {"hiptensorAmdLoggerCallback_t"})


def exported():
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    return {l.split()[-1] for l in out.splitlines() if l.strip()}


def test_c_abi_symbols_exported():
    syms = exported()
    for header in ("hiptk_kernels.h", "hiptensor_amd.h"):
        names = c_functions(header)
        assert len(names) >= 6, header
        missing = [n for n in names if n not in syms]
        assert not missing, (header, missing)
        for n in names:
            assert getattr(_lib._cdll, n) is not None  # resolvable through the loader too


def test_cpp_api_symbols_exported():
    out = subprocess.run(["nm", "-DC", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    names = c_functions(os.path.join("hiptensor", "hiptensor.hpp"))
    assert "hiptensorContraction" in names and "hiptensorInitContractionPlan" in names
    for n in names:
        assert re.search(rf"\b{n}\(", out), n


def test_bindings_reach_declared_functions_only():
    """A ctypes function without argument types passes Python ints as C ints, which cuts a
    device address to 32 bits; the binding therefore refuses any function it has no signature for,
    and every address parameter of a declared one is pointer-sized."""
    import ctypes

    import pytest

    with pytest.raises(AttributeError):
        _lib.lib.hiptk_permute  # kernel-layer entry that Python has no business calling
    for name, (_, args) in _lib._SIGS.items():
        assert getattr(_lib.lib, name).argtypes == args
    assert _lib._SIGS["hiptk_fill_pattern"][1][0] is ctypes.c_void_p
