"""The C ABI library loads and exports every symbol include/stingray_sampler.h declares (no GPU needed)."""
import ctypes
import os
import re

import opentail.stingray_amd as sa

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "stingray_sampler.h")).read()
    return sorted(set(re.findall(r"SR_API\s+[\w\s\*]+?\b(sr_\w+)\s*\(", text)))


def _test_hook_symbols():
    text = open(os.path.join(ROOT, "include", "stingray_sampler_test.h")).read()
    return sorted(set(re.findall(r"SR_API\s+[\w\s\*]+?\b(sr_\w+)\s*\(", text)))


def test_the_test_hooks_are_declared_apart_and_exported_by_the_hooks_build_only():
    hooks = _test_hook_symbols()
    assert hooks and not set(hooks) & set(_declared_symbols())
    lib = ctypes.CDLL(sa.lib_path())
    assert not [s for s in hooks if hasattr(lib, s)], "the product library ships a test hook"
    with_hooks = ctypes.CDLL(sa.lib_path().replace("libstingray_sampler.so", "libstingray_sampler_hooks.so"))
    assert not [s for s in hooks if not hasattr(with_hooks, s)]
    assert not [s for s in _declared_symbols() if not hasattr(with_hooks, s)]


def test_header_and_python_symbol_lists_agree():
    assert _declared_symbols() == sorted(sa.EXPORTED_SYMBOLS)


def test_the_managed_binding_names_every_entry_point():
    text = open(os.path.join(ROOT, "opentail", "stingray_amd", "managed", "StingraySamplerInterop.cs")).read()
    bound = sorted(set(re.findall(r'EntryPoint = "(sr_\w+)"', text)))
    assert bound == _declared_symbols()
    # ... and the managed sampler calls only bindings that exist
    calls = set()
    for f in ("RocmBatchSampler.cs", "EngineSeam.cs"):
        calls |= set(re.findall(r"StingraySamplerInterop\.(\w+)\(", open(os.path.join(ROOT, "opentail", "stingray_amd", "managed", f)).read()))
    declared = set(re.findall(r"internal static (?:partial )?\w+ (\w+)\(", text))
    assert calls and calls <= declared, calls - declared


def test_library_exports_every_declared_symbol():
    assert os.path.exists(sa.lib_path()), "build with: python -m opentail.stingray_amd.build"
    lib = ctypes.CDLL(sa.lib_path())
    missing = [s for s in _declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing
    assert lib.sr_version is not None


def test_version_and_host_helpers_without_a_device():
    import numpy as np

    L = sa.load_library()
    assert re.match(rb"\d+\.\d+\.\d+", L.sr_version())
    row = np.array([1.0, -np.inf, 0.0, -np.inf, 5.0] + [-np.inf] * 30 + [2.0], dtype=np.float32)
    words = np.zeros(2, dtype=np.uint32)
    assert L.sr_pack_allow_mask(row.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), len(row),
                                words.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))) == 0
    assert words[0] == 0b10101 and words[1] == 0b1000
    assert np.array_equal(sa.pack_allow_mask(row != -np.inf), words)


def test_no_device_is_reported_not_hidden():
    import pytest
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    h = ctypes.c_void_p()
    assert sa.load_library().sr_create(0, ctypes.byref(h)) == sa.SR_ERR_NO_DEVICE
    with pytest.raises(sa.NativeLibraryError):
        sa.SamplerContext(0)
