"""CPU-side checks of the boundary: the library loads and exports every declared symbol."""
import ctypes
import os

import numpy as np

from eisen_amd import hip
from eisen_amd.lib import HSACO_PATH, LIB_PATH, declared_symbols, load_library


def test_library_exports_every_declared_symbol():
    lib = load_library()
    for header in sorted(h for h in os.listdir(os.path.join(os.path.dirname(LIB_PATH), "..", "include")) if h.endswith(".h")):
        names = declared_symbols(header)
        assert names, header
        missing = [n for n in names if not hasattr(lib, n)]
        assert not missing, f"{header}: not exported: {missing}"


def test_code_object_is_built_for_gfx950():
    blob = open(HSACO_PATH, "rb").read()
    assert (blob[:4] == b"\x7fELF" or blob.startswith(b"__CLANG_OFFLOAD_BUNDLE__")) and b"amdgcn-amd-amdhsa--gfx950" in blob
    for name in (b"fill_f32", b"scale_f32", b"copy_f32", b"cast_f32_to_bf16", b"cast_bf16_to_f32"):
        assert name in blob


def test_no_device_is_an_error_not_a_fallback():
    lib = load_library()
    h = ctypes.c_void_p()
    rc = lib.eisen_hip_init(9999, ctypes.byref(h))
    assert rc != 0 and not h.value
    assert lib.eisen_hip_stream_sync(None) == -1          # EISEN_E_ARG on a null context


def test_bf16_host_rounding_is_rne():
    import torch
    x = np.concatenate([np.random.default_rng(0).standard_normal(4096).astype(np.float32) * 37,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.4e38, -3.4e38, 1e-40], np.float32)])
    assert np.array_equal(hip.round_bf16(x), torch.tensor(x).bfloat16().float().numpy())
    # reference test vector: exact round trip (tests/test_bf16.rs)
    v = np.array([1.5, -2.25, 3.125, 0.0], np.float32)
    assert np.array_equal(hip.round_bf16(v), v)
