"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares,
and reports errors instead of computing when no GPU is present."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "yscv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(yscv_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import ctypes

    from yscv_amd import capi

    declared = _declared_symbols()
    assert len(declared) >= 30
    cdll = ctypes.CDLL(capi.library_path())
    missing = [s for s in declared if not hasattr(cdll, s)]
    assert not missing, missing
    # the Python binding covers the same set
    assert sorted(capi.EXPORTED_SYMBOLS) == declared


def test_abi_version_and_error_reporting():
    import torch

    import yscv_amd

    l = yscv_amd.lib()
    assert l.abi_version() == 1
    if torch.cuda.is_available():
        pytest.skip("error path below is the no-device one")
    with pytest.raises(yscv_amd.YscvHipError) as ei:
        l.init(0)
    assert ei.value.code == -5 and "no HIP device" in ei.value.message


def test_host_wrappers_validate_shapes_before_touching_the_device():
    import numpy as np

    from yscv_amd import kernels

    out = np.zeros(4, np.float32)
    with pytest.raises(ValueError):
        kernels.packed_int4_gemv_dispatch(np.zeros(10, np.uint8), np.zeros(4, np.float32), np.zeros(8, np.float32), out, 4, 8, 8)
    with pytest.raises(ValueError):
        kernels.int8_matmul_dispatch(np.zeros(5, np.int8), np.zeros(6, np.int8), 2, 3, 2, np.zeros(4, np.int32))
