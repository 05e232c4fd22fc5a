"""CPU tests of the C-ABI library: it loads, exports every symbol include/gptrs_hip.h declares,
and fails loudly (no CPU fallback) when no GPU is present."""
import ctypes
import os
import re

import pytest

from gptrs_amd import backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "gptrs_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gptrs_hip_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = backend.load_library()
    names = declared_symbols()
    assert len(names) >= 19
    for n in names:
        assert hasattr(lib, n), f"libgptrs_hip.so does not export {n}"
    assert set(names) == set(backend.EXPORTS)


def test_backend_name_and_null_safety():
    lib = backend.load_library()
    assert lib.gptrs_hip_backend_name(None) == b"hip"
    assert lib.gptrs_hip_counter(None, b"kernel_launches") == -1
    lib.gptrs_hip_tensor_release(None)
    lib.gptrs_hip_tensor_retain(None)
    assert lib.gptrs_hip_supports_decode_sampling(None, 0.0, 0, 0) == 1
    assert lib.gptrs_hip_supports_decode_sampling(None, 1.0, 0, 0) == 0
    assert lib.gptrs_hip_supports_decode_sampling(None, 1.0, 1, 1) == 0


def gpu_present():
    return os.path.exists("/dev/kfd")


@pytest.mark.skipif(gpu_present(), reason="a GPU is visible: creation succeeds there")
def test_create_without_gpu_is_an_execution_error_not_a_fallback():
    with pytest.raises(backend.BackendError) as ei:
        backend.HipBackend(0)
    assert ei.value.kind == "execution"
    assert "no CPU fallback" in str(ei.value) or "HIP" in str(ei.value)
