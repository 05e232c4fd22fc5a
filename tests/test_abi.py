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


def test_library_reads_pretty_printed_program_json():
    """`Program::to_json_string` is serde_json::to_string_pretty (crates/gpt-rs/src/backend/spec.rs:799-801): the text
    the Rust binding hands over is indented over many lines.  The library's reader must take it as it takes the
    compact form (checked through the device-free fusion report)."""
    import ctypes
    import json

    from gptrs_amd import backend as B
    from gptrs_amd import functional as F
    from gptrs_amd.ptir import FunctionBuilder, Program
    fb = FunctionBuilder("main", "F32")
    x, g, w = fb.param("F32", [1, 64]), fb.param("F32", [64]), fb.param("F32", [64, 128])
    fb.set_results([F.rms_norm(x, g, 1e-5)[0].matmul(w)])
    prog = Program(fb)
    compact = B.fusion_report(prog)
    lib = B.load_library()
    pretty = json.dumps(prog.obj, indent=2).encode()
    assert pretty.count(b"\n") > 100
    needed = ctypes.c_size_t(0)
    assert lib.gptrs_hip_fusion_report(pretty, len(pretty), None, 3, None, 0, ctypes.byref(needed)) == 0
    buf = ctypes.create_string_buffer(needed.value)
    assert lib.gptrs_hip_fusion_report(pretty, len(pretty), None, 3, buf, needed.value, ctypes.byref(needed)) == 0
    assert buf.value.decode().splitlines() == compact and any("rms_norm" in line for line in compact)
