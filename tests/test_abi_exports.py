"""CPU-side checks of the C ABI library: it loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ahpc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ahpc_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from attention_amd import hip
    lib = hip.load()
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(hip.SIGNATURES) == names  # the Python view binds exactly the header


def test_no_gpu_calls_that_must_work_anywhere():
    from attention_amd import hip
    assert hip.error_string(0) == "success"
    assert "head dimension" in hip.error_string(-4)
    assert hip.device_count() >= 0
    assert hip.paged_decode_workspace_bytes(64, 32, 128, 4096, 16, 256) == 64 * 16 * 32 * 130 * 4
    assert hip.paged_decode_workspace_bytes(2, 4, 64, 100, 16, 1024) == 0  # one chunk: no partials
