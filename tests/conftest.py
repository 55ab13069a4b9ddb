import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    # the whole-API conformance binary goes last so that a failure there does not hide kernel-level results
    items.sort(key=lambda it: 1 if "test_zz" in it.nodeid else 0)


@pytest.fixture(scope="session")
def gpu():
    """The C ABI view for GPU tests.  Refuses to go on unless what is loaded is the in-tree gfx950 library on a
    gfx950 device: a same-named CPU look-alike exists for the executor tests, and AHPC_HIP_LIB can point elsewhere."""
    import torch
    from attention_amd import hip
    hip.load()
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    want = os.path.join(ROOT, "attention_amd", "lib", "libahpc_hip.so")
    assert os.path.realpath(hip.LIB_PATH) == os.path.realpath(want), f"GPU tests loaded {hip.LIB_PATH}, not {want}"
    with open("/proc/self/maps") as maps:
        loaded = {line.split()[-1] for line in maps if line.rstrip().endswith("libahpc_hip.so")}
    assert loaded == {os.path.realpath(want)}, f"libahpc_hip.so mapped from {sorted(loaded)}"
    info = hip.device_info(0)
    arch = info["arch"] if isinstance(info, dict) else info.arch
    arch = arch.decode() if isinstance(arch, bytes) else arch
    assert arch.startswith("gfx950"), f"device architecture {arch!r}: these kernels are built for gfx950 only"
    return hip
