"""The C-ABI library builds for gfx950, loads without a GPU, and exports every symbol include/oxhip.h
declares. No compute calls here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from oxinfer_amd import hip
    if not os.path.exists(hip.library_path()):
        from oxinfer_amd import build
        build.build()
    return hip.load_library()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "oxhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(oxhip_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = declared_functions()
    assert len(names) >= 14
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/oxhip.h but not exported: {missing}"


def test_open_declines_without_a_device(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    ctx = ctypes.c_void_p()
    assert lib.oxhip_open(0, ctypes.byref(ctx)) == 0 and not ctx.value
    assert lib.oxhip_last_error()  # says why


def test_probe_without_a_device_reports_none(lib):
    import torch
    from oxinfer_amd import hip
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    assert hip.probe() == []


def test_null_arguments_decline(lib):
    assert lib.oxhip_upload(None, None) is None
    assert lib.oxhip_matmul(None, None, 0, 0, None, 0) == 0
    assert lib.oxhip_wants(None, 64, 64, 1) == 0
    lib.oxhip_close(None)
    lib.oxhip_free_weight(None, None)


def test_product_does_not_reach_the_oracle():
    """Nothing under the package or the C sources may import, link or open the oracle."""
    pkg = os.path.join(ROOT, "oxinfer_amd")
    for d, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(d, f), errors="ignore").read()
                assert "oxref" not in text and "oracle" not in text, os.path.join(d, f)
