"""CPU-side checks of the product boundary: the C-ABI library loads and exports every entry
point include/glades_hip.h declares.  No compute call is made here (no GPU in this run)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "glades-ml_amd", "libglades_hip.so")
HEADER = os.path.join(ROOT, "include", "glades_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ghip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for need in ("ghip_init", "ghip_net_create", "ghip_net_destroy", "ghip_net_set_params", "ghip_net_get_params",
                 "ghip_net_set_dataset", "ghip_net_run_epochs_exact", "ghip_net_train_step", "ghip_net_forward",
                 "ghip_net_quantize_fp8", "ghip_last_error"):
        assert need in syms


@pytest.mark.skipif(not os.path.exists(LIB), reason="libglades_hip.so not built (python glades-ml_amd/build.py)")
def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB)
    for s in declared_symbols():
        assert hasattr(lib, s), s
    lib.ghip_version.restype = ctypes.c_char_p
    assert b"gfx950" in lib.ghip_version()


@pytest.mark.skipif(not os.path.exists(LIB), reason="libglades_hip.so not built")
def test_binding_covers_the_header():
    import pyglades
    assert sorted(pyglades.EXPORTS) == declared_symbols()
    assert ctypes.sizeof(pyglades.Metrics) == 16


def test_product_never_touches_the_oracle():
    """Nothing under glades-ml_amd/ may import, link or read anything under oracle/."""
    pkg = os.path.join(ROOT, "glades-ml_amd")
    for dp, _, fns in os.walk(pkg):
        if os.path.basename(dp) in ("build", "__pycache__"):
            continue
        for fn in fns:
            if fn.endswith((".py", ".hip", ".h", ".cpp", ".hpp")):
                text = open(os.path.join(dp, fn), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(dp, fn)
