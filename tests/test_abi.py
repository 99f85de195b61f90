"""The C-ABI library loads and exports every symbol include/monet_hip.h declares
(no compute calls, so this runs without a GPU)."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "monet_hip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_symbols():
    names = declared_symbols()
    assert "mn_relu_fwd_mask_f32" in names and "mn_bn_bwd_from_y_f32" in names
    assert len(names) >= 20


def test_library_exports_every_declared_symbol():
    from monet_amd import _lib
    if not _lib.LIB_PATH.exists():
        pytest.fail(f"{_lib.LIB_PATH} missing: run `python -m monet_amd.build`")
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_table_matches_header():
    from monet_amd import _lib
    assert sorted(_lib.exported_names()) == declared_symbols()
    lib = _lib.load()
    assert lib.mn_abi_version() == _lib.ABI_VERSION
    assert lib.mn_status_string(0) == b"ok"
    assert b"unsupported" in lib.mn_status_string(2)


def test_host_only_entry_points():
    from monet_amd import _lib
    from oracle import lm_oracle as O
    lib = _lib.load()
    for size, k, p, s, d, ceil in [(112, 3, 1, 2, 1, 0), (13, 3, 1, 2, 1, 1), (7, 4, 2, 3, 1, 1),
                                   (416, 2, 0, 2, 1, 0), (5, 3, 1, 1, 2, 0), (6, 2, 1, 2, 1, 1)]:
        assert lib.mn_pool_out_size(size, k, p, s, d, ceil) == O.pool_out_size(size, k, p, s, d, ceil)
    assert lib.mn_pool_out_size(0, 3, 1, 2, 1, 0) == -1
    assert lib.mn_bn_ws_bytes(184, 256, 3136) >= 256 * 2 * 4
