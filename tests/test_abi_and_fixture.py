"""CPU-only checks: the C-ABI library loads and exports what the header declares, the size
functions (pure host arithmetic) follow the documented layout, the committed fixture is what
the oracle produces, and the package refuses to work without its library."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("w4a32_hip.h", "w4a32_decoder.h")]


def declared_symbols():
    names = set()
    for header in HEADERS:
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(w4a32_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol(pkg):
    if not os.path.exists(pkg.LIB_PATH):
        pytest.fail(f"{pkg.LIB_PATH} not built: run __graft_entry__.build()")
    raw = ctypes.CDLL(pkg.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 15
    for name in names:
        assert hasattr(raw, name), f"{name} declared in the header but not exported"
    assert sorted(pkg.ABI) == names, "python binding and header disagree"
    assert pkg.lib().w4a32_abi_version() == 1
    assert pkg.lib().w4a32_error_string(-2).decode().startswith("unsupported shape")


def test_size_functions(pkg):
    L = pkg.lib()
    # tiles of 16 rows x 128 k = 1024 B nibbles + 128 B scales; then the rsum, bias and rowmul
    # planes (f32 per row) and the f16 copy of the scales (128 B per tile)
    tiles = (8960 // 16) * (1536 // 128)
    assert L.w4a32_packed_bytes(8960, 1536) == tiles * 1152 + 3 * 8960 * 4 + tiles * 128
    assert L.w4a32_packed_bytes(50, 96) == 4 * 1152 + 3 * 64 * 4 + 4 * 128   # padded to 64 x 128
    assert L.w4a32_packed_bytes(16, 48) == 0 and L.w4a32_packed_bytes(0, 32) == 0
    assert L.w4a32_native_u4_bytes(256, 1536) == 256 * 768
    assert L.w4a32_native_scale_bytes(256, 1536) == 256 * 48 * 2
    assert L.w4a32_workspace_bytes(1, 1536) == 256 + 32 * 1536            # header + 32 padded rows
    assert L.w4a32_workspace_bytes(512, 1536) == 4096 + 512 * 1536 * 3    # + the f16 copy
    assert L.w4a32_workspace_bytes(1, 100) == 0


def test_nibbles_and_scales_are_the_algorithmic_bytes(pkg):
    # when N % 16 == 0 and K % 128 == 0 the tiles hold exactly the format's own bytes (what the
    # decode kernels stream); the rest of the blob is three f32 planes and the f16 scale copy
    for n, k in [(1536, 1536), (256, 1536), (8960, 1536), (1536, 8960), (151936, 1536)]:
        fmt = n * k // 2 + n * (k // 32) * 2
        assert pkg.packed_bytes(n, k) == fmt + 3 * 4 * n + n * (k // 32) * 2


def test_fixture_matches_oracle(orc):
    g = np.load(os.path.join(ROOT, "tests", "golden", "w4a32_small.npz"))
    u4, sc = orc.quant_rhs(g["w"])
    assert np.array_equal(u4, g["u4"]) and np.array_equal(sc, g["scales"])
    aq, recip, neg_zp, _ = orc.quant_lhs(g["x"])
    assert np.array_equal(aq, g["aq"]) and np.array_equal(neg_zp, g["neg_zp"])
    assert np.array_equal(recip, g["recip"])
    assert np.array_equal(orc.linear(g["x"], u4, sc, bias=g["bias"]), g["y"])
    assert np.array_equal(orc.dequant(u4, sc, int(g["k"])), g["dequant"])
    # facts of the fixture that hold by construction
    assert np.all(g["u4"][1, :16] == 0x88) and g["scales"][1, 0] == 0x8000    # the zero block
    assert np.all(g["u4"][2, 16:] == 0x00)                                    # the constant block
    assert g["neg_zp"][2] == 128                                              # the one-sided row


def test_missing_library_is_an_error(pkg, monkeypatch):
    monkeypatch.setattr(pkg, "_lib", None)
    monkeypatch.setattr(pkg, "LIB_PATH", os.path.join(ROOT, "no_such_dir", "libw4a32_hip.so"))
    with pytest.raises(pkg.W4A32Error):
        pkg.lib()
