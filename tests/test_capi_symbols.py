"""The C-ABI library loads and exports every symbol include/h2x.h declares
(no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "h2x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(h2x_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared_functions()
    for must in ("h2x_bn_channel_sums_and_sqsums", "h2x_bn_sums_to_statistics", "h2x_bn_batch_normalization",
                 "h2x_bn_backprop1", "h2x_bn_backprop2", "h2x_softmax_channel_forward",
                 "h2x_softmax_channel_backward", "h2x_halo_pack_or_unpack", "h2x_shuffle_pack",
                 "h2x_shuffle_unpack"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from dihydrogen_amd import capi
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/h2x.h but not exported"


def test_binding_covers_every_declared_symbol():
    from dihydrogen_amd import capi
    assert sorted(capi.SIGNATURES) == _declared_functions()
    lib = capi.load()
    assert lib.h2x_abi_version() == capi.ABI_VERSION
    assert lib.h2x_status_string(0) == b"success"
    assert lib.h2x_status_string(-1) == b"invalid argument"
    assert lib.h2x_bn_workspace_bytes(64) % 256 == 0 and lib.h2x_bn_workspace_bytes(64) > 0
    shp = capi.i64_array((130, 130, 130, 32, 1))
    assert lib.h2x_halo_size(5, shp, 1, 1) == 130 * 130 * 32  # legacy/.../halo_exchange_cuda.hpp:267-271


def test_struct_layouts_match_the_header():
    from dihydrogen_amd import capi
    # 2 pointers + 6 int64 + 8 int32 ; 2 int32 + 18 int64 + 2 pointers
    assert ctypes.sizeof(capi.HaloFace) == 16 + 48 + 32
    assert ctypes.sizeof(capi.ShuffleGeometry) == 8 + 144 + 16


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from dihydrogen_amd import capi
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "libh2x.so"))
    import pytest
    with pytest.raises(capi.H2XError):
        capi.load()
