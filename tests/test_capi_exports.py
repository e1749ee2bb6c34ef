"""The C-ABI library loads without a GPU, exports every symbol the header declares, and
rejects bad arguments before touching the device."""
import ctypes
import os
import re

import pytest

from fgattn_tk_cuda_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "spattn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(?:void|int|const char\*)\s+([a-z_0-9]+)\s*\(", text)))


def test_header_declares_expected_surface():
    names = _declared()
    for ref in ("attn_fwd_wg_impl", "attn_sparse_fwd_wg_impl", "allindex_mask_impl", "attn_maxq_denom_impl",
                "maxq_denom_impl", "booleanmask_128_impl", "booleanmask_to_indexmask_impl"):
        assert ref in names
    assert "spattn_sp_attn_blocks" in names and "spattn_packedmask_to_indexmask" in names and "spattn_qk_topkmask_indices" in names and "spattn_qblock_order" in names
    assert "spattn_booleanmask_packed" in names and "spattn_packedmask_to_blocklists" in names and "spattn_booleanmask_to_blocklists" in names


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    for name in _declared():
        assert hasattr(lib, name), name
    assert sorted(capi.exported_symbols()) == _declared()
    assert lib.spattn_version() >= 1


def test_status_strings():
    lib = capi.load()
    assert lib.spattn_status_string(0) == b"ok"
    for st in range(-6, 0):
        assert len(lib.spattn_status_string(st)) > 3


def test_argument_checks_return_before_any_launch():
    lib = capi.load()
    buf = (ctypes.c_char * 64)()
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    assert lib.spattn_full_attn(None, None, None, None, None, 1, 1, 128, 128, 0, 0.0, None) == -1
    assert lib.spattn_last_status() == -1
    assert lib.spattn_full_attn(p16, None, p16, p16, p16, 1, 1, 128, 96, 0, 0.0, None) == -2
    assert lib.spattn_full_attn(p16, None, p16, p16, p16, 0, 1, 128, 128, 0, 0.0, None) == -6
    assert lib.spattn_full_attn(p16, None, p16 + 4, p16, p16, 1, 1, 128, 128, 0, 0.0, None) == -5
    assert lib.spattn_sp_attn(p16, None, p16, p16, p16, p16, p16, 100, 128, 1, 1, 128, 128, 0, 0.0, None) == -3
    assert lib.spattn_sp_attn(p16, None, p16, p16, p16, p16, p16, 128, 32, 1, 1, 128, 128, 0, 0.0, None) == -4
    assert lib.spattn_booleanmask_to_indexmask(p16, p16, p16, 1, 1, 10, 1, 100, None) == -3
    assert lib.spattn_all_index_mask(None, p16, 1, 1, 1, 1, 128, None) == -1
    assert lib.spattn_full_attn(p16, None, p16, p16, p16, 1, 1, 1 << 24, 128, 0, 0.0, None) == -6
    assert lib.spattn_booleanmask_packed(p16, 0.5, 128, 96, p16, p16, p16, p16, 1, 1, 128, 64, 0, 0.0, None) == -4
    assert lib.spattn_booleanmask_packed(p16, 0.5, 64, 128, p16, p16, p16, p16, 1, 1, 128, 64, 0, 0.0, None) == -3
    assert lib.spattn_packedmask_to_blocklists(p16, p16, None, p16, 1, 1, 10, 1, 128, 0, None) == -6
    assert lib.spattn_booleanmask_to_blocklists(p16, p16, None, None, 1, 1, 10, 1, 128, 2, None) == -1
    # the reference-named wrappers record their status instead of returning it
    lib.attn_fwd_wg_impl(None, None, None, None, 1, 1, 128, 128)
    assert lib.spattn_last_status() == -1


def test_block_maxima_entry_points_check_their_arguments():
    lib = capi.load()
    buf = (ctypes.c_char * 64)()
    p16 = (ctypes.addressof(buf) + 15) & ~15
    assert lib.spattn_maxq_denom_blockmax(p16, p16, None, p16, p16, 1, 1, 128, 64, 0, 0.0, None) == -1
    assert lib.spattn_fullattn_maxq_denom_blockmax(p16, p16, p16, p16, p16, p16, p16, 1, 1, 128, 96, 0, 0.0, None) == -2
    assert lib.spattn_blockmax_to_blocklists(p16, p16, None, p16, p16, p16, 0.5, 32, 1, 1, 128, 64, 0, 0.0, 2, None) == -4
    assert lib.spattn_blockmax_to_blocklists(p16, p16, None, p16, p16, p16, 0.5, 64, 1, 1, 128, 64, 0, 0.0, 0, None) == -6
    assert lib.spattn_blockmax_to_blocklists(p16, p16, None, None, p16, p16, 0.5, 64, 1, 1, 128, 64, 0, 0.0, 2, None) == -1


def test_debug_library_loads_and_exports():
    """The NaN-poisoning build exports the product library's whole surface."""
    from fgattn_tk_cuda_amd import build as bld

    assert bld.POISON_LIB.exists(), "build them with `python -m fgattn_tk_cuda_amd.build`"
    poison = ctypes.CDLL(str(bld.POISON_LIB))
    for name in _declared():
        assert hasattr(poison, name), name


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "_LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(RuntimeError):
        capi.load()
