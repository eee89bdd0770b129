"""The C-ABI library loads and exports every symbol include/ttpa.h declares (no GPU
work is issued), and argument validation on the host side answers before any launch."""

import ctypes
import os
import re

import pytest

import __graft_entry__ as entry

HEADER = os.path.join(entry.ROOT, "include", "ttpa.h")


@pytest.fixture(scope="module")
def native():
    entry.ensure_built()
    from tt_xla_amd import _native

    _native.lib()
    return _native


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ttpa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(native):
    names = _declared()
    assert len(names) >= 10
    raw = ctypes.CDLL(native.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} not exported"
        assert n in native.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(native.SIGNATURES) == names


def test_abi_version_and_error_string(native):
    lib = native.lib()
    assert lib.ttpa_abi_version() == 1
    # null pointers are rejected on the host, before any HIP call
    rc = lib.ttpa_paged_update_cache(None, None, 0, 0, None, 0, None, 0, 1, 1, 32, 64, 1, 1, 0, None)
    assert rc == native.ERR_INVALID_ARGUMENT
    assert b"null" in lib.ttpa_last_error()
    rc = lib.ttpa_paged_sdpa_decode(16, 0, 0, 16, 0, 0, 16, 16, 16, 0, 16, 0, 1, 3, 2, 128, 64, 1, 1,
                                    1.0, 0, None, 0, None)
    assert rc == native.ERR_INVALID_ARGUMENT and b"divisible" in lib.ttpa_last_error()
    rc = lib.ttpa_paged_sdpa_decode(16, 0, 0, 16, 0, 0, 16, 16, 16, 0, 16, 0, 1, 4, 2, 96, 64, 1, 1,
                                    1.0, 0, None, 0, None)
    assert rc == native.ERR_UNSUPPORTED
    with pytest.raises(native.TtpaError):
        native.call("ttpa_bfp8_quantize", 16, 16, 16, 17, None)


def test_workspace_size_is_positive_and_monotone(native):
    lib = native.lib()
    a = lib.ttpa_paged_decode_workspace_bytes(32, 32, 8, 128)
    b = lib.ttpa_paged_decode_workspace_bytes(128, 64, 8, 128)
    assert 0 < a < b
    assert lib.ttpa_paged_decode_workspace_bytes(32, 30, 8, 128) == 0


def test_ops_are_registered_and_refuse_cpu_tensors(native):
    import torch

    import tt_xla_amd  # noqa: F401

    for name in (
        "paged_update_cache", "paged_fill_cache", "paged_scaled_dot_product_attention_decode",
        "chunked_scaled_dot_product_attention", "scaled_dot_product_attention",
        "paged_update_cache_", "paged_fill_cache_", "paged_update_kv_cache_", "paged_fill_kv_cache_",
        "paged_update_kv_decode_", "paged_update_kv_decode_out_", "paged_fill_kv_prefill_out_",
        "scaled_dot_product_attention_out", "chunked_scaled_dot_product_attention_out",
    ):
        assert hasattr(torch.ops.tt, name)
    cache = torch.zeros(2, 1, 32, 64, dtype=torch.bfloat16)
    fill = torch.zeros(1, 1, 1, 64, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):  # no CPU implementation, and no fallback
        torch.ops.tt.paged_update_cache(cache, fill, torch.zeros(1, dtype=torch.int32),
                                        torch.zeros(1, 2, dtype=torch.int32))


def test_latent_decode_entry_validates_on_the_host():
    """The latent (MLA) decode entry point rejects bad arguments before any launch (no GPU needed)."""
    from tt_xla_amd import _native as N

    rc = N.lib().ttpa_paged_mla_decode(None, 0, 0, None, 0, 0, None, None, None, 0, None, 0, 1, 16, 1, 576,
                                       512, 32, 1, 1, 1.0, None, None, 0, None)
    assert rc == N.ERR_INVALID_ARGUMENT
    assert b"null" in N.lib().ttpa_last_error()


def test_latent_decode_refuses_more_segments_than_the_grid_has_threads(native, monkeypatch):
    """The 16-head latent kernel publishes one segment row per thread of its grid: a grid made
    small by TTPA_DECODE_WAVES_PER_CU must be refused on the host when users x kv_heads does not
    fit, before any launch (the merge would read rows nobody wrote)."""
    lib = native.lib()
    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "0.01")
    users, hq, hkv, d = 1024, 64, 8, 128
    need = lib.ttpa_paged_mla_decode_workspace_bytes(users, hq, hkv, d)
    assert need > 0
    rc = lib.ttpa_paged_mla_decode(256, 8 * d, d, 256, 8 * d, d, 256, None, 256, 1, 256, 0, users, hq, hkv, d, d,
                                   32, 1, 4, 1.0, None, 256, need, None)
    assert rc == native.ERR_UNSUPPORTED and b"segments" in lib.ttpa_last_error()
