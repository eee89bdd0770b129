"""The registered torch.ops.tt.* schemas, pinned as literal strings.  Names, argument order and
defaults are those of the reference's operator definitions (tt-xla
python_package/tt_torch/custom_ops.py:635-646, 745-759, 857-867, 915-921, 962-971, 1016-1024,
1198-1214, 1334-1346 and the latent operators :223-236, :381-397): a renamed or reordered
argument would break every caller that passes it by keyword, and nothing else in the suite
would notice.  No GPU needed: the operators are registered at import."""

import pytest
import torch

import __graft_entry__ as entry

SCHEMAS = {
    # the five operators of the hot path
    "paged_update_cache":
        "tt::paged_update_cache(Tensor cache, Tensor fill_value, Tensor update_indices, Tensor page_table, "
        "bool share_cache=False) -> Tensor",
    "paged_fill_cache":
        "tt::paged_fill_cache(Tensor cache, Tensor fill_value, Tensor page_table, Tensor? batch_idx=None) -> Tensor",
    "paged_scaled_dot_product_attention_decode":
        "tt::paged_scaled_dot_product_attention_decode(Tensor query, Tensor key, Tensor value, Tensor page_table, "
        "bool is_causal=False, Tensor? attn_mask=None, Tensor? cur_pos_tensor=None, Tensor? attention_sink=None, "
        "float? scale=None, SymInt? sliding_window_size=None) -> Tensor",
    "chunked_scaled_dot_product_attention":
        "tt::chunked_scaled_dot_product_attention(Tensor query, Tensor key, Tensor value, Tensor page_table, "
        "Tensor chunk_start_idx_tensor, float? scale=None) -> Tensor",
    "scaled_dot_product_attention":
        "tt::scaled_dot_product_attention(Tensor query, Tensor key, Tensor value, Tensor? attn_mask=None, "
        "bool is_causal=True, float? scale=None, SymInt? sliding_window_size=None) -> Tensor",
    # the static-cache operators
    "update_cache":
        "tt::update_cache(Tensor cache, Tensor fill_value, Tensor cache_position, SymInt? batch_offset=None) -> Tensor",
    "fill_cache":
        "tt::fill_cache(Tensor cache, Tensor fill_value, SymInt? batch_offset=None) -> Tensor",
    "scaled_dot_product_attention_decode":
        "tt::scaled_dot_product_attention_decode(Tensor query, Tensor key, Tensor value, Tensor cur_pos_tensor, "
        "Tensor? attn_mask=None, Tensor? attention_sink=None, bool is_causal=True, float? scale=None) -> Tensor",
    # the latent-attention operators
    "flash_mla_prefill":
        "tt::flash_mla_prefill(Tensor query, Tensor key, SymInt head_dim_v, Tensor? value=None, "
        "Tensor? attn_mask=None, bool is_causal=True, float? scale=None) -> Tensor",
    "paged_flash_mla_decode":
        "tt::paged_flash_mla_decode(Tensor query, Tensor key, SymInt head_dim_v, Tensor page_table, "
        "Tensor? value=None, bool is_causal=True, Tensor? attn_mask=None, Tensor? cur_pos_tensor=None, "
        "Tensor? attention_sink=None, float? scale=None) -> Tensor",
}


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


@pytest.mark.parametrize("name", sorted(SCHEMAS))
def test_schema(name):
    assert str(getattr(torch.ops.tt, name).default._schema) == SCHEMAS[name]
