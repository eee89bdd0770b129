"""vLLM attention backend for multi-head latent attention (MLA) on MI355X.

Mirrors the interface of tt-xla's
``integrations/vllm_plugin/vllm_tt/attention_impls/attention_mla.py``: backend name and
static methods (:67-110), the constructor's arguments and refusals (:118-165), ``forward``'s
signature, its prefill / decode dispatch and its output contract (:184-422).  The latent
cache is ONE tensor ``[num_blocks, 1, block_size, kv_lora_rank + qk_rope_head_dim]`` per layer
(K and V share it: V is the leading ``kv_lora_rank`` features of K).

What a forward pass does, in the order of the reference:
  1. absorb ``W_UK_T`` into the no-position part of the query (:230-244) and concatenate the
     rotary part: latent query ``[users, S, N, L + R]``; latent key of the new tokens
     ``[users, S, 1, L + R]`` from ``kv_c_normed`` and ``k_pe`` (:246-248);
  2. prefill (more than one token per user, :283-297): causal attention of the new tokens
     against themselves (``tt::flash_mla_prefill``), then the new latent keys go into the paged
     cache through the fill page table (:337-359);
     decode: the new token's latent key goes into the cache at ``cache_position`` first
     (:379-389), then ``tt::paged_flash_mla_decode`` attends over the paged cache (:394-405);
  3. expand the latent output with ``W_UV`` and write ``[tokens, N * v_head_dim]`` (:322-335,
     :408-422).
Differences from the reference, invisible in results: the cache writes use the in-place
operators (one batched fill instead of a per-user loop over functional fills followed by a
copy of the whole cache); ``functional_cache_ops=True`` restores the reference's call sequence.

The two latent attention operators sit on ``ttpa_paged_mla_decode``.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import custom_ops  # noqa: F401  (registers torch.ops.tt.*)
from .attention import TTAttentionMetadataBuilder, TTMetadata

# the operator namespace, looked up once: host-logic tests substitute it
_ops = torch.ops.tt

try:  # pragma: no cover - vLLM is not part of the test image
    from vllm.v1.attention.backend import AttentionBackend as _BackendBase
    from vllm.v1.attention.backend import MLAAttentionImpl as _ImplBase
except Exception:  # vLLM absent: same surface, no base classes
    _BackendBase = object
    _ImplBase = object


class TTMLAAttentionBackend(_BackendBase):
    """Backend descriptor for the latent-attention layers (reference :67-110)."""

    @staticmethod
    def get_name() -> str:
        return "FLASH_ATTN_MLA"

    @staticmethod
    def get_impl_cls():
        return TTMLAAttentionBackendImpl

    @staticmethod
    def get_builder_cls():
        return TTAttentionMetadataBuilder  # the same stub builder as the non-latent backend

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                           cache_dtype_str: str = "auto") -> Tuple[int, ...]:
        # one concatenated latent tensor per slot: head_size = kv_lora_rank + qk_rope_head_dim
        assert num_kv_heads == 1, "num_kv_heads must be 1 for MLA"
        return (num_blocks, num_kv_heads, block_size, head_size)

    @staticmethod
    def get_page_size(vllm_config) -> int:
        return 32

    @staticmethod
    def swap_blocks(src_kv_cache, dst_kv_cache, src_to_dst) -> None:
        raise RuntimeError("swap_blocks is not used for the TT MLA backend.")


class TTMLAAttentionBackendImpl(_ImplBase):
    def __init__(
        self,
        num_heads: int,
        head_size: int,
        scale: float,
        num_kv_heads: int,
        alibi_slopes: Optional[List[float]],
        sliding_window: Optional[int],
        kv_cache_dtype: str,
        logits_soft_cap: Optional[float],
        attn_type: str,
        kv_sharing_target_layer_name: Optional[str],
        q_lora_rank: Optional[int] = None,
        kv_lora_rank: int = 0,
        qk_nope_head_dim: int = 0,
        qk_rope_head_dim: int = 0,
        qk_head_dim: int = 0,
        v_head_dim: int = 0,
        kv_b_proj=None,
        indexer: Optional[object] = None,
        q_pad_num_heads: Optional[int] = None,
        functional_cache_ops: bool = False,
        **kwargs,
    ) -> None:
        self.num_heads = num_heads
        self.head_size = head_size
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.kv_cache_dtype = kv_cache_dtype
        self.q_lora_rank = q_lora_rank
        self.kv_lora_rank = kv_lora_rank
        self.qk_nope_head_dim = qk_nope_head_dim
        self.qk_rope_head_dim = qk_rope_head_dim
        self.qk_head_dim = qk_head_dim
        self.v_head_dim = v_head_dim
        self.functional_cache_ops = functional_cache_ops
        if alibi_slopes is not None:
            raise NotImplementedError("Alibi slopes are not supported for MLA on TT.")
        if kv_cache_dtype != "auto":
            raise NotImplementedError(
                f"Quantized MLA KV cache ({kv_cache_dtype}) is not yet supported on TT."
            )

    # vLLM's generic MLA entry points are bypassed by the layer, which calls forward() directly
    def forward_mha(self, *args, **kwargs) -> None:
        raise RuntimeError(
            "TTMLAAttentionBackendImpl.forward_mha should never be called; the TT MLA layer "
            "routes through forward() directly."
        )

    def forward_mqa(self, *args, **kwargs):
        raise RuntimeError(
            "TTMLAAttentionBackendImpl.forward_mqa should never be called; the TT MLA layer "
            "routes through forward() directly."
        )

    # ------------------------------------------------------------------ forward
    def forward(
        self,
        q: Tuple[torch.Tensor, torch.Tensor],
        kv_c_normed: torch.Tensor,
        k_pe: torch.Tensor,
        kv_cache: torch.Tensor,
        attn_metadata: Optional[TTMetadata],
        layer,
        output: Optional[torch.Tensor] = None,
        **kwargs,
    ) -> None:
        """q = (q_nope [tokens, N, P], q_pe [tokens, N, R]); kv_c_normed [tokens, L];
        k_pe [tokens, 1, R]; kv_cache [num_blocks, 1, block_size, L + R]; the result is written
        into ``output`` [tokens, N * v_head_dim].  ``layer`` carries ``W_UK_T`` [N, P, L] and
        ``W_UV`` [N, L, V]."""
        assert output is not None, "TTMLAAttentionBackendImpl.forward requires an output tensor."
        q_nope, q_pe = q
        prefill = self._infer_is_prefill(q_nope, attn_metadata)
        users = 1
        if attn_metadata is not None and attn_metadata.cache_position is not None:
            users = attn_metadata.cache_position.shape[0]
        tokens = q_nope.shape[0]
        assert tokens % users == 0, f"total_tokens ({tokens}) not divisible by users ({users})."
        s = tokens // users
        n, lat, rope, nope = self.num_heads, self.kv_lora_rank, self.qk_rope_head_dim, self.qk_nope_head_dim

        act_dtype, device = q_pe.dtype, q_nope.device
        # W_UK_T is a plain attribute of the layer, not a parameter: it may still sit elsewhere
        w_uk_t = layer.W_UK_T.to(device=device)
        q_abs = torch.einsum("bsnp,npl->bsnl", q_nope.view(users, s, n, nope), w_uk_t).to(act_dtype)
        q_lat = torch.cat([q_abs, q_pe.view(users, s, n, rope)], dim=-1)             # [users, S, N, L+R]
        k_lat = torch.cat([kv_c_normed.view(users, s, 1, lat), k_pe.view(users, s, 1, rope)], dim=-1)

        if prefill:
            out = self._forward_prefill(q_lat, k_lat, kv_cache, attn_metadata, layer, s, users)
        else:
            out = self._forward_decode(q_lat, k_lat, kv_cache, attn_metadata, layer, users)
        output.copy_(out.to(act_dtype).reshape_as(output))

    @staticmethod
    def _infer_is_prefill(q_nope: torch.Tensor, attn_metadata: Optional[TTMetadata]) -> bool:
        """More than one token per user.  A pass is all prefill or all decode (the scheduler
        guarantees it); a pass without metadata is a profiling run and counts as prefill."""
        if attn_metadata is None or attn_metadata.cache_position is None:
            return True
        users = attn_metadata.cache_position.shape[0]
        assert users > 0, "Invalid number of users"
        return q_nope.shape[0] // users > 1

    @staticmethod
    def _has_cache(kv_cache) -> bool:
        return isinstance(kv_cache, torch.Tensor) and kv_cache.numel() > 0

    def _expand(self, out_lat: torch.Tensor, layer, pattern: str) -> torch.Tensor:
        return torch.einsum(pattern, out_lat, layer.W_UV.to(device=out_lat.device))

    def _forward_prefill(self, q_lat, k_lat, kv_cache, attn_metadata, layer, seq_len, users):
        out_lat = _ops.flash_mla_prefill(
            query=q_lat.transpose(1, 2).contiguous(),        # [users, N, S, L+R]
            key=k_lat.transpose(1, 2).contiguous(),          # [users, 1, S, L+R]
            head_dim_v=self.kv_lora_rank,
            value=None,
            attn_mask=attn_metadata.attn_mask if attn_metadata is not None else None,
            is_causal=attn_metadata.is_causal if attn_metadata is not None else True,
            scale=self.scale,
        )                                                    # [users, N, S, L]
        out = self._expand(out_lat, layer, "bnsl,nlv->bnsv")  # [users, N, S, V]
        out = out.transpose(1, 2).reshape(users * seq_len, self.num_heads * self.v_head_dim)

        # the new tokens' latent keys go into the paged cache (skipped in profiling runs)
        if attn_metadata is not None and self._has_cache(kv_cache):
            fill = k_lat.transpose(1, 2)                     # [users, 1, S, L+R], a view
            table = attn_metadata.fill_page_table
            if self.functional_cache_ops:
                filled = kv_cache
                for u in range(users):
                    filled = _ops.paged_fill_cache(
                        filled, fill[u : u + 1], table,
                        batch_idx=torch.tensor([u], dtype=torch.int32, device=kv_cache.device))
                kv_cache.copy_(filled)
            else:
                _ops.paged_fill_cache_(
                    kv_cache, fill, table,
                    torch.arange(users, dtype=torch.int32, device=kv_cache.device))
        return out

    def _forward_decode(self, q_lat, k_lat, kv_cache, attn_metadata, layer, users):
        # the new token's latent key goes into the cache first (skipped in profiling runs)
        if self._has_cache(kv_cache):
            fresh = k_lat.transpose(0, 1)                    # [1, users, 1, L+R]
            if self.functional_cache_ops:
                kv_cache.copy_(_ops.paged_update_cache(
                    kv_cache, fresh, attn_metadata.cache_position, attn_metadata.page_table))
            else:
                _ops.paged_update_cache_(
                    kv_cache, fresh, attn_metadata.cache_position, attn_metadata.page_table)
        is_causal = attn_metadata.is_causal if attn_metadata is not None else True
        out_lat = _ops.paged_flash_mla_decode(
            query=q_lat.transpose(0, 1),                     # [1, users, N, L+R]
            key=kv_cache,
            head_dim_v=self.kv_lora_rank,
            page_table=attn_metadata.page_table,
            value=None,
            is_causal=is_causal,
            attn_mask=None if is_causal else attn_metadata.attn_mask,
            cur_pos_tensor=attn_metadata.cache_position,
            scale=self.scale,
        )                                                    # [1, users, N, L]
        out = self._expand(out_lat.reshape(users, self.num_heads, self.kv_lora_rank), layer, "bnl,nlv->bnv")
        return out.reshape(users, self.num_heads * self.v_head_dim)
