"""vLLM attention backend for the paged path on MI355X.

Mirrors the interface of tt-xla's
``integrations/vllm_plugin/vllm_tt/attention_impls/attention.py``: class names, static
methods, the metadata fields, ``forward``'s signature and its error behaviour are the
reference's (:89-160, :177-218, :221-668), so vLLM's attention layer can drive either.
vLLM itself is optional: when it is importable the classes derive from its
``AttentionBackend`` / ``AttentionImpl``; otherwise they are plain classes with the same
surface.

Differences from the reference, both invisible in results:
  * cache writes go through the in-place operators, so a decode step moves
    users x kv_heads x head_size elements instead of cloning and copying back the whole
    cache (reference: functional op followed by ``kv_cache[i].copy_``, :473-515), and a
    causal decode step issues the write and the attention as one operator
    (``tt::paged_update_kv_decode_``).  ``functional_cache_ops=True`` restores the reference's
    exact call sequence.
  * ``get_page_size`` still answers 32 like the reference (:147-152); the kernels accept
    any block size that is a multiple of 4.
"""

from __future__ import annotations

from collections import namedtuple
from dataclasses import dataclass
from typing import List, Optional

import torch

from . import custom_ops  # noqa: F401  (registers torch.ops.tt.*)

try:  # pragma: no cover - vLLM is not part of the test image
    from vllm.v1.attention.backend import AttentionBackend as _BackendBase
    from vllm.v1.attention.backend import AttentionImpl as _ImplBase
    from vllm.v1.attention.backend import AttentionType

    _DECODER = AttentionType.DECODER
    _ENCODER = AttentionType.ENCODER
    _ENCODER_ONLY = AttentionType.ENCODER_ONLY
except Exception:  # vLLM absent: same surface, no base classes
    _BackendBase = object
    _ImplBase = object
    _DECODER, _ENCODER, _ENCODER_ONLY = "decoder", "encoder", "encoder_only"

# Head sizes are padded to a multiple of this by the model runner (reference :37-38).
TT_HEAD_SIZE_ALIGNMENT = 32

# kv_cache_dtype string -> storage dtype (reference :42-51).
STR_DTYPE_TO_TORCH_DTYPE = {
    "half": torch.half,
    "bfloat16": torch.bfloat16,
    "float": torch.float,
    "fp8": torch.float8_e4m3fn,
    "fp8_e4m3": torch.float8_e4m3fn,
    "fp8_e5m2": torch.float8_e5m2,
    "int8": torch.int8,
    "uint8": torch.uint8,
}


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


@dataclass
class TTMetadata:
    """Per-pass attention metadata (reference :177-218).

    cache_position  [users] int32: position written this step / last attended; -1 for
                    padded rows.
    page_table      [users, blocks_per_user] int32 physical block ids.
    fill_page_table page_table with already-computed prefix blocks rolled out of the
                    way so that column 0 is the first block to write; defaults to
                    page_table.
    chunk_start_idx [1] int32 = tokens already in the cache for a continuation chunk, or
                    None for a first / unchunked prefill.
    batch_idx       [users] int32 page-table row of each fill_value row.
    """

    cache_position: Optional[torch.Tensor]
    attn_mask: Optional[torch.Tensor]
    page_table: Optional[torch.Tensor]
    is_causal: bool
    fill_page_table: Optional[torch.Tensor]
    chunk_start_idx: Optional[torch.Tensor]
    batch_idx: Optional[torch.Tensor] = None
    num_users: Optional[int] = None

    def __init__(
        self,
        cache_position: Optional[torch.Tensor] = None,
        attn_mask: Optional[torch.Tensor] = None,
        page_table: Optional[torch.Tensor] = None,
        is_causal: bool = True,
        fill_page_table: Optional[torch.Tensor] = None,
        dp_size: int = 1,
        chunk_start_idx: Optional[torch.Tensor] = None,
        batch_idx: Optional[torch.Tensor] = None,
        num_users: Optional[int] = None,
    ):
        self.cache_position = cache_position
        self.attn_mask = attn_mask
        self.page_table = page_table
        self.is_causal = is_causal
        self.fill_page_table = page_table if fill_page_table is None else fill_page_table
        self.dp_size = dp_size
        self.chunk_start_idx = chunk_start_idx
        self.num_users = num_users
        self.batch_idx = batch_idx


class TTAttentionMetadataBuilder:
    """Stub builder vLLM's encoder-only layer asks for (reference :56-86); real metadata
    is produced by the model runner."""

    def build(self, common_prefix_len: int, common_attn_metadata, fast_build: bool = False):
        return TTMetadata(
            cache_position=None,
            attn_mask=None,
            page_table=None,
            is_causal=getattr(common_attn_metadata, "causal", True),
        )


class TTAttentionBackend(_BackendBase):
    @staticmethod
    def get_name() -> str:
        return "CUSTOM"

    @staticmethod
    def get_impl_cls():
        return TTAttentionBackendImpl

    @staticmethod
    def get_builder_cls():
        return TTAttentionMetadataBuilder

    @staticmethod
    def get_kv_cache_shape(
        num_blocks: int,
        block_size: int,
        num_kv_heads: int,
        head_size: int,
        cache_dtype_str: str = "auto",
    ) -> tuple:
        # one such tensor for K and one for V per layer
        return (num_blocks, num_kv_heads, block_size, head_size)

    @staticmethod
    def get_kv_cache_storage_shape(
        num_blocks: int,
        block_size: int,
        num_kv_heads: int,
        head_size: int,
        cache_dtype_str: str = "auto",
    ) -> tuple:
        """Shape of the tensor that actually holds one cache.  As ``get_kv_cache_shape`` except
        under the block-float-8 option (``experimental_kv_cache_dtype="bfp_bf8"``, reference
        vllm_tt/platform.py:165, 232-233, where the reference keeps the logical shape and its
        compiler picks the layout): a uint8 tensor with block_size / 16 more rows per block for
        the shared exponents (``custom_ops.bfp8_cache_shape``)."""
        if cache_dtype_str.lower().strip() in ("bfp_bf8", "bfp8"):
            return custom_ops.bfp8_cache_shape(num_blocks, num_kv_heads, block_size, head_size)
        return (num_blocks, num_kv_heads, block_size, head_size)

    @staticmethod
    def swap_blocks(src_kv_cache, dst_kv_cache, src_to_dst) -> None:
        raise RuntimeError("swap_blocks is not used for the TPU backend.")

    @staticmethod
    def get_min_page_size(vllm_config) -> int:
        per_req = 1024 * 1024 // 2 // vllm_config.scheduler_config.max_num_seqs // 4
        size = _cdiv(vllm_config.model_config.max_model_len, per_req)
        return 1 << (size - 1).bit_length()

    @staticmethod
    def get_max_num_seqs(model_len: int, page_size: int) -> int:
        return 1024 * 1024 // 2 // _cdiv(model_len, page_size) // 4

    @staticmethod
    def get_page_size(vllm_config) -> int:
        return 32


AttentionInputs = namedtuple(
    "AttentionInputs",
    [
        "query",
        "key",
        "value",
        "orig_query_shape",
        "orig_query_ndim",
        "users",
        "query_num_tokens",
        "is_prefill",
        "users_kv",
        "kv_num_tokens",
    ],
)


class TTAttentionBackendImpl(_ImplBase):
    def __init__(
        self,
        num_heads: int,
        head_size: int,
        scale: float,
        num_kv_heads: int,
        alibi_slopes: Optional[List[float]] = None,
        sliding_window: Optional[int] = None,
        kv_cache_dtype: str = "auto",
        logits_soft_cap: Optional[float] = None,
        attn_type: str = _DECODER,
        kv_sharing_target_layer_name: Optional[str] = None,
        sinks: Optional[torch.Tensor] = None,
        functional_cache_ops: bool = False,
    ) -> None:
        self.num_heads = num_heads
        self.head_size = head_size
        self.scale = float(scale)
        self.num_kv_heads = num_kv_heads
        self.sliding_window = sliding_window
        self.logits_soft_cap = logits_soft_cap
        self.kv_sharing_target_layer_name = kv_sharing_target_layer_name
        self.num_queries_per_kv = num_heads // num_kv_heads
        self.functional_cache_ops = functional_cache_ops
        if alibi_slopes is not None:
            raise NotImplementedError("Alibi slopes is not supported.")
        if attn_type not in (_DECODER, _ENCODER, _ENCODER_ONLY):
            raise NotImplementedError(
                f"TT attention only supports encoder or decoder attention, but got {attn_type}."
            )
        self.kv_cache_stored = None
        self.kv_cache_quantized_dtype = None
        if kv_cache_dtype != "auto":
            self.kv_cache_quantized_dtype = STR_DTYPE_TO_TORCH_DTYPE.get(
                kv_cache_dtype.lower().strip()
            )
        self.sinks = sinks
        if sinks is not None:
            assert sinks.shape[0] == num_heads, (
                "Sinks must have the same number of heads as the number of heads in the layer"
            )

    # ------------------------------------------------------------------ forward
    def forward(
        self,
        layer,
        query: torch.Tensor,
        key: torch.Tensor,
        value: torch.Tensor,
        kv_cache,
        attn_metadata: TTMetadata,
        output: Optional[torch.Tensor] = None,
        output_scale: Optional[torch.Tensor] = None,
        output_block_scale: Optional[torch.Tensor] = None,
    ) -> None:
        """query [tokens, Hq*D]; key / value [tokens, Hkv*D]; kv_cache = [k_cache, v_cache];
        the result is written into ``output`` [tokens, Hq*D]."""
        assert attn_metadata is not None, "TT attention requires metadata."
        assert output is not None, "TT attention requires an output buffer."
        inputs = self._prepare_inputs(query, key, value, attn_metadata)

        # a scalar placeholder stands in for the cache while vLLM profiles memory;
        # layers that share another layer's cache never write it
        writes_cache = (
            isinstance(kv_cache, (list, tuple))
            and kv_cache[0].numel() > 0
            and self.kv_sharing_target_layer_name is None
        )
        # a causal decode step writes its token inside the attention call (one operator)
        fused_step = (
            writes_cache
            and not inputs.is_prefill
            and not self.functional_cache_ops
            and attn_metadata.is_causal
            and attn_metadata.attn_mask is None
        )
        # The reference copies the operator's result into vLLM's output buffer (:330-336).  Where
        # the buffer can be viewed as [users, tokens, heads, head_size] the operators write into
        # it directly (their out-variants take any strides) and return None.
        direct = None if self.functional_cache_ops else self._output_view(output, inputs)
        # a first-chunk prefill pass (fill K, fill V, dense attention on the fresh K / V) is one
        # operator too: the attention does not read the caches, so the fills ride in its launch
        fused_prefill = (
            writes_cache
            and inputs.is_prefill
            and direct is not None
            and attn_metadata.chunk_start_idx is None
            and attn_metadata.attn_mask is None
            and attn_metadata.is_causal
            and self.sinks is None
            and kv_cache[0].dtype == torch.bfloat16
            and inputs.key.shape[0] == inputs.query.shape[0]
            and inputs.query_num_tokens % 32 == 0
        )
        if fused_prefill:
            batch_idx = attn_metadata.batch_idx
            assert batch_idx is not None, "batch_idx must be provided for prefill."
            if attn_metadata.dp_size > 1:
                batch_idx = batch_idx % (inputs.key.shape[0] // attn_metadata.dp_size)
            torch.ops.tt.paged_fill_kv_prefill_out_(
                inputs.query.transpose(1, 2), inputs.key.transpose(1, 2), inputs.value.transpose(1, 2),
                kv_cache[0], kv_cache[1], attn_metadata.fill_page_table, batch_idx, direct.transpose(1, 2),
                is_causal=True, scale=self.scale, sliding_window_size=self.sliding_window,
            )
            return
        if writes_cache and not fused_step:
            self._handle_paged_attention(inputs, kv_cache, attn_metadata)

        if inputs.is_prefill:
            assert self.sinks is None, "Attention sink is unsupported in SDPA prefill"
            attn_output = self._compute_full_attention(inputs, kv_cache, attn_metadata, direct)
        else:
            attn_output = self._compute_decode_attention(inputs, kv_cache, attn_metadata, fused_step, direct)
        if attn_output is None:
            return
        flat = attn_output.reshape(-1, self.num_heads * self.head_size)
        output.copy_(flat.reshape_as(output))

    def _output_view(self, output: torch.Tensor, inputs) -> Optional[torch.Tensor]:
        """``output`` as [users, tokens, heads, head_size] without a copy, or None."""
        if output.dtype != torch.bfloat16 or not output.is_contiguous() or output.data_ptr() % 16:
            return None
        shape = (inputs.users, inputs.query_num_tokens, self.num_heads, self.head_size)
        if output.numel() != shape[0] * shape[1] * shape[2] * shape[3] or self.head_size % 8:
            return None
        return output.view(shape)

    # ------------------------------------------------------------------ reshapes
    def _normalize_to_attention_format(
        self, tensor: torch.Tensor, tensor_name: str, expected_num_heads: int,
        expected_head_size: int, num_users: int,
    ) -> torch.Tensor:
        """-> [users, tokens, heads, head_size]; the leading dim is always flattened tokens."""
        if tensor.ndim < 2:
            raise ValueError(f"{tensor_name} must have rank >= 2, got shape={tuple(tensor.shape)}")
        hidden = expected_num_heads * expected_head_size
        if tensor.ndim == 2 and tensor.shape[-1] == hidden:
            t = tensor.reshape(-1, expected_num_heads, expected_head_size)
        elif (
            tensor.ndim == 3
            and tensor.shape[-2] == expected_num_heads
            and tensor.shape[-1] == expected_head_size
        ):
            t = tensor
        else:
            raise ValueError(
                f"{tensor_name} must be either a flattened-token tensor with "
                f"shape[-1] == {hidden} or a head-shaped tensor with "
                f"shape[-2:] == ({expected_num_heads}, {expected_head_size}); "
                f"got shape={tuple(tensor.shape)}"
            )
        if t.shape[0] % num_users != 0:
            raise ValueError(
                f"{tensor_name} total tokens ({t.shape[0]}) must be divisible "
                f"by num_users ({num_users})"
            )
        return t.reshape(num_users, -1, expected_num_heads, expected_head_size)

    def _prepare_inputs(self, query, key, value, attn_metadata: TTMetadata) -> AttentionInputs:
        users = attn_metadata.num_users
        assert users is not None, "num_users must be provided in attn_metadata."
        q = self._normalize_to_attention_format(query, "query", self.num_heads, self.head_size, users)
        k = self._normalize_to_attention_format(key, "key", self.num_kv_heads, self.head_size, users)
        v = self._normalize_to_attention_format(value, "value", self.num_kv_heads, self.head_size, users)
        if k.shape != v.shape:
            raise ValueError(
                f"key and value must match after normalization, got "
                f"key={tuple(k.shape)} value={tuple(v.shape)}"
            )
        return AttentionInputs(
            query=q,
            key=k,
            value=v,
            orig_query_shape=query.shape,
            orig_query_ndim=query.ndim,
            users=users,
            query_num_tokens=q.shape[1],
            is_prefill=q.shape[1] > 1,
            users_kv=k.shape[0],
            kv_num_tokens=k.shape[1],
        )

    # ------------------------------------------------------------------ cache write
    def _handle_paged_attention(self, inputs, kv_cache, attn_metadata: TTMetadata) -> None:
        ops = torch.ops.tt
        if not inputs.is_prefill:
            # [users, 1, Hkv, D] -> [1, users, Hkv, D]
            k_new = inputs.key.transpose(0, 1)
            v_new = inputs.value.transpose(0, 1)
            args = (attn_metadata.cache_position, attn_metadata.page_table)
            if self.functional_cache_ops:
                kv_cache[0].copy_(ops.paged_update_cache(kv_cache[0], k_new, *args))
                kv_cache[1].copy_(ops.paged_update_cache(kv_cache[1], v_new, *args))
            else:  # both scatters in one launch
                ops.paged_update_kv_cache_(kv_cache[0], kv_cache[1], k_new, v_new, *args)
            return
        # prefill: [users, S, Hkv, D] -> [users, Hkv, S, D], all users in one call
        k_new = inputs.key.transpose(1, 2)
        v_new = inputs.value.transpose(1, 2)
        batch_idx = attn_metadata.batch_idx
        assert batch_idx is not None, "batch_idx must be provided for prefill."
        if attn_metadata.dp_size > 1:
            # rows are sharded over batch replicas; make the ids local to the shard
            batch_idx = batch_idx % (k_new.shape[0] // attn_metadata.dp_size)
        table = attn_metadata.fill_page_table
        if self.functional_cache_ops:
            kv_cache[0].copy_(ops.paged_fill_cache(kv_cache[0], k_new, table, batch_idx=batch_idx))
            kv_cache[1].copy_(ops.paged_fill_cache(kv_cache[1], v_new, table, batch_idx=batch_idx))
        else:
            ops.paged_fill_kv_cache_(kv_cache[0], kv_cache[1], k_new, v_new, table, batch_idx=batch_idx)  # one launch

    # ------------------------------------------------------------------ attention
    def _compute_full_attention(self, inputs, kv_cache, attn_metadata: TTMetadata,
                                direct: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        has_paged_cache = (
            isinstance(kv_cache, (list, tuple)) and len(kv_cache) >= 2 and kv_cache[0].numel() > 0
        )
        shared_kv = self.kv_sharing_target_layer_name is not None and has_paged_cache
        q = inputs.query.transpose(-3, -2)  # [users, Hq, tokens, D]
        if attn_metadata.chunk_start_idx is not None and has_paged_cache and not shared_kv:
            # continuation chunk: keys come from the cache, prefix included
            if direct is not None:
                torch.ops.tt.chunked_scaled_dot_product_attention_out(
                    q, kv_cache[0], kv_cache[1], attn_metadata.page_table,
                    attn_metadata.chunk_start_idx, direct.transpose(-3, -2), scale=self.scale,
                )
                return None
            out = torch.ops.tt.chunked_scaled_dot_product_attention(
                q, kv_cache[0], kv_cache[1], attn_metadata.page_table,
                attn_metadata.chunk_start_idx, scale=self.scale,
            )
            return out.transpose(-3, -2)
        if shared_kv:
            k = self._gather_paged_to_dense(kv_cache[0], attn_metadata.page_table, inputs.kv_num_tokens)
            v = self._gather_paged_to_dense(kv_cache[1], attn_metadata.page_table, inputs.kv_num_tokens)
        else:
            k = inputs.key.transpose(-3, -2)
            v = inputs.value.transpose(-3, -2)
        kwargs = {
            "is_causal": attn_metadata.is_causal,
            "attn_mask": attn_metadata.attn_mask,
            "scale": self.scale,
        }
        if self.sliding_window is not None:
            kwargs["sliding_window_size"] = self.sliding_window
        if direct is not None:
            torch.ops.tt.scaled_dot_product_attention_out(q, k, v, direct.transpose(-3, -2), **kwargs)
            return None
        out = torch.ops.tt.scaled_dot_product_attention(q, k, v, **kwargs)
        return out.transpose(-3, -2)  # [users, tokens, Hq, D]

    def _gather_paged_to_dense(self, cache: torch.Tensor, page_table: torch.Tensor, num_tokens: int):
        """[NB, Hkv, bs, D] -> [users, Hkv, num_tokens, D] in page-table order (a block-float-8
        cache comes out as the bfloat16 values it encodes)."""
        users, width = page_table.shape
        # ids outside the cache (padding -1, stale entries) read block 0, as in the kernels; left
        # alone they would trip a device-side index assert
        ids = page_table.reshape(-1).to(torch.int64)
        ids = torch.where((ids >= 0) & (ids < cache.shape[0]), ids, torch.zeros_like(ids))
        g = torch.index_select(cache, 0, ids)
        if cache.dtype == torch.uint8:
            g = custom_ops.bfp8_unpack_cache(g)
        _, hkv, bs, d = g.shape
        g = g.view(users, width, hkv, bs, d).permute(0, 2, 1, 3, 4).contiguous()
        return g.reshape(users, hkv, -1, d)[:, :, :num_tokens, :]

    def _compute_decode_attention(self, inputs, kv_cache, attn_metadata: TTMetadata,
                                  fused_step: bool = False,
                                  direct: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        q = inputs.query.transpose(0, 1)  # [1, users, Hq, D]
        if fused_step:  # cache update (reference :473-483) and attention (:634-668) in one operator
            if direct is not None:
                torch.ops.tt.paged_update_kv_decode_out_(
                    q, kv_cache[0], kv_cache[1], inputs.key.transpose(0, 1), inputs.value.transpose(0, 1),
                    attn_metadata.page_table, attn_metadata.cache_position, direct.transpose(0, 1),
                    attention_sink=self.sinks, scale=self.scale, sliding_window_size=self.sliding_window,
                )
                return None
            out = torch.ops.tt.paged_update_kv_decode_(
                q, kv_cache[0], kv_cache[1], inputs.key.transpose(0, 1), inputs.value.transpose(0, 1),
                attn_metadata.page_table, attn_metadata.cache_position, attention_sink=self.sinks,
                scale=self.scale, sliding_window_size=self.sliding_window,
            )
            return out.transpose(0, 1)
        kwargs = {
            "cur_pos_tensor": attn_metadata.cache_position,
            "is_causal": attn_metadata.is_causal,
            "attn_mask": attn_metadata.attn_mask,
            "attention_sink": self.sinks,
            "scale": self.scale,
        }
        if self.sliding_window is not None:
            kwargs["sliding_window_size"] = self.sliding_window
        out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
            q, kv_cache[0], kv_cache[1], attn_metadata.page_table, **kwargs
        )
        return out.transpose(0, 1)  # [users, 1, Hq, D]
