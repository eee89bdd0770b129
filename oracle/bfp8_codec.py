"""Block-float-8 KV codec (numpy, integer arithmetic).  TEST INFRASTRUCTURE.

PARITY UNPINNED against the reference: tt-xla only forwards the option
``experimental_kv_cache_dtype="bfp_bf8"`` (vllm_tt/platform.py:165, 232-233;
pjrt_implementation/src/api/module_builder/module_builder.cc:1050-1063) to a
compiler that is not vendored; no CPU quantiser exists in the reference.  The only
in-repo evidence of the format is the tile size 32*32 + 64 bytes
(python_package/tt_torch/tt_lang.py:738): one shared 8-bit exponent per 16 values.
The codec is therefore specified here and pinned by invariants (tests/test_oracle_bfp8.py).

Format
------
A group is 16 consecutive head-dim elements of one token.  Per group one byte ``e``
(the largest biased bfloat16 exponent in the group) and per element one byte
``b = 128 + v`` with the signed 7-bit mantissa ``v`` in [-127, 127] (offset binary:
one byte permute turns it into a half-precision number on the device, no sign
handling).  The decoded value is

    (b - 128) * 2^(e - 133)             (133 = 127 bias + 6 fraction bits)

so the largest element keeps its hidden bit plus 6 fraction bits.  Byte 0 (v = -128)
is never produced by the encoder but decodes by the same formula; a zero-filled,
never written cache therefore reads as -2^-126 per element, not as 0.  Encoding a
bfloat16 with exponent field ``ex`` and 8-bit significand ``sig = 128 | frac``:
``|v| = min(127, rne(sig >> (e - ex + 1)))`` with round-half-to-even on the bits
shifted out; ``ex == 0`` (zero / subnormal, either sign) encodes as v = 0.  Inf / NaN inputs are
rejected here (the device kernel does not check).

Cache layout
------------
A bf16 cache ``[NB, Hkv, bs, D]`` becomes uint8 ``[NB, Hkv, bs + bs//16, D]``: rows
``0..bs-1`` hold the element bytes of token ``t``; the remaining ``bs//16`` rows, read
as a flat ``[bs, D//16]`` array, hold the exponent byte of (token, group).
"""

from __future__ import annotations

import numpy as np
import torch

GROUP = 16


def _bits(x: torch.Tensor) -> np.ndarray:
    assert x.dtype == torch.bfloat16, "codec input is bfloat16"
    return x.contiguous().view(torch.int16).numpy().astype(np.uint16)


def quantize(x: torch.Tensor):
    """bf16 [..., D] -> (elem uint8 [..., D], exps uint8 [..., D//16])."""
    b = _bits(x).astype(np.int64)
    d = b.shape[-1]
    assert d % GROUP == 0
    sign = (b >> 15) & 1
    ex = (b >> 7) & 0xFF
    frac = b & 0x7F
    if np.any(ex == 255):
        raise ValueError("Inf/NaN cannot be block-float encoded")
    g = ex.reshape(*ex.shape[:-1], d // GROUP, GROUP)
    e = g.max(axis=-1)  # [..., D/16]
    e_full = np.repeat(e, GROUP, axis=-1)
    sig = np.where(ex == 0, 0, 128 | frac)
    sh = e_full - ex + 1  # >= 1
    sh = np.minimum(sh, 16)  # anything >= 10 shifts an 8-bit value to zero
    q = sig >> sh
    rem = sig & ((1 << sh) - 1)
    half = 1 << (sh - 1)
    up = (rem > half) | ((rem == half) & ((q & 1) == 1))
    m = np.minimum(q + up.astype(np.int64), 127)
    elem = (128 + np.where(sign == 1, -m, m)).astype(np.uint8)
    # a group of zeros / subnormals has e == 0 and all v == 0 already
    return elem, e.astype(np.uint8)


def dequantize(elem: np.ndarray, exps: np.ndarray) -> np.ndarray:
    """(elem uint8 [..., D], exps uint8 [..., D//16]) -> float32 [..., D] (exact)."""
    v = elem.astype(np.float64) - 128.0
    e = np.repeat(exps.astype(np.int64), GROUP, axis=-1)
    return np.ldexp(v, e - 133).astype(np.float32)


def pack_cache(cache: torch.Tensor) -> torch.Tensor:
    """bf16 [NB, Hkv, bs, D] -> uint8 [NB, Hkv, bs + bs//16, D] (layout above)."""
    nb, h, bs, d = cache.shape
    assert bs % GROUP == 0 and d % GROUP == 0
    elem, exps = quantize(cache)
    out = np.zeros((nb, h, bs + bs // GROUP, d), dtype=np.uint8)
    out[:, :, :bs, :] = elem
    out[:, :, bs:, :] = exps.reshape(nb, h, bs // GROUP, d)
    return torch.from_numpy(out)


def unpack_cache(packed: torch.Tensor, block_size: int) -> torch.Tensor:
    """uint8 [NB, Hkv, bs + bs//16, D] -> float32 [NB, Hkv, bs, D]."""
    p = packed.numpy()
    nb, h, rows, d = p.shape
    bs = block_size
    assert rows == bs + bs // GROUP
    elem = p[:, :, :bs, :]
    exps = p[:, :, bs:, :].reshape(nb, h, bs, d // GROUP)
    return torch.from_numpy(dequantize(elem, exps))


def roundtrip(x: torch.Tensor) -> torch.Tensor:
    """bf16 [..., D] -> float32 [..., D] after encode + decode."""
    elem, exps = quantize(x)
    return torch.from_numpy(dequantize(elem, exps))
