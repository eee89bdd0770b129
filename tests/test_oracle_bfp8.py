"""Invariants that pin the block-float-8 codec (oracle/bfp8_codec.py).  The reference
holds no CPU codec for this format, so nothing here compares against it: the format is
this build's specification and these are the properties a wrong shift, a dropped sign,
a wrong rounding rule or a mis-sized group would break.
"""

import numpy as np
import pytest
import torch

from oracle import bfp8_codec as C


def _brute_encode_group(vals):
    """16 python floats (bf16-representable) -> (bytes, exponent) by the written spec,
    using exact rational arithmetic on floats (ldexp / frexp), not bit tricks."""
    import math
    from fractions import Fraction

    ex = []
    for v in vals:
        if v == 0.0 or abs(v) < 2.0**-126:
            ex.append(0)
        else:
            ex.append(math.frexp(abs(v))[1] - 1 + 127)
    e = max(ex)
    out = []
    for v, x in zip(vals, ex):
        if x == 0:
            out.append(128)
            continue
        r = Fraction(abs(v)) / (Fraction(2) ** (e - 133))
        fl = r.numerator // r.denominator
        frac = r - fl
        if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and fl % 2 == 1):
            fl += 1
        m = min(127, fl)
        out.append(128 - m if v < 0 else 128 + m)
    return out, e


def test_brute_force_small():
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(40, 32, generator=g) * torch.logspace(-3, 3, 40).view(40, 1)).to(torch.bfloat16)
    x[3, 5] = 0.0
    x[4, :16] = 0.0
    elem, exps = C.quantize(x)
    for r in range(40):
        for grp in range(2):
            vals = [float(v) for v in x[r, grp * 16 : grp * 16 + 16]]
            b, e = _brute_encode_group(vals)
            assert exps[r, grp] == e
            assert list(elem[r, grp * 16 : grp * 16 + 16]) == b


def test_representable_values_roundtrip_exactly():
    # integers up to 127 times a power of two share an exponent window -> exact
    g = torch.Generator().manual_seed(1)
    m = torch.randint(-127, 128, (64, 128), generator=g).float()
    m[:, ::16] = 127.0  # the group maximum fixes e; 127 = 1.984 * 2^6
    x = (m * 2.0**-9).to(torch.bfloat16)
    assert torch.equal(x.float(), m * 2.0**-9)
    assert torch.equal(C.roundtrip(x), x.float())


def test_requantising_decoded_values_is_identity():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(128, 128, generator=g).to(torch.bfloat16)
    elem, exps = C.quantize(x)
    dq = torch.from_numpy(C.dequantize(elem, exps))
    assert torch.equal(dq.to(torch.bfloat16).float(), dq)  # 7-bit magnitudes fit bf16
    elem2, exps2 = C.quantize(dq.to(torch.bfloat16))
    dq2 = C.dequantize(elem2, exps2)
    assert np.array_equal(dq2, dq.numpy())


def test_error_bound_half_ulp_of_group_scale():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(256, 128, generator=g).to(torch.bfloat16)
    x[:, 7] *= 20  # outlier channel
    elem, exps = C.quantize(x)
    dq = C.dequantize(elem, exps)
    bound = np.repeat(np.ldexp(1.0, exps.astype(np.int64) - 134), 16, axis=-1)
    assert np.all(np.abs(dq - x.float().numpy()) <= bound)


def test_outlier_only_coarsens_its_own_group():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(32, 64, generator=g).to(torch.bfloat16)
    y = x.clone()
    y[:, 3] *= 20
    a, b = C.roundtrip(x), C.roundtrip(y)
    assert torch.equal(a[:, 16:], b[:, 16:])
    assert not torch.equal(a[:, :16], b[:, :16])


def test_zero_group_and_signs():
    x = torch.zeros(2, 32, dtype=torch.bfloat16)
    x[1, 16:] = torch.tensor([-1.0, 1.0] * 8, dtype=torch.bfloat16)
    elem, exps = C.quantize(x)
    assert exps[0, 0] == 0 and exps[0, 1] == 0 and (elem[0] == 128).all()
    assert exps[1, 1] == 127
    assert list(elem[1, 16:18]) == [128 - 64, 128 + 64]
    assert torch.equal(C.roundtrip(x), x.float())


def test_ties_round_to_even_and_top_clamps():
    # group scale from 1.0 (e = 127): unit = 2^-6.  2^-7 = half a unit -> ties.
    u = 2.0**-6
    vals = [1.0, 0.5 * u, 1.5 * u, 2.5 * u, 0.25 * u, 0.75 * u, 1.9921875] + [0.0] * 9
    x = torch.tensor([vals], dtype=torch.bfloat16)
    assert torch.equal(x.float(), torch.tensor([vals]))
    elem, exps = C.quantize(x)
    assert exps[0, 0] == 127
    assert list(elem[0, :7]) == [128 + m for m in (64, 0, 2, 2, 0, 1, 127)]  # 127.5 -> 128 -> clamp 127


def test_inf_nan_rejected():
    x = torch.zeros(1, 16, dtype=torch.bfloat16)
    x[0, 0] = float("inf")
    with pytest.raises(ValueError):
        C.quantize(x)


def test_cache_pack_layout():
    g = torch.Generator().manual_seed(5)
    cache = torch.randn(3, 2, 32, 64, generator=g).to(torch.bfloat16)
    p = C.pack_cache(cache)
    assert p.shape == (3, 2, 34, 64) and p.dtype == torch.uint8
    elem, exps = C.quantize(cache)
    assert np.array_equal(p[:, :, :32].numpy(), elem)
    flat = p[:, :, 32:].reshape(3, 2, -1).numpy()
    assert np.array_equal(flat.reshape(3, 2, 32, 4), exps)
    assert torch.equal(C.unpack_cache(p, 32), C.roundtrip(cache))
