"""Pins oracle/awq.py: the two derivations of the weight storage, hand-evaluated positions, and the
arithmetic against the library matmul."""

import numpy as np
import torch

from oracle import awq


def test_two_derivations_agree_and_invert():
    rng = np.random.default_rng(0)
    for oc, ic in ((4, 64), (8, 128), (16, 192)):
        codes = rng.integers(0, 16, size=(oc, ic))
        packed = awq.pack_w4(codes)
        assert packed.shape == (oc // 4, ic) and packed.dtype == np.int16
        assert np.array_equal(awq.unpack_w4(packed), codes)
        assert np.array_equal(awq.unpack_w4(packed.view(np.int32)), codes)


def test_known_positions():
    """The comment of the reference's packer: [0, 1, ..., 31] -> [0, 8, 16, 24, 1, 9, 17, 25, ...]
    (tinychat_utils.py:102): the first 16-bit word of a row holds channels 0, 8, 16, 24."""
    oc, ic = 4, 64
    codes = np.zeros((oc, ic), dtype=np.int64)
    codes[0, [0, 8, 16, 24]] = [1, 2, 3, 4]
    codes[1, 1] = 9         # row 1, second word of its 32 bytes
    codes[0, 33] = 7        # second half of the 64-block: bytes 16..31 of row 0
    words = awq.pack_w4(codes).view(np.uint16).reshape(-1)
    assert words[0] == 1 | (2 << 4) | (3 << 8) | (4 << 12)
    assert words[16 + 1] == 9           # rows are interleaved per 64 channels: row 1 starts at word 16
    assert words[8 + 1] == 7            # channel 33 = word 1 of the second group of 32


def test_gemv_against_library_matmul_and_product_rounding_is_small():
    oc, ic = 64, 256
    codes, scales, zeros, _ = awq.make_layer(oc, ic, seed=3)
    x = torch.randn(3, ic, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)
    w = awq.dequant(codes, scales, zeros)
    # one rounding: equal to the fp32 fma followed by rounding wherever that is exact, and within half a bf16 ulp of the real value
    real = codes.double() * scales.t().double().repeat_interleave(64, 1) + zeros.t().double().repeat_interleave(64, 1)
    assert ((w.double() - real).abs() <= real.abs() * 2.0**-8 + 1e-30).all()
    got = awq.gemv(x, codes, scales, zeros)
    want = torch.nn.functional.linear(x.double(), w.double()).float()
    assert torch.equal(got, want)
    lossy = awq.gemv(x, codes, scales, zeros, round_products=True)
    rel = ((lossy - got).norm() / got.norm()).item()
    assert rel < 5e-3  # the reference's bf16 products: a loss of a few 1e-4, not part of the definition


def test_against_the_reference_packer_and_converter():
    """Golden vectors written by the reference's own ``pack_w4`` and ``convert_to_tinychat_w4x16y16_linear_weight``
    (tests/golden/make_awq_vectors.py): the storage order of the codes, and the convention that the stored zero is
    minus the weight-unit zero point, so that ``code * scale + zero`` gives the weight back."""
    from pathlib import Path

    v = np.load(Path(__file__).parent / "golden" / "awq_vectors.npz")
    codes = v["codes"].astype(np.int64)
    oc, ic = codes.shape
    assert np.array_equal(awq.pack_w4(codes), v["packed"])
    assert np.array_equal(awq.unpack_w4(v["packed"]), codes)
    # the converter: a weight that is exactly (code - zero_point) * scale comes back as the same codes ...
    assert np.array_equal(awq.unpack_w4(v["qweight"]), codes)
    ng = ic // 64
    scale = torch.from_numpy(v["scale_bits"]).view(torch.bfloat16)  # [oc, ng]
    qscale = torch.from_numpy(v["qscale_bits"]).view(torch.bfloat16)  # [padded groups, oc]
    qzero = torch.from_numpy(v["qzero_bits"]).view(torch.bfloat16)
    assert torch.equal(qscale[:ng], scale.t())
    assert torch.equal(qzero[:ng].float(), -(torch.from_numpy(v["zero_point"]).float() * scale.float()).t())
    assert not qscale[ng:].any() and not qzero[ng:].any()
    # ... and the oracle's dequantization of what the converter stored is the weight, bit for bit
    w = torch.from_numpy(v["weight_bits"]).view(torch.bfloat16)
    got = awq.dequant(torch.from_numpy(codes), qscale[:ng], qzero[:ng])
    assert torch.equal(got.view(torch.int16), w.view(torch.int16))
