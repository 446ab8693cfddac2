"""Pins the oracle's quantizers (oracle/quant.py) against what the arithmetic fixes: closed forms,
ties, saturation, zero groups, error bounds and an exhaustive sweep over every bf16 value."""

import numpy as np
import torch

from oracle import quant


def _bf(x):
    return torch.tensor(x, dtype=torch.float32).to(torch.bfloat16)


def test_constants():
    assert np.float32(quant.RECIP_7).view(np.uint32) == 0x3E124925
    assert np.float32(quant.RECIP_15).view(np.uint32) == 0x3D888889
    assert quant.SHIFT_GELU == 11 / 64  # exactly representable in bf16
    assert float(_bf([quant.SHIFT_GELU])[0]) == quant.SHIFT_GELU


def test_int4_known_answers():
    # one group whose absmax is 7: 7 * fl32(1/7) = 1.0000000447 rounds to 1.0 in fp32, so s = 1, r = 1 and
    # the codes are the inputs rounded half to even (worked out by hand, literal)
    x = torch.zeros(1, 64)
    x[0, :8] = torch.tensor([7.0, -7.0, 3.5, 2.5, 1.5, 0.5, -0.5, -3.5])
    codes, scales = quant.quantize_act_int4(x.to(torch.bfloat16))
    assert scales.shape == (1, 1)
    assert scales[0, 0].view(torch.int16).item() == 0x3F80  # bf16 1.0
    assert codes[0, :8].tolist() == [7, -7, 4, 2, 2, 0, 0, -4]
    assert codes[0, 8:].abs().max() == 0
    # absmax 3 -> s = 3 * fl32(1/7) = 0.42857146 (stored bf16 0x3EDB = 0.427734375), r = 2.3333333:
    # 1 -> 2.33 -> 2, 2 -> 4.67 -> 5, -0.75 -> -1.75 -> -2
    x2 = torch.zeros(1, 64)
    x2[0, :4] = torch.tensor([3.0, 1.0, 2.0, -0.75])
    codes2, scales2 = quant.quantize_act_int4(x2.to(torch.bfloat16))
    assert scales2[0, 0].view(torch.int16).item() == 0x3EDB
    assert codes2[0, :4].tolist() == [7, 2, 5, -2]


def test_int4_ties_round_half_even():
    # amax = 14 -> s = 2 up to rounding; make s exactly 2 by checking, then 1.0/3.0/5.0 are ties
    x = torch.zeros(1, 64)
    x[0, :5] = torch.tensor([14.0, 1.0, 3.0, 5.0, -5.0])
    codes, scales = quant.quantize_act_int4(x.to(torch.bfloat16))
    # 14 * fl32(1/7) = 2.00000009 rounds to 2.0: r = 0.5 and 0.5, 1.5, 2.5, -2.5 are exact ties -> 0, 2, 2, -2
    assert scales[0, 0].view(torch.int16).item() == 0x4000
    assert codes[0, :5].tolist() == [7, 0, 2, 2, -2]


def test_int4_unsigned_shift_and_clamp():
    x = torch.full((2, 64), -1.0)
    x[0, 0] = 15.0
    x[1, :] = torch.linspace(0, 3, 64)
    codes, scales = quant.quantize_act_int4(x.to(torch.bfloat16), unsigned=True, shift=quant.SHIFT_GELU)
    assert codes.min() >= 0 and codes.max() <= 15
    assert codes[0, 1:].max() == 0  # negative inputs clamp to 0
    assert codes[0, 0] == 15
    # scale uses 1/15 of the shifted absmax: bf16(15 + 0.171875) = 15.1875, times fl32(1/15) = 1.0125,
    # stored bf16 1.015625 (0x3F82)
    assert scales[0, 0].view(torch.int16).item() == 0x3F82
    # row 1: -1 + 0.171875 < 0 nowhere (linspace 0..3): largest shifted value bf16(3.171875) = 3.171875 -> code 15
    assert codes[1, 63] == 15 and codes[1, 0] == 1  # 0.171875 / (3.171875 / 15) = 0.81 -> 1


def test_int4_zero_group_and_invariants():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(8, 256, generator=g)
    x[3, 64:128] = 0
    sm = (0.5 + 1.5 * torch.rand(256, generator=g)).to(torch.bfloat16)
    xb = x.to(torch.bfloat16)
    codes, scales = quant.quantize_act_int4(xb, sm)
    assert codes[3, 64:128].abs().max() == 0 and float(scales[1, 3]) == 0.0
    assert codes.min() >= -7 - 1 and codes.max() <= 7
    # dequant error <= scale/2, plus |code| <= 7 times the bf16 rounding of the stored scale (2^-9 relative)
    y = quant.bf16(xb.float() / sm.float()[None, :])
    deq = quant.dequant_int4(codes, scales)
    s = scales.float().t().repeat_interleave(64, dim=1)
    assert ((y - deq).abs() <= s * (0.5 + 7 * 2**-8) + 1e-30).all()


def test_int4_single_value_group_exhaustive_bf16():
    # every finite bf16 value alone in its group: |code| must be 7 (or 0 for zero), sign kept
    bits = torch.arange(0, 1 << 16, dtype=torch.int32)
    vals = (bits << 16).view(torch.float32)
    finite = torch.isfinite(vals) & (vals.abs() < 1e30) & ((vals.abs() > 1e-30) | (vals == 0))
    vals = vals[finite]
    x = torch.zeros(vals.numel(), 64)
    x[:, 0] = vals
    codes, scales = quant.quantize_act_int4(x.to(torch.bfloat16))
    want = torch.sign(vals) * 7
    assert torch.equal(codes[:, 0].float(), want)
    assert (codes[:, 1:] == 0).all()


def test_smooth_divide_is_ieee():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4, 64, generator=g).to(torch.bfloat16)
    sm = (0.5 + 1.5 * torch.rand(64, generator=g)).to(torch.bfloat16)
    y = quant._smooth_divide(x, sm, 0.0)
    want = (x.double() / sm.double()[None, :]).float().to(torch.bfloat16).float()  # double->float is exact enough here
    assert torch.equal(y, want)


def test_e2m1_table_brute_force():
    grid = torch.tensor(quant.E2M1_VALUES)
    v = torch.linspace(-7, 7, 28001)
    code = quant.e2m1_encode(v)
    dec = quant.e2m1_decode(code)
    # nearest grid point (saturating)
    d = (v.abs()[:, None] - grid[None, :]).abs()
    best = d.min(dim=1).values
    assert torch.allclose((dec.abs() - v.abs()).abs(), best, atol=0)
    # ties go to the even pattern
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    assert quant.e2m1_encode(ties).tolist() == [0, 2, 2, 4, 4, 6, 6]
    assert quant.e2m1_encode(-ties).tolist() == [8, 10, 10, 12, 12, 14, 14]
    assert quant.e2m1_encode(torch.tensor([100.0, -100.0])).tolist() == [7, 15]


def test_nvfp4_known_answers():
    x = torch.zeros(1, 32)
    x[0, :4] = torch.tensor([6.0, 3.0, -1.5, 0.5])
    x[0, 16] = 4000.0  # scale saturates at 448
    codes, scales = quant.quantize_act_nvfp4(x.to(torch.bfloat16))
    assert scales.dtype == torch.float8_e4m3fn and scales.shape == (2, 1)
    # 6 * fl32(1/6) = 1.00000003 rounds to 1.0: scale e4m3 1.0 (0x38), codes are the E2M1 patterns of the inputs:
    # 6 -> 7, 3 -> 5, -1.5 -> sign | 3 = 11, 0.5 -> 1
    assert scales[0, 0].view(torch.uint8).item() == 0x38
    assert codes[0, :4].tolist() == [7, 5, 11, 1]
    assert scales[1, 0].view(torch.uint8).item() == 0x7E and float(scales[1, 0].float()) == 448.0
    assert codes[0, 16] == 7  # 4000/448 saturates to 6
    assert (codes[0, 17:] == 0).all()


def test_pack_unpack_nibbles():
    c = torch.randint(-8, 8, (4, 64), generator=torch.Generator().manual_seed(0)).to(torch.int8)
    p = quant.pack_nibbles(c)
    assert p.shape == (4, 32)
    assert torch.equal(quant.unpack_nibbles(p, signed=True), c)
    assert int(p[0, 0]) == ((int(c[0, 0]) & 15) | ((int(c[0, 1]) & 15) << 4))


def test_weight_quantizer_roundtrip_error():
    w = 0.02 * torch.randn(128, 128, generator=torch.Generator().manual_seed(2))
    wq, ws = quant.quantize_weight_int4(w)
    assert wq.abs().max() <= 7 and ws.shape == (2, 128)
    err = (quant.dequant_int4(wq, ws) - w).abs()
    assert (err <= ws.float().t().repeat_interleave(64, dim=1) * 0.51).all()
