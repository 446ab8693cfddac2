"""Pins ``oracle/linear.py`` (the CPU restatement every GEMM / epilogue / fused-MLP parity test compares
against) with answers worked out by hand: every expected number below is a literal, none is recomputed
with the oracle's own formula.  Each case is built so that a plausible mis-statement changes the answer:
per-channel scales applied to the bias or to the low-rank term, the bf16 rounding of ``lora_act * scale``
left out, ``lora_scales`` indexed per rank instead of per 16 ranks, the low-rank projection taken from the
smoothed or the shifted input, padding rows not zero, the GELU constants, the order bias -> low-rank ->
activation function."""

import pytest
import torch

from oracle import linear as olin
from oracle import quant


def test_gemm_epilogue_order_with_literal_answers():
    # 2 tokens, K = 2, N = 2, identity weights: acc = act
    act = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    wgt = torch.eye(2)
    bias = torch.tensor([10.0, 20.0])
    wcs = torch.tensor([2.0, 3.0])
    R = 32
    la = torch.zeros(2, R)
    la[0, 0] = 1.00390625  # 1 + 2^-8: a bf16 tie, rounds to 1.0 (scale 1)
    la[0, 16] = 3.0        # second group of 16 ranks: scale 0.5 -> 1.5
    up = torch.zeros(2, R)
    up[0, 0] = 2.0
    up[1, 16] = 4.0
    out = olin.gemm_w4a4(act, wgt, bias=bias, lora_act_in=la, lora_up=up, lora_scales=[1.0, 0.5], alpha=0.5, wcscales=wcs)
    # main term: act * 0.5 * wcs = [[1, 3], [3, 6]]; + bias = [[11, 23], [13, 26]];
    # low-rank: row 0: bf16(1.00390625) * 2 = 2 on column 0, bf16(3 * 0.5) * 4 = 6 on column 1 (not scaled by wcs)
    assert out.dtype == torch.float32
    assert out.tolist() == [[13.0, 29.0], [13.0, 26.0]]
    # without the bf16 rounding of lora_act * scale column 0 would be 13.015625; with wcs on the low-rank term 15
    # lora_scales defaults to ones
    out1 = olin.gemm_w4a4(act, wgt, bias=bias, lora_act_in=la, lora_up=up)
    assert out1.tolist() == [[1.0 + 10.0 + 2.0, 2.0 + 20.0 + 12.0], [13.0, 24.0]]
    # a scale list shorter than the rank groups leaves the remaining groups out (svdq_gemm_w4a4 pads with zeros)
    out2 = olin.gemm_w4a4(act, wgt, lora_act_in=la, lora_up=up, lora_scales=[1.0])
    assert out2.tolist() == [[3.0, 2.0], [3.0, 4.0]]


def test_gemm_activation_functions_come_last_and_match_literal_values():
    # bias moves the argument of the activation function: gelu(acc + bias), not gelu(acc) + bias
    act = torch.tensor([[1.0], [-3.0], [0.5]])
    wgt = torch.tensor([[1.0]])
    out = olin.gemm_w4a4(act, wgt, bias=torch.tensor([1.0]), gelu=True)  # arguments 2, -2, 1.5
    # tanh-GELU x (0.5 + 0.5 tanh(0.79788456 (x + 0.044715 x^3))) (epilogues.cuh:22-44), evaluated by hand in double
    assert out[:, 0].tolist() == pytest.approx([1.9545976939197902, -0.04540230608020978, 1.3995715767318297], abs=2e-6)
    g = olin.gemm_w4a4(torch.tensor([[1.0], [-1.0], [2.0], [3.0], [-3.0], [0.5], [0.0]]), wgt, gelu=True)[:, 0]
    want = [0.8411919903841787, -0.15880800961582126, 1.9545976939197902, 2.9963626078936834, -0.0036373921063166947, 0.34571400973853866, 0.0]
    assert g.tolist() == pytest.approx(want, abs=2e-6)
    s = olin.gemm_w4a4(torch.tensor([[1.0], [-2.0], [4.0], [0.0]]), wgt, silu=True)[:, 0]
    assert s.tolist() == pytest.approx([0.7310585786300049, -0.2384058440442351, 3.928055160151634, 0.0], abs=2e-6)
    # the low-rank term is inside the activation function too
    la = torch.zeros(1, 16)
    la[0, 0] = 1.0
    up = torch.zeros(1, 16)
    up[0, 0] = 1.0
    both = olin.gemm_w4a4(torch.tensor([[1.0]]), wgt, lora_act_in=la, lora_up=up, gelu=True)
    assert both.item() == pytest.approx(1.9545976939197902, abs=2e-6)  # gelu(1 + 1), not gelu(1) + 1 = 1.841


def test_quantize_act_fuse_lora_padding_and_unsmoothed_projection():
    K, R = 64, 16
    x = torch.zeros(3, K)
    x[0, 0] = 7.0
    x[1, 5] = -14.0
    x[2, 63] = 1.0
    smooth = torch.full((K,), 2.0, dtype=torch.bfloat16)
    down = torch.zeros(K, R, dtype=torch.bfloat16)
    down[0, 0] = 1.0
    down[5, 1] = 0.5
    codes, scales, lora = olin.quantize_act_fuse_lora(x.to(torch.bfloat16), down, smooth)
    assert codes.shape == (256, K) and scales.shape == (1, 256) and lora.shape == (256, R) and lora.dtype == torch.float32
    # row 0: y = 3.5, s = 3.5 * fl32(1/7) = 0.5 exactly, code 7; row 1: y = -7, s = 1, code -7; row 2: y = 0.5, code 7
    assert codes[0, 0] == 7 and codes[1, 5] == -7 and codes[2, 63] == 7
    assert scales[0, :3].float().tolist() == [0.5, 1.0, 0.0712890625]  # bf16(0.5 / 7) = 0x3D92
    assert int(codes[:3].abs().sum()) == 21
    # rows 3 .. 255 do not exist: zero-filled by the loader, so code 0, scale 0, projection 0
    assert int(codes[3:].abs().sum()) == 0 and float(scales[0, 3:].float().abs().sum()) == 0 and float(lora[3:].abs().sum()) == 0
    # the projection sees the raw x (7, -14), not x / smooth (3.5, -7)
    assert lora[0, 0] == 7.0 and lora[1, 1] == -7.0 and float(lora[:3].abs().sum()) == 14.0
    # NVFP4 flavour: 16-wide groups, e4m3 scales
    c4, s4, l4 = olin.quantize_act_fuse_lora(x.to(torch.bfloat16), down, None, fp4=True)
    assert c4.shape == (256, K) and s4.shape == (4, 256) and s4.dtype == torch.float8_e4m3fn
    # row 0: amax 7 -> s = fl32(7/6) = 1.1666..., stored e4m3 1.125; code = e2m1(7 / 1.1666) = e2m1(6) = 7
    assert c4[0, 0] == 7 and float(s4[0, 0].float()) == 1.125 and float(s4[1, 0].float()) == 0.0
    assert l4[0, 0] == 7.0


def _identity_layer(K, N, R, down_entry=None, up_entry=None, bias=None):
    """wq = 4 I with scale 0.25: the dequantized weight is exactly the identity."""
    wq = (4 * torch.eye(N, K)).to(torch.int8)
    ws = torch.full((K // 64, N), 0.25, dtype=torch.bfloat16)
    down = torch.zeros(K, R, dtype=torch.bfloat16)
    up = torch.zeros(N, R, dtype=torch.bfloat16)
    if down_entry:
        down[down_entry[0], down_entry[1]] = down_entry[2]
    if up_entry:
        up[up_entry[0], up_entry[1]] = up_entry[2]
    return olin.FakeQuantLinear(wq, ws, torch.ones(K, dtype=torch.bfloat16), down, up, bias)


def test_glu_input_literal_answers():
    # pairs (value, gate).  silu(1) = 0.7310586 -> bf16 0.73046875 (187 * 2^-8); silu(-1) = -0.2689414 -> bf16
    # -0.26953125 (138 * 2^-9); silu(2) = 1.7615942 -> bf16 1.7578125 (225 * 2^-7); silu(0) = 0
    x = torch.tensor([[2.0, 1.0, 3.0, -1.0, 1.0, 2.0, 5.0, 0.0, 1.0078125, 1.0, -4.0, 1.0]], dtype=torch.bfloat16)
    got = olin.glu_input(x)
    # 2 * 0.73046875; 3 * -0.26953125 (exact in bf16); 1 * 1.7578125 (value and gate exchanged: not 1.4609375);
    # 5 * 0; (1 + 2^-7) * 0.73046875 = 0.7361755 -> bf16 0.734375 (188 * 2^-8); -4 * 0.73046875
    want = torch.tensor([[1.4609375, -0.80859375, 1.7578125, 0.0, 0.734375, -2.921875]])
    assert got.dtype == torch.bfloat16 and torch.equal(got.float(), want)
    # (the fifth pair also fixes that silu is rounded to bf16 before the product: with silu(1) kept in fp32 it would be
    # (1 + 2^-7) * 0.7310586 = 0.73677 -> bf16 0.73828125)
    # through the whole operator: the low-rank projection sees the product, not the raw columns
    x = torch.zeros(1, 256, dtype=torch.bfloat16)
    x[0, 0], x[0, 1] = 2.0, 1.0   # column 0 of the product: 1.4609375
    x[0, 2], x[0, 3] = 3.0, -1.0  # column 1: -0.80859375
    down = torch.zeros(128, 16, dtype=torch.bfloat16)
    down[0, 0], down[1, 0], down[1, 1] = 1.0, 1.0, 2.0
    codes, scales, la = olin.quantize_act_fuse_lora(x, down, None, fuse_glu=True)
    assert codes.shape == (256, 128) and scales.shape == (2, 256)
    assert la[0, 0].item() == 1.4609375 - 0.80859375 and la[0, 1].item() == -1.6171875
    # group scale = bf16(1.4609375 / 7) = bf16(0.208705) = 0.208984375 (214 * 2^-10); codes rne(1.4609375 / 0.20870535) = 7,
    # rne(-0.80859375 / 0.20870535 = -3.874) = -4
    assert scales[0, 0].item() == 0.208984375 and codes[0, :3].tolist() == [7, -4, 0]


def test_fake_quant_linear_literal():
    lin = _identity_layer(64, 64, 16, down_entry=(0, 0, 1.0), up_entry=(1, 0, 2.0), bias=torch.arange(64, dtype=torch.float32).to(torch.bfloat16))
    x = torch.zeros(2, 64)
    x[0, 0] = 7.0   # s = 1, code 7, dequantized 7
    x[1, 2] = -3.5  # s = 0.5, code -7, dequantized -3.5
    y = lin.forward(x.to(torch.bfloat16))
    assert y.shape == (2, 64)
    want = torch.arange(64, dtype=torch.float32).repeat(2, 1)  # bias
    want[0, 0] += 7.0
    want[1, 2] += -3.5
    want[0, 1] += 7.0 * 2.0  # low-rank: (x @ down)[0, 0] = 7, times up[1, 0] = 2
    assert torch.equal(y, want)


def test_fused_gelu_mlp_shift_unsigned_and_unshifted_projection():
    fc1 = _identity_layer(64, 64, 16)
    fc2 = _identity_layer(64, 64, 16, down_entry=(0, 0, 1.0), up_entry=(0, 0, 1.0))
    x = torch.zeros(1, 64)
    x[0, 0] = 7.0
    out, mid = olin.fused_gelu_mlp(x.to(torch.bfloat16), fc1, fc2)
    # fc1: dequantized input 7 -> identity -> gelu(7) = 7 (tanh saturates), gelu(0) = 0
    assert mid["h"].shape == (256, 64) and mid["h"][0, 0] == 7.0 and float(mid["h"].abs().sum()) == 7.0
    # fc2's low-rank input comes from the UNSHIFTED tile: 7, not 7.171875
    assert mid["lora2"][0, 0] == 7.0 and float(mid["lora2"].abs().sum()) == 7.0
    # fc2's quantizer: bf16(7 + 0.171875) = 7.1875 (a tie, to even); the zeros become 0.171875;
    # s = 7.1875 * fl32(1/15) = 0.4791667, stored bf16 0.478515625 (0x3EF5); codes 15 and rne(0.171875 / s) = 0
    assert mid["qcodes"].dtype == torch.int8 and mid["qcodes"][0, 0] == 15 and int(mid["qcodes"][0, 1:].sum()) == 0
    assert mid["qscales"].shape == (1, 256) and mid["qscales"][0, 0].view(torch.int16).item() == 0x3EF5
    # padding rows: h = gelu(0) = 0, shifted 0.171875 in every column -> s = 0.171875 / 15, codes all 15
    assert int(mid["qcodes"][1].min()) == 15 and mid["qscales"][0, 1].view(torch.int16).item() == 0x3C3C  # bf16(0.011458334)
    # fc2: unsigned code 15 dequantized literally (15 * 0.478515625 = 7.177734375) + low-rank 7 * 1
    assert out.shape == (1, 64)
    assert out[0, 0].item() == 14.177734375 and float(out[0, 1:].abs().sum()) == 0.0


def test_rows_are_independent_and_linear_in_the_weights():
    """Properties the definition fixes: a row's output depends on that row only; doubling every weight
    scale doubles the main term."""
    g = torch.Generator().manual_seed(0)
    codes = torch.randint(-8, 8, (4, 128), generator=g).to(torch.int8)
    scales = (torch.rand(2, 4, generator=g) + 0.5).to(torch.bfloat16)
    wq = torch.randint(-8, 8, (8, 128), generator=g).to(torch.int8)
    ws = (torch.rand(2, 8, generator=g) + 0.5).to(torch.bfloat16)
    a = quant.dequant_int4(codes, scales)
    full = olin.gemm_w4a4(a, quant.dequant_int4(wq, ws))
    for r in range(4):
        assert torch.equal(olin.gemm_w4a4(a[r:r + 1], quant.dequant_int4(wq, ws)), full[r:r + 1])
    assert torch.equal(olin.gemm_w4a4(a, quant.dequant_int4(wq, (ws.float() * 2).to(torch.bfloat16))), 2 * full)
    # and the integer core: unit scales give the integer matrix product exactly
    ones_a, ones_w = torch.ones(2, 4, dtype=torch.bfloat16), torch.ones(2, 8, dtype=torch.bfloat16)
    want = (codes.to(torch.int32) @ wq.to(torch.int32).t()).float()
    assert torch.equal(olin.gemm_w4a4(quant.dequant_int4(codes, ones_a), quant.dequant_int4(wq, ones_w)), want)


def test_litela_literal_answers():
    """One head (N = 96), two batch entries of two rows each.  Column order [q 32 | k 32 | v 32], the ReLU on q and
    k but not on v, v index = row of vk and k index = column, the ones row, the batch split: all by hand."""
    out = torch.zeros(4, 96)
    # batch 0, row 0: q0 = -1 (ReLU -> 0), q1 = 2; k0 = 3, k1 = -5 (ReLU -> 0); v0 = -2, v3 = 0.5
    out[0, 0], out[0, 1] = -1.0, 2.0
    out[0, 32], out[0, 33] = 3.0, -5.0
    out[0, 64], out[0, 67] = -2.0, 0.5
    # batch 0, row 1: k0 = 1, k2 = 4; v0 = 10
    out[1, 32], out[1, 34] = 1.0, 4.0
    out[1, 64] = 10.0
    # batch 1, row 0 (row 2 of the GEMM): k5 = 1.00390625 (bf16 tie -> 1.0), v7 = 7
    out[2, 32 + 5] = 1.00390625
    out[2, 64 + 7] = 7.0
    q, vk = olin.litela(out, batch=2)
    assert q.shape == (2, 2, 32) and vk.shape == (2, 1, 33, 32)
    assert q[0, 0, 0] == 0.0 and q[0, 0, 1] == 2.0 and q.abs().sum() == 2.0
    want = torch.zeros(33, 32, dtype=torch.float64)
    want[0, 0] = -2.0 * 3.0 + 10.0 * 1.0   # v0 k0 over both rows = 4
    want[0, 2] = 10.0 * 4.0                # v0 k2
    want[3, 0] = 0.5 * 3.0                 # v3 k0
    want[32, 0] = 3.0 + 1.0                # sums of relu(k)
    want[32, 2] = 4.0
    assert torch.equal(vk[0, 0], want)     # (k1 = -5 contributes nowhere: not to row 0, not to the sums)
    want1 = torch.zeros(33, 32, dtype=torch.float64)
    want1[7, 5] = 7.0
    want1[32, 5] = 1.0
    assert torch.equal(vk[1, 0], want1)


def test_linearattn_vk_mul_q_literal_answers():
    vk = torch.zeros(1, 2, 33, 32)
    vk[0, 0, 0, 0], vk[0, 0, 0, 1] = 2.0, 1.0     # o[0] = 2 q0 + q1
    vk[0, 0, 5, 1] = 3.0                          # o[5] = 3 q1
    vk[0, 0, 32, 0], vk[0, 0, 32, 1] = 1.0, 1.0   # denominator q0 + q1
    vk[0, 1, 1, 0] = 4.0                          # head 1: o[1] = 4 q0, denominator 0 + eps
    q = torch.zeros(1, 3, 64)
    q[0, 0, 0], q[0, 0, 1] = 1.0, 3.0             # head 0 of token 0
    q[0, 0, 32] = 0.5                             # head 1 of token 0
    q[0, 2, 0] = 9.0                              # token 2 is beyond num_tokens
    got = olin.linearattn_vk_mul_q(q, vk, num_tokens=2, eps=0.25)
    assert got[0, 0, 0].item() == 5.0 / 4.25 and got[0, 0, 5].item() == 9.0 / 4.25
    assert got[0, 0, 33].item() == 2.0 / 0.25
    assert got[0, 2, 0].item() == 9.0 and got[0, 1].abs().sum() == 0.0
    assert got[0, 0].count_nonzero() == 3
