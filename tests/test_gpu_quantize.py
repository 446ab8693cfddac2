"""Operator 1 on the GPU against the oracle: activation codes and group scales bit for bit, the
low-rank projection to fp32 tolerance (summation order is free)."""

import pytest
import torch

from conftest import announce
from oracle import linear as olin
from oracle import quant, synth

pytestmark = pytest.mark.gpu


def _run(dev, x, layer, fp4=False, smooth=True, fuse_glu=False):
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_quantize_w4a4_act_fuse_lora

    sd = synth.to_reference_checkpoint(layer)
    out, osc, la = svdq_quantize_w4a4_act_fuse_lora(
        x.to(dev), lora_down=sd["proj_down"].to(dev), smooth=sd["smooth_factor"].to(dev) if smooth else None, fp4=fp4, fuse_glu=fuse_glu
    )
    torch.cuda.synchronize()
    K = x.shape[1] // (2 if fuse_glu else 1)
    return packing.act_to_logical(out.cpu(), K, fp4=fp4), packing.scales_to_logical(osc.cpu(), fp4), la.cpu()


def _check(x, layer, codes, osc, la, fp4=False, smooth=True):
    want_codes, want_scales, want_la = olin.quantize_act_fuse_lora(x, layer.proj_down, layer.smooth if smooth else None, fp4=fp4)
    assert codes.shape == want_codes.shape
    if fp4:
        assert torch.equal(codes.to(torch.uint8), want_codes)
        assert torch.equal(osc.view(torch.uint8), want_scales.view(torch.uint8))
    else:
        assert torch.equal(codes, want_codes), f"{(codes != want_codes).sum().item()} codes differ"
        assert torch.equal(osc.view(torch.int16), want_scales.view(torch.int16))
    scale = want_la.abs().max().item() + 1e-6
    assert (la - want_la).abs().max().item() <= 2e-5 * scale + 1e-6


@pytest.mark.parametrize("M,K,R", [(256, 256, 32), (100, 384, 16), (512, 3072, 32), (300, 1024, 128), (1, 128, 64)])
def test_int4_bit_exact(dev, M, K, R):
    announce(f"quantize int4 M={M} K={K} R={R}")
    layer = synth.make_layer(128, K, R, seed=M + K)
    x = synth.make_activations(M, K, seed=M * 7 + K)
    _check(x, layer, *_run(dev, x, layer))


def test_int4_no_smooth_and_padding_rows(dev):
    M, K, R = 70, 256, 32
    announce(f"quantize int4 no smooth M={M} K={K}")
    layer = synth.make_layer(128, K, R, seed=3)
    x = synth.make_activations(M, K, seed=3)
    codes, osc, la = _run(dev, x, layer, smooth=False)
    _check(x, layer, codes, osc, la, smooth=False)
    assert (codes[M:] == 0).all() and (osc.float()[:, M:] == 0).all() and (la[M:] == 0).all()


@pytest.mark.parametrize("fp4", [False, True])
def test_long_k_reads_smoothing_factors_from_global_memory(dev, fp4):
    """K = 16512 (129 chunks, an odd count, 66 KB of reciprocal factors): beyond what the kernel keeps in LDS."""
    M, K, R = 40, 16512, 32
    announce(f"quantize long K M={M} K={K} fp4={fp4}")
    layer = synth.make_layer(128, K, R, seed=5, fp4=fp4)
    x = synth.make_activations(M, K, seed=5)
    _check(x, layer, *_run(dev, x, layer, fp4=fp4), fp4=fp4)


def test_int4_edge_values(dev):
    # zero groups, negative zero, exact .5 ties of the smoothing quotient, huge and tiny magnitudes
    M, K, R = 256, 256, 16
    announce("quantize int4 edge values")
    layer = synth.make_layer(128, K, R, seed=11)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=g)
    x[0] = 0.0
    x[1, :64] = -0.0
    x[2] = 1e-20
    x[3] = torch.randn(K, generator=g) * 1e4
    x[4, ::2] = 0.0
    # quotients that are exact bf16 rounding ties: x = (odd 9-bit significand) * smooth
    sm = layer.smooth.float()
    x[5] = (1.00390625 * sm)  # 257/256 * s, not representable in bf16 after rounding x; exercise anyway
    x[6] = torch.round(torch.randn(K, generator=g) * 4) * 0.5
    x = x.to(torch.bfloat16)
    _check(x, layer, *_run(dev, x, layer))


def test_smoothing_quotient_all_significand_pairs(dev):
    """bf16(x / smooth) for every pair of 8-bit significands (and a few exponents): the kernel
    multiplies by the stored reciprocal, the oracle divides; they must agree bit for bit.  (A quotient
    of two 8-bit significands is never exactly a bf16 rounding midpoint -- that would need 2^8 to
    divide an odd number times a significand below 2^8 -- and otherwise stays >= 2^-16 away from
    one, so the two roundings cannot differ.)"""
    announce("quantize all significand pairs")
    for ms in range(128, 256):
        for b in range(257, 512, 2):
            assert (b * ms) % 256 != 0
    mx = torch.arange(128, 256, dtype=torch.float32) / 128.0
    ms = torch.arange(128, 256, dtype=torch.float32) / 128.0
    xs = mx.repeat(128)                     # K = 16384
    ss = ms.repeat_interleave(128)
    K = xs.numel()
    layer = synth.make_layer(128, K, 16, seed=1)
    layer.smooth = ss.to(torch.bfloat16)
    x = torch.stack([xs, -xs, xs * 4, xs * 0.125, xs * 3.0]).to(torch.bfloat16)
    assert torch.equal(x[0].float(), xs) and torch.equal(layer.smooth.float(), ss)
    _check(x, layer, *_run(dev, x, layer))


@pytest.mark.parametrize("M,K,R", [(256, 256, 32), (130, 640, 16)])
def test_nvfp4_bit_exact(dev, M, K, R):
    announce(f"quantize nvfp4 M={M} K={K} R={R}")
    layer = synth.make_layer(128, K, R, seed=M + K + 1)
    x = synth.make_activations(M, K, seed=M + 5)
    x[0, :16] = 0
    x[1, 16:32] = 3000.0
    codes, osc, la = _run(dev, x, layer, fp4=True)
    _check(x, layer, codes, osc, la, fp4=True)


def test_rejects_bad_shapes(dev):
    from nunchaku_amd.ops import svdq_quantize_w4a4_act_fuse_lora

    x = torch.zeros(16, 192, dtype=torch.bfloat16, device=dev)  # K not a multiple of 128
    with pytest.raises(ValueError):
        svdq_quantize_w4a4_act_fuse_lora(x, lora_down=torch.zeros(192, 16, dtype=torch.bfloat16, device=dev).contiguous())


def test_nvfp4_negative_zero_inputs_give_pattern_zero(dev):
    """-0.0 inputs: the reference adds a zero shift before smoothing (gemm_w4a4.cuh:986), so the E2M1 sign bit
    must not be set for them."""
    M, K, R = 64, 256, 16
    announce("quantize nvfp4 negative zeros")
    layer = synth.make_layer(128, K, R, seed=13, fp4=True)
    x = synth.make_activations(M, K, seed=13)
    x[::3, ::5] = -0.0
    x[1] = -0.0
    for smooth in (True, False):
        codes, osc, la = _run(dev, x, layer, fp4=True, smooth=smooth)
        _check(x, layer, codes, osc, la, fp4=True, smooth=smooth)
        assert (codes[1] == 0).all()


def _glu_pairs(value, gate):
    return torch.stack([value, gate], dim=2).reshape(value.shape[0], -1).to(torch.bfloat16)


@pytest.mark.parametrize("fp4", [False, True])
@pytest.mark.parametrize("M,K,R", [(256, 256, 32), (70, 640, 16), (300, 1024, 128), (40, 16512, 64)])
def test_fuse_glu_saturated_gates_bit_exact(dev, M, K, R, fp4):
    """Gates where sigmoid is 1 or 0 in fp32 whatever its approximation (|gate| >= 32): silu(gate) is the
    gate itself or minus zero, and the product value * gate has one correct bf16 rounding.  Codes, scales
    and the projection are then held to the same bar as without the gated unit; a wrong pair order or
    column mapping changes every group."""
    announce(f"quantize fuse_glu saturated gates M={M} K={K} R={R} fp4={fp4}")
    layer = synth.make_layer(128, K, R, seed=M + K, fp4=fp4)
    g = torch.Generator().manual_seed(M + K)
    value = synth.make_activations(M, K, seed=M + 3 * K).float() / 32
    gate = 32.0 + 8 * torch.rand(M, K, generator=g)
    gate[torch.rand(M, K, generator=g) < 0.1] = -120.0
    x2 = _glu_pairs(value, gate)
    assert x2.shape == (M, 2 * K)
    codes, osc, la = _run(dev, x2, layer, fp4=fp4, fuse_glu=True)
    x = olin.glu_input(x2)
    assert torch.equal(x.float(), (x2[:, 0::2].float() * torch.where(x2[:, 1::2].float() > 0, x2[:, 1::2].float(), torch.zeros(())))
                       .to(torch.bfloat16).float()), "the oracle itself: silu is the identity or zero here"
    _check(x, layer, codes, osc, la, fp4=fp4)


@pytest.mark.parametrize("fp4", [False, True])
def test_fuse_glu_random_gates(dev, fp4):
    """Ordinary gates: sigmoid comes from the hardware's exp2 and reciprocal, the oracle's from libm, so
    bf16(silu) may differ by one ulp where the fp32 value lies next to a rounding midpoint (a few elements
    in 10^4 distinct gate values, but bf16 gates have few distinct values and large gates, whose products tend
    to be a group's maximum, repeat); one bf16 step of the product is a relative 2^-8 .. 2^-7, which the smoothing division and the
    division by 7 can each land on a coarser part of a binade.  Tolerance, stated here: at most 1e-2 of the
    groups may have a different scale, none by more than 2^-6 relative (INT4, bf16 scales) or one step of
    E4M3 (NVFP4); at most 1e-2 of the codes may differ, and every INT4 code must still be the
    nearest one to the oracle's smoothed value under the kernel's own scale (half a step, plus one bf16 step
    of the value); the projection to 1e-3 of its largest magnitude."""
    M, K, R = 512, 1536, 32
    announce(f"quantize fuse_glu random gates M={M} K={K} fp4={fp4}")
    layer = synth.make_layer(128, K, R, seed=21, fp4=fp4)
    g = torch.Generator().manual_seed(21)
    x2 = _glu_pairs(synth.make_activations(M, K, seed=21).float(), 2.0 * torch.randn(M, K, generator=g))
    codes, osc, la = _run(dev, x2, layer, fp4=fp4, fuse_glu=True)
    want_codes, want_scales, want_la = olin.quantize_act_fuse_lora(x2, layer.proj_down, layer.smooth, fp4=fp4, fuse_glu=True)
    assert codes.shape == want_codes.shape == (512, K)
    if fp4:
        sc_diff = (osc.view(torch.uint8).int() - want_scales.view(torch.uint8).int()).abs()
        code_diff = codes.to(torch.uint8) != want_codes
        assert sc_diff.max().item() <= 1
    else:
        sc_diff = (osc.float() - want_scales.float()).abs()
        code_diff = codes != want_codes
        assert (sc_diff <= 2.0**-6 * want_scales.float().abs()).all()
        y = quant._smooth_divide(olin.glu_input(x2), layer.smooth, 0.0).float()
        step = osc.float().t().repeat_interleave(64, dim=1)[:M]
        assert ((codes[:M].float() * step - y).abs() <= 0.5 * step * (1 + 2.0**-6) + 2.0**-7 * y.abs()).all()
    assert (sc_diff > 0).float().mean().item() <= 1e-2
    assert code_diff.float().mean().item() <= 1e-2, f"{code_diff.sum().item()} codes differ"
    assert (la - want_la).abs().max().item() <= 1e-3 * want_la.abs().max().item()
    # and the padding rows stay zero
    assert (codes[M:] == 0).all() and (la[M:] == 0).all()


@pytest.mark.parametrize("M,K,R,fp4,smooth", [(16500, 256, 64, False, True), (16500, 384, 128, False, True), (16384, 256, 128, True, True),
                                              (16400, 256, 96, False, False), (16384, 16512, 112, False, True)])
def test_high_rank_many_rows(dev, M, K, R, fp4, smooth):
    """Ranks above 32 with at least 16384 padded rows take the variant in which the waves of a workgroup split its rows and
    share proj_down through LDS: ragged last workgroup (M = 16500: waves with some, and with no, valid rows), ranks that do
    not fill the last rank tile pair (96, 112), NVFP4, no smoothing, K beyond what LDS holds of smoothing factors.  The
    oracle runs on a sample of the rows (they are independent), all padding rows are checked to be zero."""
    announce(f"quantize high rank M={M} K={K} R={R} fp4={fp4} smooth={smooth}")
    _check_row_sample(dev, M, K, R, fp4, smooth)


@pytest.mark.parametrize("M,K,R,fp4", [(4608, 256, 32, False), (9000, 384, 32, False), (4500, 6272, 16, False), (2300, 256, 128, False),
                                       (2300, 384, 64, False), (9000, 256, 128, False), (2300, 256, 256, False), (1000, 256, 144, False),
                                       (4608, 256, 32, True), (2300, 256, 128, True), (2300, 384, 64, True), (9000, 256, 32, True)])
def test_workgroup_shapes_by_rows_and_rank(dev, M, K, R, fp4):
    """The launcher picks the workgroup's shape (waves, rows, requests ahead, rows or chunks split among the waves) by
    precision, rank, row count and row length; one case per branch of that choice beyond those the other tests take:
    32 rows on eight waves (M = 4608; long rows; ranks 64 and 128 from 8 rows per compute unit on; the windows of rank
    256), 16 rows on four waves with two chunks ahead (many short rows; NVFP4 at 4608 rows and at rank 128; few rows at
    ranks above 128), the rows-split form from 32 rows per compute unit on at rank 128."""
    announce(f"quantize workgroup shapes M={M} K={K} R={R} fp4={fp4}")
    _check_row_sample(dev, M, K, R, fp4, True)


def _check_row_sample(dev, M, K, R, fp4, smooth):
    layer = synth.make_layer(128, K, R, seed=R + K, fp4=fp4)
    x = synth.make_activations(M, K, seed=M % 1000 + K)
    codes, osc, la = _run(dev, x, layer, fp4=fp4, smooth=smooth)
    M_pad = codes.shape[0]
    g = torch.Generator().manual_seed(1)
    rows = torch.cat([torch.arange(0, 130), torch.randperm(M, generator=g)[:190], torch.arange(M - 70, M)])
    want_codes, want_scales, want_la = olin.quantize_act_fuse_lora(x[rows], layer.proj_down, layer.smooth if smooth else None, fp4=fp4)
    n = rows.numel()
    if fp4:
        assert torch.equal(codes[rows].to(torch.uint8), want_codes[:n])
        assert torch.equal(osc[:, rows].view(torch.uint8), want_scales[:, :n].view(torch.uint8))
    else:
        assert torch.equal(codes[rows], want_codes[:n])
        assert torch.equal(osc[:, rows].view(torch.int16), want_scales[:, :n].view(torch.int16))
    assert (la[rows] - want_la[:n]).abs().max().item() <= 2e-5 * want_la.abs().max().item() + 1e-6
    assert (codes[M:] == 0).all() and (osc.float()[:, M:] == 0).all() and (la[M:] == 0).all()
    assert not torch.isnan(la).any()
