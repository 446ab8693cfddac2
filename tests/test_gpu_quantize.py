"""Operator 1 on the GPU against the oracle: activation codes and group scales bit for bit, the
low-rank projection to fp32 tolerance (summation order is free)."""

import pytest
import torch

from conftest import announce
from oracle import linear as olin
from oracle import quant, synth

pytestmark = pytest.mark.gpu


def _run(dev, x, layer, fp4=False, smooth=True):
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_quantize_w4a4_act_fuse_lora

    sd = synth.to_reference_checkpoint(layer)
    out, osc, la = svdq_quantize_w4a4_act_fuse_lora(
        x.to(dev), lora_down=sd["proj_down"].to(dev), smooth=sd["smooth_factor"].to(dev) if smooth else None, fp4=fp4
    )
    torch.cuda.synchronize()
    return packing.act_to_logical(out.cpu(), x.shape[1], fp4=fp4), packing.scales_to_logical(osc.cpu(), fp4), la.cpu()


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
