"""NVFP4 variant (E2M1 codes, E4M3 group-16 scales, per-tensor alpha, per-channel wcscales) on the
GPU against the oracle."""

import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_module, make_oracle
from oracle import linear as olin
from oracle import quant, synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,K,N,R", [(256, 128, 256, 16), (256, 512, 384, 32), (130, 1024, 256, 32)])
def test_nvfp4_gemm_handmade_operands(dev, M, K, N, R):
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    announce(f"nvfp4 gemm M={M} K={K} N={N} R={R}")
    g = torch.Generator().manual_seed(M + K + N)
    layer = synth.make_layer(N, K, R, seed=K + N, fp4=True)
    layer.wq = torch.randint(0, 16, (N, K), generator=g).to(torch.uint8)  # every E2M1 pattern incl. -0
    layer.wcscales = (0.5 + torch.rand(N, generator=g)).to(torch.bfloat16)
    M_pad = (M + 255) // 256 * 256
    codes = torch.randint(0, 16, (M_pad, K), generator=g).to(torch.uint8)
    scales = ((torch.rand(K // 16, M_pad, generator=g) * 3 + 0.05) * torch.where(torch.rand(K // 16, 1, generator=g) < 0.2, 64.0, 1.0))
    scales = scales.clamp(max=448).to(torch.float8_e4m3fn)
    lora_act = torch.randn(M_pad, R, generator=g)
    m = make_module(layer, dev)
    t = m.native_tensors()
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    svdq_gemm_w4a4(
        act=packing.logical_to_act(codes, fp4=True).to(dev), wgt=t["qweight"], out=out,
        ascales=packing.logical_to_scales(scales, fp4=True).to(dev), wscales=t["wscales"], lora_act_in=lora_act.to(dev),
        lora_up=t["proj_up"], bias=t["bias"], fp4=True, alpha=m.alpha, wcscales=t["wcscales"],
    )
    torch.cuda.synchronize()
    want = olin.gemm_w4a4(
        quant.dequant_nvfp4(codes, scales), quant.dequant_nvfp4(layer.wq, layer.ws), bias=layer.bias, lora_act_in=lora_act,
        lora_up=layer.proj_up, alpha=float(torch.tensor(layer.wtscale).to(torch.bfloat16)), wcscales=layer.wcscales,
    )[:M]
    assert not torch.isnan(out.float()).any()
    check_output(out, want)


def test_nvfp4_layer_end_to_end(dev):
    from nunchaku_amd import packing

    M, K, N, R = 300, 768, 512, 32
    announce(f"nvfp4 layer M={M} K={K} N={N}")
    layer = synth.make_layer(N, K, R, seed=31, fp4=True)
    x = synth.make_activations(M, K, seed=31)
    m = make_module(layer, dev)
    y = m(x.to(dev).view(1, M, K))[0]
    torch.cuda.synchronize()
    ref = make_oracle(layer)
    ref.wtscale = float(torch.tensor(layer.wtscale).to(torch.bfloat16))  # the checkpoint stores wtscale as bf16
    qx, asc, la = m.quantize(x.to(dev))
    codes, scales, lora = ref.quantize(x)
    assert torch.equal(packing.act_to_logical(qx.cpu(), K, fp4=True).to(torch.uint8), codes)
    assert torch.equal(packing.scales_to_logical(asc.cpu(), True).view(torch.uint8), scales.view(torch.uint8))
    check_output(y, ref.forward_quant(codes, scales, lora)[:M])


def test_nvfp4_zero_per_channel_scale_is_refused(dev):
    """The NVFP4 kernel divides the low-rank term by the per-channel factor: a zero in wcscales is refused when the
    layer's tensors are converted, instead of silently dropping the term for that channel."""
    M, K, N, R = 256, 256, 256, 16
    announce("nvfp4 layer with a zero in wcscales")
    layer = synth.make_layer(N, K, R, seed=32, fp4=True)
    layer.wcscales = torch.ones(N, dtype=torch.bfloat16)
    layer.wcscales[5] = 0.0
    m = make_module(layer, dev)
    with pytest.raises(ValueError, match="wcscales"):
        m(synth.make_activations(M, K, seed=32).to(dev).view(1, M, K))


@pytest.mark.parametrize("M,K1,N1,R", [(256, 256, 512, 16), (2304, 256, 7680, 32), (3072, 256, 10752, 32)])
def test_nvfp4_fused_mlp_epilogue(dev, M, K1, N1, R):
    """NVFP4 GEMM producing the next layer's NVFP4 input (no shift, signed patterns).  The second shape has 270 tiles,
    which the persistent workgroups share, and 60 column chunks whose shares of the low-rank projection are added in
    order afterwards: the projection must be fully written (it starts as NaN) and the same from launch to launch.  The
    third has 504 tiles: 252 workgroups of two whole tiles each, taken in the windowed order."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    announce(f"nvfp4 next-layer epilogue M={M} K1={K1} N1={N1} R={R}")
    fc1 = synth.make_layer(N1, K1, R, seed=41, fp4=True)
    fc2 = synth.make_layer(256, N1, R, seed=42, fp4=True)
    x = synth.make_activations(M, K1, seed=41)
    m1, m2 = make_module(fc1, dev), make_module(fc2, dev)
    t1, t2 = m1.native_tensors(), m2.native_tensors()
    qx, asc, la = m1.quantize(x.to(dev))
    out = torch.empty(M, N1, dtype=torch.bfloat16, device=dev)
    qout = torch.empty(M, N1 // 2, dtype=torch.uint8, device=dev)
    osc = torch.empty(N1 // 16, M, dtype=torch.float8_e4m3fn, device=dev)
    la2 = torch.full((M, R), float("nan"), dtype=torch.float32, device=dev)

    def run():
        svdq_gemm_w4a4(act=qx, wgt=t1["qweight"], out=out, qout=qout, ascales=asc, wscales=t1["wscales"], oscales=osc,
                       lora_act_in=la, lora_up=t1["proj_up"], lora_down=t2["proj_down"], lora_act_out=la2, bias=t1["bias"],
                       smooth_factor=t2["smooth_factor"], fp4=True, alpha=m1.alpha, wcscales=t1["wcscales"])
        torch.cuda.synchronize()

    run()
    first, first_out, first_codes = la2.clone(), out.clone(), qout.clone()
    for _ in range(6):
        la2.fill_(float("nan"))
        run()
        # (which of a shared tile's workgroups finishes last changes from launch to launch; the sums must not)
        assert torch.equal(out, first_out) and torch.equal(qout, first_codes), "the output changed between two launches"
        assert torch.equal(la2, first), "the next layer's low-rank input changed between two launches"
    h = out.cpu()
    want_codes, want_scales = quant.quantize_act_nvfp4(h, fc2.smooth)
    assert torch.equal(packing.act_to_logical(qout.cpu(), N1, fp4=True).to(torch.uint8), want_codes)
    assert torch.equal(packing.scales_to_logical(osc.cpu(), True).view(torch.uint8), want_scales.view(torch.uint8))
    want_la2 = (h.double() @ fc2.proj_down.double()).float()
    assert (la2.cpu() - want_la2).abs().max().item() <= 3e-5 * want_la2.abs().max().item() + 1e-6
