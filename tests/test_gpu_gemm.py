"""Operator 2 on the GPU against the oracle (fp64-accumulated dequantize-then-matmul, rounded to
bf16 where the kernel stores bf16).  Tolerance: rel-L2 <= 1e-3 and max(2e-2, 1 bf16 ulp) per element."""

import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_module, make_oracle
from oracle import linear as olin
from oracle import quant, synth

pytestmark = pytest.mark.gpu


def _gemm_case(dev, M, K, N, R, seed, bias=True, act_unsigned=False, hand_codes=False, lora_scales=None):
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    layer = synth.make_layer(N, K, R, seed=seed, bias=bias)
    g = torch.Generator().manual_seed(seed)
    M_pad = (M + 255) // 256 * 256
    if hand_codes:
        lo, hi = (0, 16) if act_unsigned else (-8, 8)
        codes = torch.randint(lo, hi, (M_pad, K), generator=g).to(torch.int8)
        layer.wq = torch.randint(-8, 8, (N, K), generator=g).to(torch.int8)  # includes -8
    else:
        x = synth.make_activations(M_pad, K, seed=seed)
        codes, _ = quant.quantize_act_int4(x, layer.smooth, unsigned=act_unsigned, shift=quant.SHIFT_GELU if act_unsigned else 0.0)
    # activation scales with a wide dynamic range across groups (outlier groups 2^6 larger)
    scales = (torch.rand(K // 64, M_pad, generator=g) * 0.5 + 0.01) * torch.where(torch.rand(K // 64, 1, generator=g) < 0.2, 64.0, 1.0)
    scales = scales.to(torch.bfloat16)
    lora_act = torch.randn(M_pad, R, generator=g) * 3 if R else None

    m = make_module(layer, dev, act_unsigned=act_unsigned)
    t = m.native_tensors()
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    svdq_gemm_w4a4(
        act=packing.logical_to_act(codes, unsigned=act_unsigned).to(dev), wgt=t["qweight"], out=out,
        ascales=scales.to(dev), wscales=t["wscales"], lora_act_in=None if lora_act is None else lora_act.to(dev),
        lora_up=t["proj_up"] if R else None, bias=t["bias"], act_unsigned=act_unsigned, lora_scales=lora_scales,
    )
    torch.cuda.synchronize()
    want = olin.gemm_w4a4(
        quant.dequant_int4(codes, scales), quant.dequant_int4(layer.wq, layer.ws), bias=layer.bias,
        lora_act_in=lora_act, lora_up=layer.proj_up if R else None, lora_scales=lora_scales,
    )[:M]
    assert not torch.isnan(out.float()).any()
    return check_output(out, want)


@pytest.mark.parametrize(
    "M,K,N,R",
    [(256, 128, 256, 32), (256, 512, 256, 16), (512, 1024, 512, 32), (100, 256, 128, 32), (300, 384, 384, 64), (256, 3072, 256, 128)],
)
def test_gemm_parity(dev, M, K, N, R):
    announce(f"gemm M={M} K={K} N={N} R={R}")
    _gemm_case(dev, M, K, N, R, seed=M + K + N)


def test_gemm_no_bias_no_lora(dev):
    announce("gemm no bias, no low-rank branch")
    _gemm_case(dev, 256, 256, 256, 0, seed=5, bias=False)


def test_gemm_extreme_codes_signed(dev):
    announce("gemm hand-made codes incl. -8")
    _gemm_case(dev, 256, 256, 256, 32, seed=6, hand_codes=True)


def test_gemm_unsigned_activations(dev):
    announce("gemm unsigned activation codes 0..15")
    _gemm_case(dev, 256, 512, 256, 32, seed=7, act_unsigned=True, hand_codes=True)
    _gemm_case(dev, 256, 512, 256, 32, seed=8, act_unsigned=True)


def test_gemm_lora_scales(dev):
    announce("gemm lora_scales per 16 ranks")
    _gemm_case(dev, 256, 256, 256, 48, seed=9, lora_scales=[0.5, 2.0, 0.0])


def test_gemm_integer_exactness(dev):
    """With unit scales the result is an integer dot product: must be exact (products and sums of
    small integers are exact in fp16 x fp16 -> fp32)."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    announce("gemm integer exactness")
    M, K, N = 256, 256, 256
    g = torch.Generator().manual_seed(1)
    codes = torch.randint(-8, 8, (M, K), generator=g).to(torch.int8)
    wq = torch.randint(-8, 8, (N, K), generator=g).to(torch.int8)
    layer = synth.make_layer(N, K, 16, seed=1, bias=False)
    layer.wq = wq
    layer.ws = torch.ones(K // 64, N, dtype=torch.bfloat16)
    m = make_module(layer, dev)
    t = m.native_tensors()
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    svdq_gemm_w4a4(act=packing.logical_to_act(codes).to(dev), wgt=t["qweight"], out=out,
                   ascales=torch.ones(K // 64, M, dtype=torch.bfloat16, device=dev), wscales=t["wscales"])
    torch.cuda.synchronize()
    want = (codes.to(torch.int32) @ wq.to(torch.int32).t()).float().to(torch.bfloat16)
    assert torch.equal(out.cpu(), want)


def test_gemm_row_scale_dynamic_range(dev):
    """Rows whose scales differ by 2^40 from each other and zero rows: the per-row power-of-two
    renormalisation must keep every row exact."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    announce("gemm row scale dynamic range")
    M, K, N = 256, 256, 128
    g = torch.Generator().manual_seed(2)
    layer = synth.make_layer(N, K, 16, seed=2, bias=False)
    codes = torch.randint(-7, 8, (M, K), generator=g).to(torch.int8)
    scales = torch.rand(K // 64, M, generator=g) + 0.5
    scales[:, 0:32] *= 2.0**-30
    scales[:, 32:64] *= 2.0**20
    scales[:, 64:70] = 0
    scales = scales.to(torch.bfloat16)
    m = make_module(layer, dev)
    t = m.native_tensors()
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    svdq_gemm_w4a4(act=packing.logical_to_act(codes).to(dev), wgt=t["qweight"], out=out, ascales=scales.to(dev), wscales=t["wscales"])
    torch.cuda.synchronize()
    want = olin.gemm_w4a4(quant.dequant_int4(codes, scales), quant.dequant_int4(layer.wq, layer.ws))
    got = out.float().cpu()
    rel_rows = (got - want.to(torch.bfloat16).float()).norm(dim=1) / want.norm(dim=1).clamp_min(1e-30)
    assert rel_rows.max().item() <= 2e-3
    assert (got[64:70] == 0).all()


def test_gemm_unsupported_raises(dev):
    from nunchaku_amd.ops import svdq_gemm_w4a4

    z = torch.zeros(256, 64, dtype=torch.uint8, device=dev)
    with pytest.raises(NotImplementedError):
        svdq_gemm_w4a4(act=z, wgt=z.view(torch.int8), ascales=z, wscales=z, out=z, poolout=z)


def test_fuse_silu_epilogue(dev):
    """fuse_silu: x * sigmoid(x) after bias and low-rank up, before the store (EpilogueSilu with
    EpilogueDefault, gemm_w4a4_launch_impl.cuh:404-417)."""
    from nunchaku_amd.ops import svdq_gemm_w4a4

    M, K, N, R = 300, 256, 384, 32
    announce(f"gemm fuse_silu M={M} K={K} N={N}")
    layer = synth.make_layer(N, K, R, seed=61)
    x = synth.make_activations(M, K, seed=61)
    m = make_module(layer, dev)
    ref = make_oracle(layer)
    qx, asc, la = m.quantize(x.to(dev))
    t = m.native_tensors()
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    svdq_gemm_w4a4(act=qx, wgt=t["qweight"], out=out, ascales=asc, wscales=t["wscales"], lora_act_in=la, lora_up=t["proj_up"],
                   bias=t["bias"], fuse_silu=True)
    torch.cuda.synchronize()
    codes, scales, lora = ref.quantize(x)
    want = olin.gemm_w4a4(quant.dequant_int4(codes, scales), ref.w_deq, bias=ref.bias, lora_act_in=lora, lora_up=ref.proj_up, silu=True)[:M]
    check_output(out, want)
    plain = m.forward_quant(qx, asc, la)[:M]  # not the identity: the plain output differs
    assert not torch.equal(plain, out)


def test_gemm_int4_per_channel_scales_and_alpha(dev):
    """INT4 with ``wcscales`` and ``alpha`` (EpilogueBias<.., USE_SCALE>, gemm_w4a4_launch_impl.cuh:174-187):
    both multiply the main term only, the bias and the low-rank term are added after."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    M, K, N, R = 256, 256, 384, 32
    announce(f"gemm INT4 wcscales + alpha M={M} K={K} N={N}")
    layer = synth.make_layer(N, K, R, seed=77)
    g = torch.Generator().manual_seed(77)
    codes = torch.randint(-8, 8, (M, K), generator=g).to(torch.int8)
    scales = (torch.rand(K // 64, M, generator=g) * 0.5 + 0.01).to(torch.bfloat16)
    lora_act = torch.randn(M, R, generator=g) * 3
    wcs = (0.25 + 2 * torch.rand(N, generator=g)).to(torch.bfloat16)
    wcs[5] = 0.0  # a zero per-channel scale leaves bias + low-rank term
    m = make_module(layer, dev)
    t = m.native_tensors()
    for alpha in (1.0, 0.625):
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        svdq_gemm_w4a4(act=packing.logical_to_act(codes).to(dev), wgt=t["qweight"], out=out, ascales=scales.to(dev), wscales=t["wscales"],
                       lora_act_in=lora_act.to(dev), lora_up=t["proj_up"], bias=t["bias"], wcscales=packing.repack_vector(
                           torch.from_numpy(__import__("oracle.layouts", fromlist=["x"]).pack_vector(wcs.view(torch.int16).numpy().view("uint16")).view("int16").copy()).view(torch.bfloat16).to(dev)),
                       alpha=alpha)
        torch.cuda.synchronize()
        want = olin.gemm_w4a4(quant.dequant_int4(codes, scales), quant.dequant_int4(layer.wq, layer.ws), bias=layer.bias,
                              lora_act_in=lora_act, lora_up=layer.proj_up, alpha=alpha, wcscales=wcs)
        check_output(out, want)
