"""Output tiles split along K (the INT4 GEMM does this when there are too few tiles to occupy the chip, or
when asked through ``k_split``): every part parks its fp32 partial sums in the workspace and the last
one to arrive adds all parts in ascending order.  Compared with the same launches unsplit, and with the
oracle.

What could go wrong and what catches it: a partial sum read before it is complete or from a stale cache
line (alternating inputs between launches: a stale read would return the other input's sums), a k-range
counted twice or not at all (the unsplit launch computes every tile in one piece), parts of a single
k-group (k_split = K / 64), an arrival counter left non-zero (eight launches in a row on one workspace),
a result that depends on the order of arrival (two runs of the same input must agree bit for bit)."""

import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_module
from oracle import linear as olin
from oracle import quant, synth

pytestmark = pytest.mark.gpu


def _inputs(M_pad, K, R, seed):
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(-8, 8, (M_pad, K), generator=g).to(torch.int8)
    scales = (torch.rand(K // 64, M_pad, generator=g) * 0.5 + 0.01).to(torch.bfloat16)
    lora_act = torch.randn(M_pad, R, generator=g) * 3
    return codes, scales, lora_act


@pytest.mark.parametrize(
    "M,K,N,R,k_split",
    [(256, 3072, 3072, 32, None), (512, 12288, 512, 32, None), (256, 1024, 512, 16, 4), (512, 12288, 256, 32, 24), (300, 640, 768, 32, 10), (256, 256, 384, 16, 3), (2304, 256, 1280, 32, 2)],
)
def test_split_tiles_match_whole_tiles(dev, M, K, N, R, k_split, monkeypatch):
    """k_split None: the library's own choice for a shape with few tiles (M = 256, K = N = 3072: 24 tiles,
    4 parts each; M = 512, K = 12288, N = 512: 8 tiles, 8 parts each); 10 parts of K = 640: one k-group each; N = 384 and 1280: a ragged last column block."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import gemm as gemm_mod

    M_out, M_pad = M, (M + 255) // 256 * 256  # operands are padded to 256 rows, the output has M_out rows
    announce(f"split tiles M={M} K={K} N={N} R={R} k_split={k_split}")
    layer = synth.make_layer(N, K, R, seed=K + N)
    m = make_module(layer, dev)
    t = m.native_tensors()
    ins = [_inputs(M_pad, K, R, seed) for seed in (1, 2)]
    dev_ins = [(packing.logical_to_act(c).to(dev), s.to(dev), la.to(dev)) for c, s, la in ins]

    def run(i, split):
        monkeypatch.setattr(gemm_mod, "K_SPLIT", split)
        out = torch.full((M_out, N), float("nan"), dtype=torch.bfloat16, device=dev)
        act, sc, la = dev_ins[i]
        gemm_mod.svdq_gemm_w4a4(act=act, wgt=t["qweight"], out=out, ascales=sc, wscales=t["wscales"], lora_act_in=la,
                                lora_up=t["proj_up"], bias=t["bias"])
        torch.cuda.synchronize()
        return out

    whole = [run(0, 1), run(1, 1)]
    first = {}
    # alternate the inputs: a partial sum left over from the previous launch would belong to the other input
    for i in (0, 1, 0, 0, 1, 1, 0, 1):
        got = run(i, k_split)
        assert not torch.isnan(got.float()).any()
        if i in first:
            assert torch.equal(got, first[i]), "two launches with the same input differ: the sum depends on the order of arrival"
        first[i] = got
        diff = (got.float() - whole[i].float()).abs()
        # a different fp32 summation order may flip the bf16 rounding of an element by one ulp, never more
        big = torch.maximum(torch.maximum(whole[i].float().abs(), got.float().abs()), torch.tensor(2.0**-126, device=dev))
        ulp = big.log2().floor().exp2() * 2.0**-7
        # (results that cancel to almost nothing keep the absolute fp32 rounding noise of their terms)
        tol = torch.maximum(ulp, 1e-5 * whole[i].float().abs().max())
        assert (diff <= tol).all(), f"launch with input {i}: max difference {diff.max().item()} beyond one bf16 ulp"
        assert (diff > 0).float().mean().item() < 2e-2
    # and the oracle, on a row sample
    rows = torch.randperm(M_out, generator=torch.Generator().manual_seed(5))[:64]
    c, s, la = ins[1]
    want = olin.gemm_w4a4(quant.dequant_int4(c[rows], s[:, rows]), quant.dequant_int4(layer.wq, layer.ws), bias=layer.bias,
                          lora_act_in=la[rows], lora_up=layer.proj_up)
    check_output(run(1, k_split)[rows.to(dev)], want)


def test_nvfp4_shared_tiles_match_whole_tiles(dev, monkeypatch):
    """The NVFP4 GEMM keeps its even work split over persistent workgroups: tiles shared by two workgroups
    (more tiles than compute units, not a multiple) against whole-tile mode (k_split = 1)."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import gemm as gemm_mod

    M, K, N, R = 2304, 256, 7680, 32
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    ntiles = (M // 256) * (N // 256)
    assert ntiles > ncu and ntiles % ncu != 0, "the shape must make the even split cut tiles"
    announce(f"nvfp4 shared tiles M={M} K={K} N={N}: {ntiles} tiles on {ncu} compute units")
    layer = synth.make_layer(N, K, R, seed=K + N, fp4=True)
    m = make_module(layer, dev)
    t = m.native_tensors()
    acts = []
    for seed in (1, 2):
        x = synth.make_activations(M, K, seed=seed)
        acts.append(m.quantize(x.to(dev)))

    def run(i, split):
        monkeypatch.setattr(gemm_mod, "K_SPLIT", split)
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        qx, asc, la = acts[i]
        gemm_mod.svdq_gemm_w4a4(act=qx, wgt=t["qweight"], out=out, ascales=asc, wscales=t["wscales"], lora_act_in=la,
                                lora_up=t["proj_up"], bias=t["bias"], fp4=True, alpha=m.alpha, wcscales=t["wcscales"])
        torch.cuda.synchronize()
        return out

    whole = [run(0, 1), run(1, 1)]
    for i in (0, 1, 0, 0, 1, 1, 0, 1):
        got = run(i, None)
        assert not torch.isnan(got.float()).any()
        diff = (got.float() - whole[i].float()).abs()
        big = torch.maximum(torch.maximum(whole[i].float().abs(), got.float().abs()), torch.tensor(2.0**-126, device=dev))
        ulp = big.log2().floor().exp2() * 2.0**-7
        tol = torch.maximum(ulp, 1e-5 * whole[i].float().abs().max())
        assert (diff <= tol).all(), f"launch with input {i}: max difference {diff.max().item()} beyond one bf16 ulp"
        assert (diff > 0).float().mean().item() < 1e-3
