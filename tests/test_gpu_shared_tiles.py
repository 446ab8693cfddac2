"""The even work split of the GEMM: output tiles shared by two workgroups, or by many when there are
fewer tiles than compute units (fp32 partial sums parked in a workspace), against the same launches in
whole-tile mode, and against the oracle.

What could go wrong and what catches it: a partial sum read before it is complete or from a stale cache
line (alternating inputs between launches: a stale read would return the other input's sums), a k-range
counted twice or not at all (whole-tile mode computes every tile in one piece), very short shares
(K = 256: shares of two k-groups)."""

import os

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


@pytest.mark.parametrize("M,K,N,R", [(2304, 256, 7680, 32), (4608, 3072, 12288, 32), (2816, 512, 6400, 16), (4500, 384, 3840, 32)])
def test_shared_tiles_match_whole_tiles(dev, M, K, N, R):
    M_pad = (M + 255) // 256 * 256
    ntiles = (M_pad // 256) * ((N + 255) // 256)
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    assert ntiles > ncu and ntiles % ncu != 0, "the shape must make the even split cut tiles"
    _compare_with_whole_tiles(dev, M, K, N, R, max_fraction_different=1e-3)


@pytest.mark.parametrize("M,K,N,R", [(256, 3072, 3072, 32), (256, 1024, 512, 16), (512, 12288, 256, 32), (300, 640, 768, 32)])
def test_few_tiles_split_among_many_workgroups(dev, M, K, N, R, monkeypatch):
    """Fewer tiles than compute units: every tile is split along K among several workgroups (6, 2, 24
    parties; K = 640 gives shares that straddle tile boundaries), the last to arrive adds up the rest."""
    M_pad = (M + 255) // 256 * 256
    ntiles = (M_pad // 256) * ((N + 255) // 256)
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    monkeypatch.setenv("SVDQ_GEMM_MIN_UNITS", "4")  # (the default of 12 units per workgroup would split only the third shape)
    assert ntiles < ncu and ntiles * (K // 128) // 4 > ntiles, "the shape must give several workgroups per tile"
    # (more parties, more fp32 additions in another order: more elements whose bf16 rounding flips)
    _compare_with_whole_tiles(dev, M, K, N, R, max_fraction_different=2e-2)


def _compare_with_whole_tiles(dev, M, K, N, R, max_fraction_different):
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    M_out, M = M, (M + 255) // 256 * 256  # operands are padded to 256 rows, the output has M_out rows
    ntiles = (M // 256) * ((N + 255) // 256)
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    announce(f"shared tiles M={M} K={K} N={N} R={R}: {ntiles} tiles on {ncu} compute units")
    layer = synth.make_layer(N, K, R, seed=K + N)
    m = make_module(layer, dev)
    t = m.native_tensors()
    ins = [_inputs(M, K, R, seed) for seed in (1, 2)]
    dev_ins = [(packing.logical_to_act(c).to(dev), s.to(dev), la.to(dev)) for c, s, la in ins]

    def run(i):
        out = torch.full((M_out, N), float("nan"), dtype=torch.bfloat16, device=dev)
        act, sc, la = dev_ins[i]
        svdq_gemm_w4a4(act=act, wgt=t["qweight"], out=out, ascales=sc, wscales=t["wscales"], lora_act_in=la,
                       lora_up=t["proj_up"], bias=t["bias"])
        torch.cuda.synchronize()
        return out

    os.environ["SVDQ_GEMM_NO_SHARED_TILES"] = "1"
    try:
        whole = [run(0), run(1)]
    finally:
        del os.environ["SVDQ_GEMM_NO_SHARED_TILES"]
    # alternate the inputs: a partial sum left over from the previous launch would belong to the other input
    for i in (0, 1, 0, 0, 1, 1, 0, 1):
        got = run(i)
        assert not torch.isnan(got.float()).any()
        diff = (got.float() - whole[i].float()).abs()
        # a different fp32 summation order may flip the bf16 rounding of an element by one ulp, never more
        big = torch.maximum(torch.maximum(whole[i].float().abs(), got.float().abs()), torch.tensor(2.0**-126, device=dev))
        ulp = big.log2().floor().exp2() * 2.0**-7
        # (results that cancel to almost nothing keep the absolute fp32 rounding noise of their terms)
        tol = torch.maximum(ulp, 1e-5 * whole[i].float().abs().max())
        assert (diff <= tol).all(), f"launch with input {i}: max difference {diff.max().item()} beyond one bf16 ulp"
        assert (diff > 0).float().mean().item() < max_fraction_different
    # and the oracle, on a row sample
    rows = torch.randperm(M_out, generator=torch.Generator().manual_seed(5))[:64]
    c, s, la = ins[1]
    want = olin.gemm_w4a4(quant.dequant_int4(c[rows], s[:, rows]), quant.dequant_int4(layer.wq, layer.ws), bias=layer.bias,
                          lora_act_in=la[rows], lora_up=layer.proj_up)
    check_output(run(1)[rows.to(dev)], want)
