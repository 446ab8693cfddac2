"""fused_qkv_norm_rottary on the GPU (RMS norm per 128-wide head of q and k, then the rotary embedding,
fused into the GEMM epilogue) against the oracle: a small case with ragged tokens and shared tiles,
the NVFP4 variant, the FLUX QKV shape, and properties that hold at any size."""

import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_module, make_oracle
from oracle import layouts as L
from oracle import linear as olin
from oracle import synth

pytestmark = pytest.mark.gpu


class _Norm:
    def __init__(self, weight):
        self.weight = weight


def _rotary(M_pad, seed):
    """A rotary table for M_pad rows: logical fp32 [M_pad, 128] and the reference's packed form [1, M_pad, 128]."""
    g = torch.Generator().manual_seed(seed)
    ang = torch.rand(M_pad, 64, generator=g, dtype=torch.float64) * 6.283
    logical = torch.stack((torch.sin(ang), torch.cos(ang)), dim=-1).reshape(M_pad, 128).float()
    packed = torch.from_numpy(L.pack_rotemb(logical.numpy())).view(1, M_pad, 128)
    return logical, packed


def _run(dev, M, K, N, R, seed, fp4=False):
    from nunchaku_amd.ops import fused_qkv_norm_rottary

    layer = synth.make_layer(N, K, R, seed=seed, fp4=fp4)
    x = synth.make_activations(M, K, seed=seed)
    m = make_module(layer, dev)
    ref = make_oracle(layer)
    if fp4:
        ref.wtscale = float(torch.tensor(layer.wtscale).to(torch.bfloat16))  # the checkpoint stores wtscale as bf16
    M_pad = (M + 255) // 256 * 256
    g = torch.Generator().manual_seed(seed + 100)
    wq = (1.0 + 0.2 * torch.randn(128, generator=g)).bfloat16()
    wk = (1.0 + 0.2 * torch.randn(128, generator=g)).bfloat16()
    logical, packed = _rotary(M_pad, seed + 200)
    y = fused_qkv_norm_rottary(x.to(dev).view(1, M, K), m, _Norm(wq.to(dev)), _Norm(wk.to(dev)), packed.to(dev))
    torch.cuda.synchronize()
    assert y.shape == (1, M, N)
    return y[0], x, ref, wq, wk, logical


def test_repack_rotemb_against_oracle_layout(dev):
    """svdq_repack_rotemb: reference packed order -> the epilogue's order [rows/32][slot 4 nt + q][lane r + 32 h][4]
    = floats 32 nt + 8 q + 4 h + [0, 4) of row 32 b + r."""
    from nunchaku_amd import packing

    rows = 96
    logical = torch.arange(rows * 128, dtype=torch.float32).reshape(rows, 128)
    packed = torch.from_numpy(L.pack_rotemb(logical.numpy()))
    native = packing.repack_rotemb(packed.to(dev)).cpu().reshape(rows // 32, 4, 4, 2, 32, 4)  # b, nt, q, h, r, e
    want = logical.reshape(rows // 32, 32, 4, 4, 2, 4).permute(0, 2, 3, 4, 1, 5)               # b, r, nt, q, h, e -> b, nt, q, h, r, e
    assert torch.equal(native, want)
    with pytest.raises(ValueError):
        packing.repack_rotemb(packed[:48].contiguous().to(dev))


@pytest.mark.parametrize("M,K,N,R,fp4", [(300, 256, 768, 32, False), (256, 384, 1536, 16, False), (200, 256, 768, 32, True)])
def test_small_against_oracle(dev, M, K, N, R, fp4):
    announce(f"qkv norm rope M={M} K={K} N={N} R={R} fp4={fp4}")
    y, x, ref, wq, wk, logical = _run(dev, M, K, N, R, seed=31, fp4=fp4)
    plain = ref.forward(x)
    want = olin.rmsnorm_rope(plain, wq.float(), wk.float(), logical[:M])
    # q and k are normalised to unit mean square per head, v is the plain projection: one tolerance for all
    check_output(y, want)


def test_v_third_equals_plain_layer_and_heads_are_normalised(dev):
    """Properties that need no oracle: the v third is bit-identical to the layer without the epilogue;
    with unit norm weights every q / k head of every row has mean square 1 (a rotation keeps it)."""
    from nunchaku_amd.ops import fused_qkv_norm_rottary

    M, K, N, R = 4608, 3072, 9216, 32  # FLUX.1-dev double-block QKV projection
    announce(f"qkv norm rope properties M={M} K={K} N={N}")
    layer = synth.make_layer(N, K, R, seed=1)
    x = synth.make_activations(M, K, seed=1).to(dev)
    m = make_module(layer, dev)
    ones = torch.ones(128, dtype=torch.bfloat16, device=dev)
    logical, packed = _rotary(M, 7)
    y = fused_qkv_norm_rottary(x.view(1, M, K), m, _Norm(ones), _Norm(ones), packed.to(dev))[0]
    plain = m(x.view(1, M, K))[0]
    torch.cuda.synchronize()
    assert torch.equal(y[:, 2 * N // 3:], plain[:, 2 * N // 3:])
    ms = (y[:, : 2 * N // 3].float().reshape(M, -1, 128) ** 2).mean(-1)
    assert (ms - 1).abs().max().item() < 2e-2, f"head mean squares off by {(ms - 1).abs().max().item()}"
    # a row sample against the oracle
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(3))[:48]
    ref = make_oracle(layer)
    codes, scales, lora = ref.quantize(x.cpu())
    want_plain = ref.forward_quant(codes[rows], scales[:, rows], lora[rows])
    want = olin.rmsnorm_rope(want_plain, torch.ones(128), torch.ones(128), logical[rows])
    check_output(y[rows], want)


def test_rejects_what_is_not_built(dev):
    from nunchaku_amd.ops import fused_qkv_norm_rottary, svdq_gemm_w4a4

    layer = synth.make_layer(768, 256, 32, seed=5)
    m = make_module(layer, dev)
    x = synth.make_activations(256, 256, seed=5).to(dev)
    ones = torch.ones(128, dtype=torch.bfloat16, device=dev)
    _, packed = _rotary(256, 1)
    with pytest.raises(NotImplementedError):
        fused_qkv_norm_rottary(x.view(1, 256, 256), m, _Norm(ones), _Norm(ones), packed.to(dev), output=(None, None, None))
    qx, asc, la = m.quantize(x)
    t = m.native_tensors()
    out = torch.empty(256, 768, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):  # norm weights without a table
        svdq_gemm_w4a4(act=qx, wgt=t["qweight"], out=out, ascales=asc, wscales=t["wscales"], norm_q=ones, norm_k=ones)
    layer2 = synth.make_layer(512, 256, 32, seed=6)  # N not three parts of whole heads
    m2 = make_module(layer2, dev)
    t2 = m2.native_tensors()
    out2 = torch.empty(256, 512, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        svdq_gemm_w4a4(act=qx, wgt=t2["qweight"], out=out2, ascales=asc, wscales=t2["wscales"], norm_q=ones, norm_k=ones, rotary_emb=packed.to(dev))
