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


def test_rejects_inconsistent_arguments(dev):
    from nunchaku_amd.ops import fused_qkv_norm_rottary, svdq_gemm_w4a4

    layer = synth.make_layer(768, 256, 32, seed=5)
    m = make_module(layer, dev)
    x = synth.make_activations(256, 256, seed=5).to(dev)
    ones = torch.ones(128, dtype=torch.bfloat16, device=dev)
    _, packed = _rotary(256, 1)
    with pytest.raises(ValueError):  # a tuple without tensors
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


@pytest.mark.parametrize("M,K,N,R,fp4", [(300, 256, 768, 32, False), (512, 384, 1536, 16, False), (200, 256, 768, 32, True)])
def test_separate_q_k_v_outputs(dev, M, K, N, R, fp4):
    """The (q, k, v) form (EpiloguePackQKV): each tensor equals its third of the single-output form, head by
    head, converted bf16 -> fp16 (bit for bit: both forms round the same fp32 values to bf16 first); rows from
    attn_tokens on hold the mask values; the tensors are row ranges of larger ones, as the joint attention block
    passes them, and nothing outside the ranges is written.  Then the oracle's restatement on the whole."""
    from nunchaku_amd.ops import fused_qkv_norm_rottary

    announce(f"qkv separate outputs M={M} K={K} N={N} R={R} fp4={fp4}")
    layer = synth.make_layer(N, K, R, seed=41, fp4=fp4)
    x = synth.make_activations(M, K, seed=41)
    m = make_module(layer, dev)
    ref = make_oracle(layer)
    if fp4:
        ref.wtscale = float(torch.tensor(layer.wtscale).to(torch.bfloat16))
    M_pad = (M + 255) // 256 * 256
    heads = N // 384
    g = torch.Generator().manual_seed(141)
    wq = (1.0 + 0.2 * torch.randn(128, generator=g)).bfloat16()
    wk = (1.0 + 0.2 * torch.randn(128, generator=g)).bfloat16()
    logical, packed = _rotary(M_pad, 241)
    nq, nk = _Norm(wq.to(dev)), _Norm(wk.to(dev))
    single = fused_qkv_norm_rottary(x.to(dev).view(1, M, K), m, nq, nk, packed.to(dev))[0]  # [M, N] bf16

    before = 256  # rows of another stream in front, as in the joint block (flux.py:139-160)
    big = [torch.full((1, heads, before + M_pad + 32, 128), 777.0, dtype=torch.float16, device=dev) for _ in range(3)]
    views = tuple(t[:, :, before:before + M_pad] for t in big)
    got = fused_qkv_norm_rottary(x.to(dev).view(1, M, K), m, nq, nk, packed.to(dev), output=views, attn_tokens=M)
    torch.cuda.synchronize()
    assert got[0].data_ptr() == views[0].data_ptr()
    for i, t in enumerate(big):
        assert (t[:, :, :before] == 777.0).all() and (t[:, :, before + M_pad:] == 777.0).all(), "rows outside the range were written"
        part = single[:, i * heads * 128:(i + 1) * heads * 128].reshape(M, heads, 128).permute(1, 0, 2)
        assert torch.equal(views[i][0, :, :M], part.float().to(torch.float16)), f"tensor {i} differs from its third of the single output"
        pad = views[i][0, :, M:]
        if pad.numel():
            assert torch.isnan(pad).all() if i == 1 else (pad == 0).all(), f"mask rows of tensor {i}"
    # the oracle on everything (its NaN rows compared as such)
    plain = ref.forward(x)
    full = torch.zeros(M_pad, N)
    full[:M] = olin.rmsnorm_rope(plain, wq.float(), wk.float(), logical[:M])
    want = olin.pack_qkv(full, attn_tokens=M)
    for i in range(3):
        check_output(views[i][0, :, :M].reshape(-1, 128), want[i][0, :, :M].reshape(-1, 128).float())

    # fewer tokens than rows given: the mask moves, the rows before it do not change
    fewer = tuple(torch.empty(1, heads, M_pad, 128, dtype=torch.float16, device=dev) for _ in range(3))
    fused_qkv_norm_rottary(x.to(dev).view(1, M, K), m, nq, nk, packed.to(dev), output=fewer, attn_tokens=M - 37)
    for i in range(3):
        assert torch.equal(fewer[i][0, :, :M - 37], views[i][0, :, :M - 37])
        pad = fewer[i][0, :, M - 37:]
        assert torch.isnan(pad).all() if i == 1 else (pad == 0).all()


def test_separate_outputs_reject_bad_arguments(dev):
    from nunchaku_amd.ops import fused_qkv_norm_rottary

    layer = synth.make_layer(768, 256, 16, seed=43)
    m = make_module(layer, dev)
    x = synth.make_activations(256, 256, seed=43).to(dev).view(1, 256, 256)
    _, packed = _rotary(256, 243)
    n = _Norm(torch.ones(128, dtype=torch.bfloat16, device=dev))
    ok = lambda: torch.empty(1, 2, 256, 128, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        fused_qkv_norm_rottary(x, m, n, n, packed.to(dev), output=(ok(), ok(), torch.empty(1, 2, 128, 128, dtype=torch.float16, device=dev)))
    with pytest.raises(ValueError):
        fused_qkv_norm_rottary(x, m, n, n, packed.to(dev), output=(ok(), ok(), ok().bfloat16()))
    with pytest.raises(ValueError):
        fused_qkv_norm_rottary(x, m, n, n, packed.to(dev), output=(ok(), ok(), ok()), attn_tokens=257)
    with pytest.raises(ValueError):
        fused_qkv_norm_rottary(x, m, n, n, packed.to(dev), output=(ok(), ok()))
