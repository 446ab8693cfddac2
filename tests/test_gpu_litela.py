"""Linear attention on the GPU: the GEMM's q / vk epilogue (EpilogueLiteLA) and the kernel that applies the sums
to q, against the oracle."""

import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_module, make_oracle
from oracle import linear as olin
from oracle import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,T,K,heads,R,fp4", [(1, 256, 256, 4, 16, False), (2, 256, 384, 8, 32, False), (1, 1024, 256, 12, 32, False),
                                               (3, 512, 128, 20, 0, False), (2, 512, 256, 12, 32, True), (1, 2304, 128, 80, 16, True)])
def test_litela_epilogue(dev, B, T, K, heads, R, fp4):
    """heads = 4: N = 384, one 256-column block of q + k/v and a ragged half block; 12 and 20 heads: the q third ends
    inside a 256-column block, so one workgroup holds a q half and a k/v half.  Several row blocks per batch entry add
    up in a fixed order; several batch entries must not mix.  NVFP4: the other GEMM kernel (256 x 256 tiles; 2304 rows x
    7680 columns are 270 tiles, which its workgroups share).  heads = 80: the q third ends inside a tile."""
    from nunchaku_amd.ops import svdq_gemm_w4a4

    N = heads * 96
    announce(f"litela B={B} T={T} K={K} heads={heads} R={R} fp4={fp4}")
    layer = synth.make_layer(N, K, R, seed=heads + K, fp4=fp4)
    m = make_module(layer, dev)
    ref = make_oracle(layer)
    if fp4:
        ref.wtscale = float(torch.tensor(layer.wtscale).to(torch.bfloat16))  # the checkpoint stores wtscale as bf16
    x = synth.make_activations(B * T, K, seed=heads)
    qx, asc, la = m.quantize(x.to(dev))
    t = m.native_tensors()
    q = torch.full((B, T, N // 3), float("nan"), dtype=torch.bfloat16, device=dev)
    vk = torch.full((B, heads, 33, 32), float("nan"), dtype=torch.float32, device=dev)  # the operator clears it
    kw = dict(act=qx, wgt=t["qweight"], ascales=asc, wscales=t["wscales"], bias=t["bias"])
    if fp4:
        kw.update(fp4=True, alpha=m.alpha, wcscales=t["wcscales"])
    if R:
        kw.update(lora_act_in=la, lora_up=t["proj_up"])
    svdq_gemm_w4a4(**kw, out_vk=vk, out_linearattn=q)
    torch.cuda.synchronize()
    # what the plain layer gives, on the GPU: q must be its ReLU bit for bit, and vk follows from its bf16 values exactly
    plain = torch.empty(B * T, N, dtype=torch.bfloat16, device=dev)
    svdq_gemm_w4a4(**kw, out=plain)
    torch.cuda.synchronize()
    assert torch.equal(q.reshape(B * T, -1), torch.relu(plain[:, : N // 3]))
    _, vk_from_plain = olin.litela(plain.float().cpu(), batch=B)
    scale = vk_from_plain.abs().amax(dim=(2, 3), keepdim=True)
    assert ((vk.cpu().double() - vk_from_plain).abs() <= 1e-5 * scale + 1e-6).all(), "vk differs from the sums over the plain layer's own output"
    # and the oracle end to end
    want_q, want_vk = olin.litela(ref.forward(x), batch=B)
    check_output(q.reshape(B * T, -1), want_q.reshape(B * T, -1))
    err = (vk.cpu().double() - want_vk).abs()
    assert (err <= 2e-2 * want_vk.abs().amax(dim=(2, 3), keepdim=True)).all(), f"vk off by {err.max().item()}"
    # a second launch on the same buffers gives the same sums again, bit for bit: they are written, not accumulated, and
    # the slabs are added in a fixed order
    first = vk.clone()
    for _ in range(3):
        vk.fill_(float("nan"))
        svdq_gemm_w4a4(**kw, out_vk=vk, out_linearattn=q)
        torch.cuda.synchronize()
        assert torch.equal(vk, first)


def test_vk_mul_q(dev):
    from nunchaku_amd.ops import linearattn_vk_mul_q

    B, T, heads, tokens = 2, 512, 6, 300
    announce(f"vk_mul_q B={B} T={T} heads={heads} tokens={tokens}")
    g = torch.Generator().manual_seed(3)
    q = torch.relu(torch.randn(B, T, heads * 32, generator=g)).to(torch.bfloat16)
    vk = torch.randn(B, heads, 33, 32, generator=g)
    vk[:, :, 32] = vk[:, :, 32].abs() + 0.5  # sums of relu(k) are positive
    want = olin.linearattn_vk_mul_q(q.float(), vk, num_tokens=tokens)
    got = linearattn_vk_mul_q(q.to(dev), vk.to(dev), num_tokens=tokens)
    torch.cuda.synchronize()
    assert torch.equal(got[:, tokens:].cpu(), q[:, tokens:]), "rows beyond num_tokens must stay as they were"
    # one bf16 rounding of the result, fp32 sums of 32 terms
    err = (got[:, :tokens].cpu().double() - want[:, :tokens]).abs()
    assert (err <= 2.0**-8 * want[:, :tokens].abs() + 1e-5 * want[:, :tokens].abs().max()).all(), err.max().item()
    with pytest.raises(ValueError):
        linearattn_vk_mul_q(q.to(dev), vk[:, :5].contiguous().to(dev))


def test_litela_rejects_bad_arguments(dev):
    from nunchaku_amd.ops import svdq_gemm_w4a4

    layer = synth.make_layer(384, 128, 16, seed=9)
    m = make_module(layer, dev)
    qx, asc, la = m.quantize(synth.make_activations(256, 128, seed=9).to(dev))
    t = m.native_tensors()
    q = torch.empty(1, 256, 128, dtype=torch.bfloat16, device=dev)
    vk = torch.empty(1, 4, 33, 32, dtype=torch.float32, device=dev)
    kw = dict(act=qx, wgt=t["qweight"], ascales=asc, wscales=t["wscales"])
    with pytest.raises(ValueError):
        svdq_gemm_w4a4(**kw, out_vk=vk)
    with pytest.raises(ValueError):
        svdq_gemm_w4a4(**kw, out_vk=vk[:, :3].contiguous(), out_linearattn=q)
    with pytest.raises(ValueError):
        svdq_gemm_w4a4(**kw, out_vk=vk, out_linearattn=q[:, :128].contiguous())
    with pytest.raises(ValueError):
        svdq_gemm_w4a4(**kw, out_vk=vk, out_linearattn=q, out=torch.empty(256, 384, dtype=torch.bfloat16, device=dev))
