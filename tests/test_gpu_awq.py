"""AWQ W4A16 GEMV on the GPU against the oracle: the module with the reference's parameter layout, every
row count 1..8, ragged K (not a multiple of 512), the Qwen-Image modulation shape, and linearity."""

import numpy as np
import pytest
import torch

from conftest import announce
from oracle import awq

pytestmark = pytest.mark.gpu


def _module(dev, oc, ic, seed, bias=True):
    from nunchaku_amd.models import AWQW4A16Linear

    codes, scales, zeros, b = awq.make_layer(oc, ic, seed)
    m = AWQW4A16Linear(ic, oc, bias=bias, device=dev)
    sd = {"qweight": torch.from_numpy(awq.pack_w4(codes.numpy()).view(np.int32).copy()), "wscales": scales, "wzeros": zeros}
    if bias:
        sd["bias"] = b
    m.load_state_dict(sd, strict=True)
    return m, (codes, scales, zeros, b if bias else None)


def _check(y, want, bias):
    """fp32 accumulation in another order, then the bf16 rounding(s) of the reference: within one bf16 ulp of
    the oracle rounded the same way, and rel-L2 1e-3."""
    want_bf = want.to(torch.bfloat16).float()
    if bias is not None:
        want_bf = (want_bf + bias.float()).to(torch.bfloat16).float()
    got = y.float().cpu()
    rel = ((got - want_bf).norm() / want_bf.norm()).item()
    assert rel <= 1e-3, f"rel-L2 {rel:.3e}"
    ulp = torch.pow(2.0, torch.floor(torch.log2(want_bf.abs().clamp_min(2.0**-126))) - 7)
    assert ((got - want_bf).abs() <= 2 * ulp + 1e-6).all()


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("oc,ic", [(256, 512), (64, 192), (520, 1088)])
def test_against_oracle(dev, rows, oc, ic):
    announce(f"awq gemv rows={rows} oc={oc} ic={ic}")
    m, (codes, scales, zeros, bias) = _module(dev, oc, ic, seed=oc + ic)
    x = torch.randn(rows, ic, generator=torch.Generator().manual_seed(rows)).to(torch.bfloat16)
    y = m(x.to(dev))
    torch.cuda.synchronize()
    assert y.shape == (rows, oc) and y.dtype == torch.bfloat16
    _check(y, awq.gemv(x, codes, scales, zeros), bias)


def test_long_k_takes_the_path_without_lds_staging(dev):
    """8 rows of K=4160 do not fit the 64 KB the kernel stages x in: the activations then come from global memory."""
    oc, ic, rows = 64, 4160, 8
    announce(f"awq gemv rows={rows} oc={oc} ic={ic} (x not staged)")
    m, (codes, scales, zeros, bias) = _module(dev, oc, ic, seed=77)
    x = torch.randn(rows, ic, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    y = m(x.to(dev))
    torch.cuda.synchronize()
    _check(y, awq.gemv(x, codes, scales, zeros), bias)
    _check(m(x[:1].to(dev)), awq.gemv(x[:1], codes, scales, zeros), bias)  # one row of the same layer: staged


def test_modulation_shape_and_linearity(dev):
    """K=3072, N=18432 (six modulation vectors of a 3072-wide block), one row; without bias the result is
    linear in x up to the bf16 rounding of the output."""
    oc, ic = 18432, 3072
    announce(f"awq gemv modulation shape oc={oc} ic={ic}")
    m, (codes, scales, zeros, _) = _module(dev, oc, ic, seed=9, bias=False)
    x = torch.randn(1, 1, ic, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    y = m(x.to(dev))
    torch.cuda.synchronize()
    assert y.shape == (1, 1, oc)
    _check(y[0], awq.gemv(x[0], codes, scales, zeros), None)
    y2 = m((x * 2).to(dev))  # doubling is exact in bf16
    assert torch.equal(y2.float(), y.float() * 2)


def test_rejects_bad_arguments(dev):
    from nunchaku_amd.ops import awq_gemv_w4a16_cuda

    m, _ = _module(dev, 64, 128, seed=1)
    x = torch.zeros(9, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):  # more than 8 rows
        m(x)
    with pytest.raises(NotImplementedError):
        awq_gemv_w4a16_cuda(x[:1], m.qweight, m.wscales, m.wzeros, 1, 64, 128, group_size=128)
    with pytest.raises(RuntimeError, match="GPU"):
        awq_gemv_w4a16_cuda(x[:1].cpu(), m.qweight, m.wscales, m.wzeros, 1, 64, 128)
