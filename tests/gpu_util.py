"""Helpers shared by the GPU parity tests."""

import torch

from oracle import linear as olin
from oracle import synth


def bf16_ulp(x: torch.Tensor) -> torch.Tensor:
    """Spacing of bf16 numbers at the magnitude of x (fp32 tensor)."""
    e = torch.floor(torch.log2(x.abs().clamp_min(2.0**-126)))
    return torch.pow(2.0, e - 7)


def check_output(got_bf16: torch.Tensor, want_f32: torch.Tensor, rel_tol: float = 1e-3):
    """The GEMM tolerance: rel-L2 <= 1e-3 against the oracle rounded to bf16, and no element further
    than max(2e-2, one bf16 ulp at its magnitude) from the oracle's fp32 value (a different fp32
    summation order may flip the final bf16 rounding of an element by one ulp, never more)."""
    got = got_bf16.float().cpu()
    want_bf = want_f32.to(torch.bfloat16).float()
    rel = ((got - want_bf).norm() / want_bf.norm().clamp_min(1e-30)).item()
    assert rel <= rel_tol, f"rel-L2 {rel:.3e} > {rel_tol}"
    err = (got - want_f32).abs()
    bound = torch.maximum(torch.full_like(err, 2e-2), bf16_ulp(want_f32))
    worst = (err - bound).max().item()
    assert worst <= 0, f"max-abs violation by {worst:.3e}"
    return rel


def make_module(layer: synth.LogicalLayer, dev, act_unsigned=False):
    from nunchaku_amd.models.linear import SVDQW4A4Linear

    m = SVDQW4A4Linear(
        layer.K, layer.N, rank=layer.R, bias=layer.bias is not None,
        precision="nvfp4" if layer.fp4 else "int4", act_unsigned=act_unsigned, device=dev,
    )
    missing = m.load_state_dict(synth.to_reference_checkpoint(layer), strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys
    return m


def make_oracle(layer: synth.LogicalLayer, act_unsigned=False):
    return olin.FakeQuantLinear(
        layer.wq, layer.ws, layer.smooth, layer.proj_down, layer.proj_up, layer.bias,
        fp4=layer.fp4, wtscale=layer.wtscale, wcscales=layer.wcscales, act_unsigned=act_unsigned,
    )


class Guarded:
    """A tensor placed inside a larger buffer filled with a byte pattern: ``check()`` asserts that the bands before and
    behind it still hold the pattern, i.e. that no kernel wrote outside the tensor."""

    PATTERN = 0xA5

    def __init__(self, shape, dtype, dev, band: int = 1 << 16):
        n = 1
        for d in shape:
            n *= d
        self.nbytes = n * torch.empty((), dtype=dtype).element_size()
        self.band = band
        padded = (self.nbytes + 255) // 256 * 256
        self.raw = torch.full((band + padded + band,), self.PATTERN, dtype=torch.uint8, device=dev)
        self.t = self.raw[band:band + self.nbytes].view(dtype).view(*shape)

    def check(self, name: str) -> None:
        before = self.raw[:self.band]
        behind = self.raw[self.band + self.nbytes:]
        assert bool((before == self.PATTERN).all()), f"{name}: bytes in front of the tensor were overwritten"
        assert bool((behind == self.PATTERN).all()), f"{name}: bytes behind the tensor were overwritten"
