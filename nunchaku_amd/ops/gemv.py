"""``awq_gemv_w4a16_cuda`` with the signature of nunchaku/ops/gemv.py:10-20."""

from __future__ import annotations

import ctypes

import torch

from .. import _native as nv


def awq_gemv_w4a16(
    in_feats: torch.Tensor,
    kernel: torch.Tensor,
    scaling_factors: torch.Tensor,
    zeros: torch.Tensor,
    m: int,
    n: int,
    k: int,
    group_size: int = 64,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """AWQ W4A16 GEMV for up to 8 rows.

    in_feats bf16 [..., k] with ``m`` rows in total; kernel int32 [n/4, k/2] and scaling_factors / zeros
    bf16 [k/64, n] exactly as the reference checkpoint stores them.  Returns bf16 [..., n].  ``bias``
    (not in the reference signature: AWQW4A16Linear adds it afterwards, linear.py:183-185) is added to the
    rounded result inside the kernel when given.
    """
    for name, t in (("in_feats", in_feats), ("kernel", kernel), ("scaling_factors", scaling_factors), ("zeros", zeros)):
        nv.require_gpu(t, name)
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    if in_feats.dtype != torch.bfloat16 or scaling_factors.dtype != torch.bfloat16 or zeros.dtype != torch.bfloat16:
        raise NotImplementedError("only bf16 activations / scales / zeros are supported")
    if in_feats.shape[-1] != k or in_feats.numel() != m * k:
        raise ValueError(f"in_feats {tuple(in_feats.shape)} does not hold m={m} rows of k={k}")
    if kernel.numel() * kernel.element_size() != n * k // 2:
        raise ValueError(f"kernel {tuple(kernel.shape)} ({kernel.dtype}) does not hold n={n} x k={k} 4-bit codes")
    if scaling_factors.shape != (k // 64, n) or zeros.shape != (k // 64, n):
        raise ValueError("scaling_factors and zeros must be [k/64, n]")
    if bias is not None:
        nv.require_gpu(bias, "bias")
        if bias.dtype != torch.bfloat16 or bias.numel() != n or not bias.is_contiguous():
            raise ValueError("bias must be a contiguous bf16 vector of n elements")
    out = torch.empty(*in_feats.shape[:-1], n, dtype=torch.bfloat16, device=in_feats.device)
    args = nv.AwqGemvArgs(
        x=in_feats.data_ptr(), qweight=kernel.data_ptr(), scales=scaling_factors.data_ptr(), zeros=zeros.data_ptr(),
        bias=nv.ptr(bias), out=out.data_ptr(), M=m, N=n, K=k, group_size=group_size,
    )
    nv.launch(nv.lib().svdq_awq_gemv_w4a16, ctypes.byref(args), in_feats.device)
    return out


awq_gemv_w4a16_cuda = awq_gemv_w4a16
