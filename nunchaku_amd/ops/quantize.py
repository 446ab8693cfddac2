"""``svdq_quantize_w4a4_act_fuse_lora``: same signature, defaults and return value as
nunchaku/ops/quantize.py:11-54; the work is done by ``svdq_quantize_w4a4_act_fuse_lora`` of the C ABI.
"""

from __future__ import annotations

import ctypes

import torch

from .. import _native as nv
from .. import packing
from ..utils import ceil_divide


def svdq_quantize_w4a4_act_fuse_lora(
    input: torch.Tensor,
    output: torch.Tensor | None = None,
    oscales: torch.Tensor | None = None,
    lora_down: torch.Tensor | None = None,
    lora_act_out: torch.Tensor | None = None,
    smooth: torch.Tensor | None = None,
    fuse_glu: bool = False,
    fp4: bool = False,
    pad_size: int = 256,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Smooth, quantize to 4 bits and project onto the low-rank basis in one pass over ``input``.

    input  bf16 [M, K] (``fuse_glu``: [M, 2K] pairs (value, gate), the K columns value * silu(gate) are what
    is quantized and projected);  lora_down  proj_down [K, R];  smooth  smooth_factor [K] (both either in the
    reference checkpoint layout, repacked once and cached, or already native, see ``packing``).
    Returns ``(output u8 [M_pad, 3K/4], oscales [K/G, M_pad], lora_act_out fp32 [M_pad, R])`` where
    M_pad rounds M up to ``pad_size`` (256).  ``output`` is private to this operator and the GEMM: INT4
    codes travel as 6-bit E2M3 patterns, the matrix-core operand format (the reference's tensor is
    [M_pad, K/2], also in a private order); NVFP4 keeps [M_pad, K/2].  ``packing.act_to_logical`` gives
    one code per element.
    """
    if input.dim() != 2:
        raise ValueError("input must be [M, K]")
    nv.require_gpu(input, "input")
    if input.dtype != torch.bfloat16:
        raise NotImplementedError("only bf16 activations are supported")
    if pad_size % 256 != 0:
        raise ValueError("pad_size must be a multiple of 256")
    if lora_down is None:
        raise ValueError("lora_down is required")  # the reference reads lora_down.shape[1] unconditionally
    batch_size, channels = input.shape
    if fuse_glu:
        # the row holds (value, gate) pairs: half as many columns are quantized (the reference sizes its
        # checks the same way, gemm_w4a4_launch_impl.cuh:466-480, and leaves the allocation to the caller)
        if channels % 2:
            raise ValueError("fuse_glu needs an even number of input columns")
        channels //= 2
    rank = lora_down.shape[1]
    batch_size_pad = ceil_divide(batch_size, pad_size) * pad_size
    dev = input.device
    if output is None:
        output = torch.empty(batch_size_pad, packing.act_nbytes_per_row(channels, fp4), dtype=torch.uint8, device=dev)
    if oscales is None:
        if fp4:
            assert channels % 16 == 0
            oscales = torch.empty(channels // 16, batch_size_pad, dtype=torch.float8_e4m3fn, device=dev)
        else:
            assert channels % 64 == 0
            oscales = torch.empty(channels // 64, batch_size_pad, dtype=input.dtype, device=dev)
    if lora_act_out is None:
        lora_act_out = torch.empty(batch_size_pad, rank, dtype=torch.float32, device=dev)
    for name, t in (("output", output), ("oscales", oscales), ("lora_act_out", lora_act_out)):
        nv.require_gpu(t, name)
    if tuple(output.shape) != (batch_size_pad, packing.act_nbytes_per_row(channels, fp4)) or output.dtype != torch.uint8:
        raise ValueError(
            f"output must be uint8 [{batch_size_pad}, {packing.act_nbytes_per_row(channels, fp4)}] (6 bits per INT4 element: the "
            "activation layout is private to the two operators), got " + str(tuple(output.shape)))
    if tuple(lora_act_out.shape) != (batch_size_pad, rank) or lora_act_out.dtype != torch.float32:
        raise ValueError(f"lora_act_out must be float32 [{batch_size_pad}, {rank}]")
    G = 16 if fp4 else 64
    if tuple(oscales.shape) != (channels // G, batch_size_pad) or oscales.dtype != (torch.float8_e4m3fn if fp4 else torch.bfloat16):
        raise ValueError(f"oscales must be [{channels // G}, {batch_size_pad}] of {'float8_e4m3fn' if fp4 else 'bfloat16'}")
    if tuple(lora_down.shape) != (channels, rank):
        raise ValueError(f"lora_down must be [{channels}, R], got {tuple(lora_down.shape)}")
    if smooth is not None and smooth.numel() != channels:
        raise ValueError(f"smooth must have {channels} elements")

    down = packing.native(lora_down, "lora_down")
    rcp = packing.native(smooth, "smooth_rcp")
    args = nv.QuantizeArgs(
        input=input.data_ptr(), output=output.data_ptr(), oscales=oscales.data_ptr(),
        lora_down=nv.ptr(down) if rank else None, lora_act_out=lora_act_out.data_ptr() if rank else None, smooth_rcp=nv.ptr(rcp),
        M=batch_size, M_pad=batch_size_pad, K=channels, R=rank, fp4=int(fp4), fuse_glu=int(fuse_glu),
    )
    nv.launch(nv.lib().svdq_quantize_w4a4_act_fuse_lora, ctypes.byref(args), dev)
    return output, oscales, lora_act_out


# the reference spells the function with a ``_cuda`` suffix (nunchaku/ops/quantize.py:11)
svdq_quantize_w4a4_act_fuse_lora_cuda = svdq_quantize_w4a4_act_fuse_lora
