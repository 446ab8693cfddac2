"""``fused_gelu_mlp`` and ``fused_qkv_norm_rottary`` with the signatures of nunchaku/ops/fused.py:10-110."""

from __future__ import annotations

import torch

from ..packing import act_nbytes_per_row
from ..utils import ceil_divide
from .gemm import svdq_gemm_w4a4


def fused_gelu_mlp(x: torch.Tensor, fc1, fc2, pad_size: int = 256) -> torch.Tensor:
    """fc1 -> GELU -> fc2 with the GELU, fc2's activation quantization (unsigned INT4 after a
    +0.171875 shift) and fc2's low-rank down projection fused into fc1's GEMM epilogue."""
    batch_size, seq_len, channels = x.shape
    x = x.view(batch_size * seq_len, channels)
    quantized_x, ascales, lora_act = fc1.quantize(x)

    batch_size_pad = ceil_divide(batch_size * seq_len, pad_size) * pad_size
    qout_act = torch.empty(batch_size_pad, act_nbytes_per_row(fc1.out_features, fc2.precision == "nvfp4"), dtype=torch.uint8, device=x.device)
    if fc2.precision == "nvfp4":
        qout_ascales = torch.empty(fc1.out_features // 16, batch_size_pad, dtype=torch.float8_e4m3fn, device=x.device)
    else:
        qout_ascales = torch.empty(fc1.out_features // 64, batch_size_pad, dtype=x.dtype, device=x.device)
    qout_lora_act = torch.empty(batch_size_pad, fc2.proj_down.shape[1], dtype=torch.float32, device=x.device)

    t1, t2 = fc1.native_tensors(), fc2.native_tensors()
    svdq_gemm_w4a4(
        act=quantized_x, wgt=t1["qweight"], qout=qout_act, ascales=ascales, wscales=t1["wscales"],
        oscales=qout_ascales, lora_act_in=lora_act, lora_up=t1["proj_up"], lora_down=t2["proj_down"],
        lora_act_out=qout_lora_act, bias=t1["bias"], smooth_factor=t2["smooth_factor"],
        fp4=fc1.precision == "nvfp4", alpha=fc1.alpha, wcscales=t1["wcscales"], lora_scales=fc1.lora_scales,
    )
    output = torch.empty(batch_size * seq_len, fc2.out_features, dtype=x.dtype, device=x.device)
    output = fc2.forward_quant(qout_act, qout_ascales, qout_lora_act, output=output)
    return output.view(batch_size, seq_len, -1)


def fused_qkv_norm_rottary(x: torch.Tensor, proj, norm_q, norm_k, rotary_emb: torch.Tensor, output=None, attn_tokens: int = 0):
    """QKV projection with the RMS norm of q and k (per 128-wide head) and the rotary embedding fused
    into the GEMM epilogue (nunchaku/ops/fused.py:50-110).  ``norm_q`` / ``norm_k`` are modules with a
    bf16 ``weight`` of 128 elements, ``rotary_emb`` is the table packed by ``pack_rotemb``.

    ``output``: None or a bf16 tensor: q | k | v side by side, one row per token.  A tuple (q, k, v) of
    fp16 [1, heads, tokens_pad, 128] tensors: the three apart, per head, rows from ``attn_tokens`` on
    masked (see ``svdq_gemm_w4a4``)."""
    batch_size, seq_len, channels = x.shape
    x = x.view(batch_size * seq_len, channels)
    quantized_x, ascales, lora_act = proj.quantize(x)
    t = proj.native_tensors()
    common = dict(
        act=quantized_x, wgt=t["qweight"], ascales=ascales, wscales=t["wscales"], lora_act_in=lora_act, lora_up=t["proj_up"],
        bias=t["bias"], fp4=proj.precision == "nvfp4", alpha=proj.alpha, wcscales=t["wcscales"], norm_q=norm_q.weight,
        norm_k=norm_k.weight, rotary_emb=rotary_emb, lora_scales=proj.lora_scales,
    )
    if isinstance(output, tuple):
        if len(output) != 3:
            raise ValueError("a tuple `output` is (q, k, v)")
        svdq_gemm_w4a4(**common, out_q=output[0], out_k=output[1], out_v=output[2], attn_tokens=attn_tokens)
        return output
    if output is None:
        output = torch.empty(quantized_x.shape[0], proj.out_features, dtype=x.dtype, device=x.device)
    svdq_gemm_w4a4(**common, out=output)
    # (the reference views the padded buffer directly, which only works for token counts that need no padding)
    return output[: batch_size * seq_len].view(batch_size, seq_len, -1)


def linearattn_vk_mul_q(q: torch.Tensor, vk: torch.Tensor, num_tokens: int | None = None, eps: float = 1e-6) -> torch.Tensor:
    """Second half of the linear attention: ``q[b, t, h] <- (vk[b, h, :32] @ q[b, t, h]) / (vk[b, h, 32] . q[b, t, h] + eps)``
    in place (kernels::linearattn_vk_mul_q, gemm_w4a4_launch_impl.cuh:427-448).  q bf16 [B, tokens_pad, heads * 32]
    (``out_linearattn`` of ``svdq_gemm_w4a4``), vk fp32 [B, heads, 33, 32] (its ``out_vk``); only the first
    ``num_tokens`` rows of every batch entry are touched (all by default, as in the reference)."""
    import ctypes

    from .. import _native as nv

    nv.require_gpu(q, "q")
    nv.require_gpu(vk, "vk")
    if q.dim() != 3 or vk.dim() != 4 or q.dtype != torch.bfloat16 or vk.dtype != torch.float32:
        raise ValueError("q is bf16 [B, tokens_pad, heads * 32] and vk fp32 [B, heads, 33, 32]")
    B, tokens_pad, width = q.shape
    heads = vk.shape[1]
    if tuple(vk.shape) != (B, heads, 33, 32) or width != heads * 32 or vk.device != q.device:
        raise ValueError(f"vk has shape {tuple(vk.shape)}; q [{B}, {tokens_pad}, {width}] takes [{B}, {width // 32}, 33, 32] on the same device")
    num_tokens = tokens_pad if num_tokens is None else int(num_tokens)
    with torch.cuda.device(q.device):
        nv.check(nv.lib().svdq_linearattn_vk_mul_q(q.data_ptr(), vk.data_ptr(), B, num_tokens, tokens_pad, heads, ctypes.c_float(eps),
                                                   nv.stream_ptr(q.device)))
    return q
