"""``fused_gelu_mlp`` and ``fused_qkv_norm_rottary`` with the signatures of nunchaku/ops/fused.py:10-110."""

from __future__ import annotations

import torch

from ..utils import ceil_divide
from .gemm import svdq_gemm_w4a4


def fused_gelu_mlp(x: torch.Tensor, fc1, fc2, pad_size: int = 256) -> torch.Tensor:
    """fc1 -> GELU -> fc2 with the GELU, fc2's activation quantization (unsigned INT4 after a
    +0.171875 shift) and fc2's low-rank down projection fused into fc1's GEMM epilogue
    (nunchaku/ops/fused.py:10-47).  Three calls into the library through the layers' prepared argument blocks."""
    batch_size, seq_len, channels = x.shape
    M = batch_size * seq_len
    x = x.view(M, channels)
    if pad_size % 256 != 0:
        raise ValueError("pad_size must be a multiple of 256")
    if fc1.out_features != fc2.in_features or fc1.precision != fc2.precision:
        raise ValueError(f"fc2 ({fc2}) does not take what fc1 ({fc1}) gives")
    if M == 0:
        return x.new_empty(batch_size, seq_len, fc2.out_features)
    c1 = fc1._prepared(x)
    dev = c1.device
    c2 = fc2._blocks(dev)
    M_pad = ceil_divide(M, pad_size) * pad_size
    quantized_x, ascales, lora_act = fc1._quantize_prepared(c1, x, M_pad)
    qout_act = torch.empty(M_pad, c2.act_bytes, dtype=torch.uint8, device=dev)
    qout_ascales = torch.empty(c2.groups, M_pad, dtype=c2.scale_dtype, device=dev)
    qout_lora_act = torch.empty(M_pad, fc2.rank, dtype=torch.float32, device=dev)
    fc1._gemm_prepared(
        c1, quantized_x, ascales, lora_act, M_pad,
        qout=qout_act.data_ptr(), oscales=qout_ascales.data_ptr(), next_smooth_rcp=c2.q.smooth_rcp,
        next_lora_down=c2.q.lora_down, next_lora_act_out=qout_lora_act.data_ptr() if fc2.rank else None, R_down=fc2.rank,
    )
    output = torch.empty(M, fc2.out_features, dtype=x.dtype, device=dev)
    fc2._gemm_prepared(c2, qout_act, qout_ascales, qout_lora_act, M_pad, out=output.data_ptr(), M_out=M)
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
    c = proj._prepared(x)
    quantized_x, ascales, lora_act = proj._quantize_prepared(c, x, ceil_divide(x.shape[0], 256) * 256)
    t = c.tensors
    common = dict(
        act=quantized_x, wgt=t["qweight"], ascales=ascales, wscales=t["wscales"], lora_act_in=lora_act, lora_up=t["proj_up"],
        bias=t["bias"], fp4=c.fp4, alpha=c.g.alpha, wcscales=t["wcscales"], norm_q=norm_q.weight,
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
