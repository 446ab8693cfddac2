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
