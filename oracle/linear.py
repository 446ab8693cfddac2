"""Logical CPU restatement of the two ops and of the layer built from them.

Test infrastructure only (see ``oracle/__init__.py``).  Everything here works on *logical*
tensors (no lane permutations, no nibble packing); ``layouts.py`` covers the storage formats.
"""

from __future__ import annotations

import math

import torch

from . import quant


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """EpilogueGelu (src/kernels/zgemm/epilogues.cuh:22-44, gemm_utils.cuh:305-312): the tanh form of
    GELU evaluated in fp32; the library routine is the reference's formula with an exact tanh."""
    return torch.nn.functional.gelu(x.to(torch.float32), approximate="tanh")


def glu_input(x: torch.Tensor) -> torch.Tensor:
    """[M, 2K] pairs (value, gate) -> bf16 [M, K] ``value * silu(gate)``, each of the two operations
    rounded to bf16 (gemm_base.cuh:612-623, gemm_utils.cuh:322-327)."""
    value, gate = x[:, 0::2].to(torch.float64), x[:, 1::2].to(torch.float64)
    silu = (gate * torch.sigmoid(gate)).to(torch.float32).to(torch.bfloat16)
    return (value * silu.to(torch.float64)).to(torch.float32).to(torch.bfloat16)


def quantize_act_fuse_lora(
    x: torch.Tensor,
    proj_down: torch.Tensor,
    smooth: torch.Tensor | None,
    fp4: bool = False,
    pad_size: int = 256,
    fuse_glu: bool = False,
):
    """quantize_w4a4_fuse_lora_kernel (gemm_w4a4.cuh:1097-1184) behind
    svdq_quantize_w4a4_act_fuse_lora_cuda (nunchaku/ops/quantize.py:11-54).

    x bf16 [M, K]; proj_down bf16 [K, R] (logical); smooth bf16 [K] (logical) or None.
    Rows M..M_pad are zero-filled by the loader (gemm_base.cuh:591-646) and therefore quantize to
    code 0 / scale 0 / lora 0.  The low-rank projection uses the raw x (no smoothing):
    gemm_w4a4.cuh:1159-1171.
    ``fuse_glu``: x is [M, 2K], pairs (value, gate); what is smoothed, quantized and projected is
    ``bf16(value * bf16(gate * sigmoid(gate)))`` (load_act_to_fpsum<fuse_glu>, gemm_base.cuh:612-623:
    ``raw[j].x * silu(raw[j].y)`` in the activation type; silu rounds to that type itself,
    gemm_utils.cuh:322-327).
    Returns (codes [M_pad, K], scales [K/G, M_pad], lora_act fp32 [M_pad, R]).
    """
    if fuse_glu:
        x = glu_input(x)
    M, K = x.shape
    M_pad = (M + pad_size - 1) // pad_size * pad_size
    xp = torch.zeros(M_pad, K, dtype=torch.bfloat16)
    xp[:M] = x
    if fp4:
        codes, scales = quant.quantize_act_nvfp4(xp, smooth)
    else:
        codes, scales = quant.quantize_act_int4(xp, smooth, unsigned=False, shift=0.0)
    lora_act = xp.to(torch.float64) @ proj_down.to(torch.float64)
    return codes, scales, lora_act.to(torch.float32)


def gemm_w4a4(
    act_deq: torch.Tensor,
    wgt_deq: torch.Tensor,
    bias: torch.Tensor | None = None,
    lora_act_in: torch.Tensor | None = None,
    lora_up: torch.Tensor | None = None,
    lora_scales: list[float] | None = None,
    alpha: float = 1.0,
    wcscales: torch.Tensor | None = None,
    gelu: bool = False,
    silu: bool = False,
    double: bool = True,
) -> torch.Tensor:
    """The GEMM and its epilogue chain on dequantized operands, fp32 (or fp64) accumulated:
    ``acc = act_deq @ wgt_deq.T`` -> ``* alpha`` (gemm_w4a4.cuh:273-356) -> ``* wcscales + bias``
    (EpilogueBias, gemm_base.cuh:710-781) -> ``+ bf16(lora_act * scale[r/16]) @ up.T``
    (EpilogueLoraUp, lora.cuh:110-241) -> GELU / SiLU (epilogues.cuh:22-44, gemm_base.cuh:783-792).
    Order of the chain: gemm_w4a4_launch_impl.cuh:172-280.  The result is fp32; the caller rounds it
    to bf16 where the reference stores bf16.
    """
    dt = torch.float64 if double else torch.float32
    acc = act_deq.to(dt) @ wgt_deq.to(dt).t()
    acc = acc * alpha
    if wcscales is not None:
        acc = acc * wcscales.to(dt)[None, :]
    if bias is not None:
        acc = acc + bias.to(dt)[None, :]
    if lora_up is not None:
        R = lora_up.shape[1]
        if lora_scales is None:
            lora_scales = [1.0] * math.ceil(R / 16)
        sc = torch.tensor([lora_scales[r // 16] if r // 16 < len(lora_scales) else 0.0 for r in range(R)], dtype=torch.float32)
        a = quant.bf16(lora_act_in.to(torch.float32) * sc[None, :])
        acc = acc + a.to(dt) @ lora_up.to(dt).t()
    acc = acc.to(torch.float32)
    if gelu:
        acc = gelu_tanh(acc)
    if silu:
        acc = acc * torch.sigmoid(acc)
    return acc


class FakeQuantLinear:
    """Logical-tensor model of SVDQW4A4Linear.forward (nunchaku/models/linear.py:89-132):
    quantize (+ low-rank down) then GEMM (+ bias, low-rank up).  Also the CPU baseline that the
    bench times."""

    def __init__(self, wq, ws, smooth, proj_down, proj_up, bias=None, fp4=False, wtscale=1.0, wcscales=None, act_unsigned=False):
        self.fp4 = fp4
        self.w_deq = quant.dequant_nvfp4(wq, ws) if fp4 else quant.dequant_int4(wq, ws)
        self.smooth, self.proj_down, self.proj_up, self.bias = smooth, proj_down, proj_up, bias
        self.wtscale, self.wcscales, self.act_unsigned = wtscale, wcscales, act_unsigned

    def quantize(self, x):
        return quantize_act_fuse_lora(x, self.proj_down, self.smooth, fp4=self.fp4)

    def forward_quant(self, codes, scales, lora_act, gelu=False, double=True):
        a = quant.dequant_nvfp4(codes, scales) if self.fp4 else quant.dequant_int4(codes, scales)
        return gemm_w4a4(
            a, self.w_deq, bias=self.bias, lora_act_in=lora_act, lora_up=self.proj_up,
            alpha=self.wtscale, wcscales=self.wcscales, gelu=gelu, double=double,
        )

    def forward(self, x, double=True):
        codes, scales, lora_act = self.quantize(x)
        return self.forward_quant(codes, scales, lora_act, double=double)[: x.shape[0]]


def fused_gelu_mlp(x: torch.Tensor, fc1: FakeQuantLinear, fc2: FakeQuantLinear, double: bool = True):
    """nunchaku/ops/fused.py:10-47: fc1 GEMM with GELU, then the post-GELU bf16 tile is (a) projected
    by fc2's down projection and (b) shifted by 0.171875, smoothed and quantized unsigned for fc2
    (gemm_w4a4_launch_impl.cuh:282-309).  Returns (out fp32 [M, N2], intermediates dict)."""
    codes, scales, lora_act = fc1.quantize(x)
    h = quant.bf16(fc1.forward_quant(codes, scales, lora_act, gelu=True, double=double))
    lora2 = (h.to(torch.float64) @ fc2.proj_down.to(torch.float64)).to(torch.float32)
    if fc2.fp4:
        qcodes, qscales = quant.quantize_act_nvfp4(h.to(torch.bfloat16), fc2.smooth)
    else:
        qcodes, qscales = quant.quantize_act_int4(h.to(torch.bfloat16), fc2.smooth, unsigned=True, shift=quant.SHIFT_GELU)
    out = fc2.forward_quant(qcodes, qscales, lora2, double=double)[: x.shape[0]]
    return out, {"h": h, "qcodes": qcodes, "qscales": qscales, "lora2": lora2}


def rmsnorm_rope(out: torch.Tensor, norm_q: torch.Tensor, norm_k: torch.Tensor, rotemb: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """EpilogueRMSNormRope (src/kernels/zgemm/epilogues.cuh:269-425) on the output of a fused QKV
    projection, composed after bias and low-rank up (gemm_w4a4_launch_impl.cuh:347-402).

    out fp32 [M, N] with N = 3 * heads * 128: columns [0, N/3) are q, [N/3, 2N/3) are k, the rest is
    v and passes through (epilogues.cuh:413-424).  Per row and 128-wide head:
    ``x *= rsqrt(mean(x^2) + eps) * weight`` (:338-372), then every pair (x[2i], x[2i+1]) is rotated:
    ``(x cos - y sin, x sin + y cos)`` with (sin, cos) = rotemb[row, 2i], rotemb[row, 2i + 1]
    (:374-392; the table is [M, 128] logical, see layouts.pack_rotemb).  Evaluated in fp64; the
    reference rounds to bf16 before and after, the caller rounds where it stores.
    """
    M, N = out.shape
    assert N % 384 == 0 and rotemb.shape == (M, 128)
    x = out.to(torch.float64).clone()
    third = N // 3
    sin, cos = rotemb[:, 0::2].to(torch.float64), rotemb[:, 1::2].to(torch.float64)  # [M, 64]
    for part, w in ((0, norm_q), (1, norm_k)):
        h = x[:, part * third:(part + 1) * third].reshape(M, third // 128, 128)
        coef = torch.rsqrt((h * h).mean(dim=-1, keepdim=True) + eps)
        h = h * coef * w.to(torch.float64)[None, None, :]
        a, b = h[..., 0::2], h[..., 1::2]
        r = torch.stack((a * cos[:, None, :] - b * sin[:, None, :], a * sin[:, None, :] + b * cos[:, None, :]), dim=-1)
        x[:, part * third:(part + 1) * third] = r.reshape(M, third)
    return x.to(torch.float32)


def pack_qkv(out: torch.Tensor, attn_tokens: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """EpiloguePackQKV (src/kernels/zgemm/epilogues.cuh:427-550), composed after the norm and rotation
    (gemm_w4a4_launch_impl.cuh:380-397), as logical tensors.

    out fp32 [M_pad, N], N = 3 * heads * 128, the epilogue's input before its bf16 rounding.  Column block b of
    128 is head ``b % heads`` of q (b < heads), k (b < 2 heads) or v (:517-533).  Values are rounded to bf16
    (the GEMM's tile type) and converted to fp16 through fp32 (``convert_half2``, :446-453).  Rows from
    ``attn_tokens`` on are replaced by the mask value of the tensor: 0 for q and v, NaN for k (:482-492,
    :539-545).  Returns three fp16 [1, heads, M_pad, 128] tensors holding [row, dim] per head; the reference
    stores the same values in the order of its attention kernel's matrix fragments (:494-512), which is
    private to that kernel and not restated.
    """
    M_pad, N = out.shape
    assert N % 384 == 0
    heads = N // 384
    x = out.to(torch.bfloat16).to(torch.float32).to(torch.float16)
    parts = []
    for i, mask in enumerate((0.0, float("nan"), 0.0)):
        t = x[:, i * heads * 128:(i + 1) * heads * 128].reshape(M_pad, heads, 128).permute(1, 0, 2).contiguous()
        t[:, attn_tokens:, :] = mask
        parts.append(t[None])
    return tuple(parts)


def litela(out: torch.Tensor, batch: int) -> tuple[torch.Tensor, torch.Tensor]:
    """EpilogueLiteLA (src/kernels/zgemm/epilogues.cuh:552-681) on the output of a fused QKV projection of a
    linear-attention block, selected as in gemm_w4a4_launch_impl.cuh:311-345.

    out fp32 [batch * tokens_pad, N], N = 3 * heads * 32, before the bf16 rounding of the GEMM tile.  Columns
    [0, N/3) are q: ``relu`` (:662-664).  The other columns hold, per head, 32 of k then 32 of v (:600-603): with
    k' = relu(k) (:605-607), ``vk[b, h, i, j] = sum_t v[t, i] * k'[t, j]`` for i < 32 (:598-622; row = v index,
    column = k index) and ``vk[b, h, 32, j] = sum_t k'[t, j]`` (:624-646, v replaced by ones), over ALL rows of batch
    entry b, padding rows included, in fp32 on the bf16-rounded values.
    Returns (q fp32 [batch, tokens_pad, N/3] holding bf16 values, vk fp64 [batch, heads, 33, 32]).
    """
    M, N = out.shape
    assert N % 96 == 0 and M % batch == 0
    heads, rows = N // 96, M // batch
    x = out.to(torch.bfloat16).to(torch.float64)
    q = torch.relu(x[:, : N // 3]).reshape(batch, rows, N // 3).to(torch.float32)
    kv = x[:, N // 3:].reshape(batch, rows, heads, 64)
    k, v = torch.relu(kv[..., :32]), kv[..., 32:]
    vk = torch.zeros(batch, heads, 33, 32, dtype=torch.float64)
    vk[:, :, :32] = torch.einsum("bthi,bthj->bhij", v, k)
    vk[:, :, 32] = k.sum(dim=1)
    return q, vk


def linearattn_vk_mul_q(q: torch.Tensor, vk: torch.Tensor, num_tokens: int, eps: float = 1e-6) -> torch.Tensor:
    """vk_mul_q_kernel (epilogues.cuh:683-744): per token and head, ``o[j] = sum_i q[i] * vk[j][i]`` for j <= 32,
    result ``o[:32] / (o[32] + eps)``; rows from ``num_tokens`` on keep their input.  fp64; q [B, T, heads * 32],
    vk [B, heads, 33, 32]."""
    B, T, W = q.shape
    heads = W // 32
    qh = q.to(torch.float64).reshape(B, T, heads, 32)
    o = torch.einsum("bthi,bhji->bthj", qh, vk.to(torch.float64))
    res = (o[..., :32] / (o[..., 32:] + eps)).reshape(B, T, W)
    res[:, num_tokens:] = q.to(torch.float64)[:, num_tokens:]
    return res
