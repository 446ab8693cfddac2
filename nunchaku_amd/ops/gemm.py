"""``svdq_gemm_w4a4``: same keyword names and defaults as nunchaku/ops/gemm.py:11-158; results are
written in place into ``out`` / ``qout`` / ``oscales`` / ``lora_act_out``.
"""

from __future__ import annotations

import ctypes
import math

import torch

from .. import _native as nv
from .. import packing

_NOT_BUILT = ("poolout", "out_vk", "out_linearattn", "out_q", "out_k", "out_v")
NORM_EPS = 1e-6  # gemm_w4a4_launch_impl.cuh:374


def svdq_gemm_w4a4(
    act: torch.Tensor,
    wgt: torch.Tensor,
    out: torch.Tensor | None = None,
    qout: torch.Tensor | None = None,
    ascales: torch.Tensor | None = None,
    wscales: torch.Tensor | None = None,
    oscales: torch.Tensor | None = None,
    poolout: torch.Tensor | None = None,
    lora_act_in: torch.Tensor | None = None,
    lora_up: torch.Tensor | None = None,
    lora_down: torch.Tensor | None = None,
    lora_act_out: torch.Tensor | None = None,
    norm_q: torch.Tensor | None = None,
    norm_k: torch.Tensor | None = None,
    rotary_emb: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    smooth_factor: torch.Tensor | None = None,
    out_vk: torch.Tensor | None = None,
    out_linearattn: torch.Tensor | None = None,
    act_unsigned: bool = False,
    lora_scales: list[float] | None = None,
    fuse_silu: bool = False,
    fp4: bool = False,
    alpha: float | None = 1.0,
    wcscales: torch.Tensor | None = None,
    out_q: torch.Tensor | None = None,
    out_k: torch.Tensor | None = None,
    out_v: torch.Tensor | None = None,
    attn_tokens: int = 0,
) -> None:
    """W4A4 GEMM with fused bias, low-rank up projection, optional GELU and next-layer quantization.

    act      u8 [M_pad, K/2] and ``ascales`` [K/G, M_pad], as returned by the quantize operator;
    wgt / wscales / lora_up / bias / wcscales / smooth_factor / lora_down: the layer's tensors, in
    the reference checkpoint layout (repacked once and cached) or already native (``packing``);
    out      bf16 [M, N] (M <= M_pad);  qout / oscales / lora_act_out: inputs of the next layer, in
    which case a tanh-GELU is applied first (gemm_w4a4_launch_impl.cuh:282-309);
    norm_q / norm_k bf16 [128] and rotary_emb fp32 [B, M/B, 128] (packed by ``pack_rotemb``): RMS norm
    and rotary embedding on the q and k thirds of ``out`` (launch_impl.cuh:347-402, the ``out`` form;
    the ``out_q / out_k / out_v`` form that packs for the attention kernel is not built).
    """
    local = locals()
    for name in _NOT_BUILT:
        if local[name] is not None:
            raise NotImplementedError(f"svdq_gemm_w4a4: `{name}` (attention / linear-attention epilogues) is not built")
    for name in ("act", "wgt", "ascales", "wscales"):
        if local[name] is None:
            raise ValueError(f"svdq_gemm_w4a4: `{name}` is required")
        nv.require_gpu(local[name], name)
    if (lora_up is None) != (lora_act_in is None):
        raise ValueError("lora_up and lora_act_in must be given together")
    if (lora_down is None) != (lora_act_out is None):
        raise ValueError("lora_down and lora_act_out must be given together")
    if out is None and qout is None:
        raise ValueError("one of out / qout is required")
    if qout is not None and (oscales is None or smooth_factor is None):
        raise ValueError("qout needs oscales and smooth_factor")
    if rotary_emb is not None and (norm_q is None or norm_k is None):
        raise ValueError("rotary_emb needs norm_q and norm_k")  # the reference asserts both (launch_impl.cuh:348-349)
    if rotary_emb is None and (norm_q is not None or norm_k is not None):
        raise ValueError("norm_q / norm_k need rotary_emb")

    if lora_up is not None and lora_up.shape[1] == 0:  # rank-0 layer: no low-rank branch
        lora_up = lora_act_in = None
    if lora_down is not None and lora_down.shape[1] == 0:
        lora_down = lora_act_out = None
    rank_up = 0 if lora_up is None else lora_up.shape[1]
    if lora_scales is None:
        lora_scales = [1.0] * math.ceil(rank_up / 16)
    if alpha is None:
        alpha = 1.0
    if isinstance(alpha, torch.Tensor):  # the reference passes the wtscale parameter here (linear.py:128)
        alpha = float(alpha.item()) if alpha.numel() == 1 else 1.0

    M_pad, K = act.shape[0], act.shape[1] * 2
    N = wgt.shape[0]
    dev = act.device
    wgt_n = packing.native(wgt, "qweight", fp4)
    wsc_n = packing.native(wscales, "wscales", fp4)
    bias_n = packing.native(bias, "vector")
    wcs_n = packing.native(wcscales, "vector")
    up_n = packing.native(lora_up, "lora_up")
    nsm_n = packing.native(smooth_factor, "smooth_rcp") if qout is not None else None
    ndown_n = packing.native(lora_down, "lora_down")
    for name, t in (("out", out), ("qout", qout), ("oscales", oscales), ("lora_act_in", lora_act_in), ("lora_act_out", lora_act_out)):
        if t is not None:
            nv.require_gpu(t, name)
    if out is not None and out.dtype != torch.bfloat16:
        raise NotImplementedError("only bf16 outputs are supported")

    rot_n = None
    if rotary_emb is not None:
        rot_n = packing.native(rotary_emb, "rotemb")
        for name, t in (("norm_q", norm_q), ("norm_k", norm_k)):
            nv.require_gpu(t, name)
            if t.dtype != torch.bfloat16 or t.numel() != 128 or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous bf16 vector of 128 elements (one head)")
        if out is None or out.shape[-1] != N:
            raise ValueError("rotary_emb needs a full-width `out`")

    n_sc = max(1, math.ceil(rank_up / 16))
    sc = (ctypes.c_float * n_sc)(*[float(lora_scales[i]) if i < len(lora_scales) else 0.0 for i in range(n_sc)])
    M_out = 0 if out is None else out.numel() // out.shape[-1]
    N_out = 0 if out is None else out.shape[-1]
    args = nv.GemmArgs(
        act=act.data_ptr(), ascales=ascales.data_ptr(), wgt=wgt_n.data_ptr(), wscales=wsc_n.data_ptr(),
        colnorm=wsc_n.colnorm.data_ptr(), bias=nv.ptr(bias_n), wcscales=nv.ptr(wcs_n),
        lora_act_in=nv.ptr(lora_act_in), lora_up=nv.ptr(up_n), lora_scales=sc, out=nv.ptr(out),
        qout=nv.ptr(qout), oscales=nv.ptr(oscales), next_smooth_rcp=nv.ptr(nsm_n),
        next_lora_down=nv.ptr(ndown_n), next_lora_act_out=nv.ptr(lora_act_out),
        M_pad=M_pad, N=N, K=K, M_out=M_out, N_out=N_out, R_up=rank_up,
        R_down=0 if lora_down is None else lora_down.shape[1],
        alpha=float(alpha), act_unsigned=int(act_unsigned), fuse_silu=int(fuse_silu), fp4=int(fp4),
        norm_q=nv.ptr(norm_q), norm_k=nv.ptr(norm_k), rotary_emb=nv.ptr(rot_n),
        rot_rows=0 if rot_n is None else rot_n.shape[0], norm_eps=NORM_EPS,
    )
    nv.check(nv.lib().svdq_gemm_w4a4(ctypes.byref(args), nv.stream_ptr(dev)))


svdq_gemm_w4a4_cuda = svdq_gemm_w4a4
