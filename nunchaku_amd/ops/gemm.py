"""``svdq_gemm_w4a4``: same keyword names and defaults as nunchaku/ops/gemm.py:11-158; results are
written in place into ``out`` / ``qout`` / ``oscales`` / ``lora_act_out``.
"""

from __future__ import annotations

import ctypes
import math

import torch

from .. import _native as nv
from .. import packing

_NOT_BUILT = ("poolout",)
NORM_EPS = 1e-6  # gemm_w4a4_launch_impl.cuh:374
# Tuning / testing knob handed to the C ABI as ``k_split``: None lets the library decide, n > 0 splits
# every output tile along K into n parts (1: never split).  No counterpart in the reference.
K_SPLIT: int | None = None
# True routes the call to ``svdq_gemm_w4a4_noalloc`` of the C ABI (same kernels, workspace from a fixed array
# in device memory instead of an allocation; for callers that cannot allocate, e.g. under graph capture).
NO_ALLOC: bool = False


def _expect(name: str, t: torch.Tensor | None, shape: tuple, dtype: torch.dtype | None, dev: torch.device) -> None:
    """The kernel reads and writes every row of these buffers: a wrong shape is an out-of-bounds access
    on the device, so it is refused here (the reference asserts the same shapes in
    gemm_w4a4_launch_impl.cuh:60-170)."""
    if t is None:
        return
    nv.require_gpu(t, name)
    if t.device != dev:
        raise ValueError(f"svdq_gemm_w4a4: `{name}` is on {t.device}, the activations on {dev}")
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"svdq_gemm_w4a4: `{name}` has shape {tuple(t.shape)}, expected {tuple(shape)}")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"svdq_gemm_w4a4: `{name}` has dtype {t.dtype}, expected {dtype}")


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

    act      u8 [M_pad, 3K/4] (INT4; [M_pad, K/2] for NVFP4) and ``ascales`` [K/G, M_pad], as returned by the
    quantize operator (the byte layout is private to the two operators);
    wgt / wscales / lora_up / bias / wcscales / smooth_factor / lora_down: the layer's tensors, in
    the reference checkpoint layout (repacked once and cached) or already native (``packing``);
    out      bf16 [M, N] (M <= M_pad);  qout / oscales / lora_act_out: inputs of the next layer, in
    which case a tanh-GELU is applied first (gemm_w4a4_launch_impl.cuh:282-309);
    norm_q / norm_k bf16 [128] and rotary_emb fp32 [B, M/B, 128] (packed by ``pack_rotemb``): RMS norm
    and rotary embedding on the q and k thirds of ``out`` (launch_impl.cuh:347-402);
    out_q / out_k / out_v fp16 [1, heads, M_pad, 128] (row ranges of larger tensors are fine) with
    attn_tokens: q, k, v apart, per head, in place of ``out``; rows from ``attn_tokens`` on hold 0 (q, v) and
    NaN (k) as in the reference (epilogues.cuh:427-550).  Within a head the values are plain [row, 128]; the
    reference orders them for its own attention kernel's matrix fragments.
    out_linearattn bf16 [B, tokens_pad, N/3] with out_vk fp32 [B, heads, 33, 32] (N = 3 * heads * 32, tokens_pad a
    multiple of 256): linear attention (launch_impl.cuh:311-345): relu(q) goes to out_linearattn;
    out_vk[b, h, i, j] = sum over tokens of v[i] * relu(k[j]) (i < 32) and of relu(k[j]) (i = 32), where the
    columns after q hold, per head, 32 of k then 32 of v.  out_vk is cleared first.
    """
    local = locals()
    for name in _NOT_BUILT:
        if local[name] is not None:
            # the reference's signature carries it, but no branch of its launcher consumes it any more (the epilogue
            # that did is commented out, gemm_w4a4_launch_impl.cuh:362-373)
            raise NotImplementedError(f"svdq_gemm_w4a4: `{name}` is not built (the reference ignores it)")
    for name in ("act", "wgt", "ascales", "wscales"):
        if local[name] is None:
            raise ValueError(f"svdq_gemm_w4a4: `{name}` is required")
        nv.require_gpu(local[name], name)
    if (lora_up is None) != (lora_act_in is None):
        raise ValueError("lora_up and lora_act_in must be given together")
    if (lora_down is None) != (lora_act_out is None):
        raise ValueError("lora_down and lora_act_out must be given together")
    qkv = (out_q, out_k, out_v)
    if any(t is not None for t in qkv) and (any(t is None for t in qkv) or rotary_emb is None or out is not None):
        raise ValueError("out_q, out_k and out_v go together, with rotary_emb and without `out` (launch_impl.cuh:380-397)")
    if (out_vk is None) != (out_linearattn is None):
        raise ValueError("out_vk and out_linearattn go together")  # the reference asserts it (launch_impl.cuh:313)
    if out_vk is not None:
        if out is not None or qout is not None or out_q is not None or rotary_emb is not None or fuse_silu:
            raise ValueError("out_vk / out_linearattn go without out, qout, out_q and rotary_emb (launch_impl.cuh:282-417 picks one branch)")
    if out is None and qout is None and out_q is None and out_vk is None:
        raise ValueError("one of out / qout / (out_q, out_k, out_v) / (out_vk, out_linearattn) is required")
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

    if act.dim() != 2 or act.dtype != torch.uint8:
        raise ValueError("svdq_gemm_w4a4: `act` must be the uint8 [M_pad, bytes] tensor written by the quantize operator")
    M_pad = act.shape[0]
    dev = act.device
    if packing.is_native(wgt, "qweight"):
        N, K = wgt.logical_shape
    else:
        N, K = wgt.shape[0], wgt.shape[1] * 2
    if M_pad % 256 != 0 or act.shape[1] != packing.act_nbytes_per_row(K, fp4):
        raise ValueError(
            f"svdq_gemm_w4a4: `act` has shape {tuple(act.shape)}; a layer with K={K} takes [M_pad, {packing.act_nbytes_per_row(K, fp4)}] "
            "with M_pad a multiple of 256 (the activation layout is private to the two operators)")
    G = 16 if fp4 else 64
    sdt = torch.float8_e4m3fn if fp4 else torch.bfloat16
    _expect("ascales", ascales, (K // G, M_pad), sdt, dev)
    if not packing.is_native(wscales, "wscales"):
        _expect("wscales", wscales, (K // G, N), sdt, dev)
    for name, t in (("bias", bias), ("wcscales", wcscales)):
        _expect(name, t, (N,), torch.bfloat16, dev)
    if lora_up is not None:
        _expect("lora_up", lora_up, (N, rank_up), torch.bfloat16, dev)
        _expect("lora_act_in", lora_act_in, (M_pad, rank_up), torch.float32, dev)
    if out is not None:
        nv.require_gpu(out, "out")
        if out.dtype != torch.bfloat16:
            raise NotImplementedError("only bf16 outputs are supported")
        if out.device != dev:
            raise ValueError("svdq_gemm_w4a4: `out` is on another device")
    if qout is not None:
        _expect("qout", qout, (M_pad, packing.act_nbytes_per_row(N, fp4)), torch.uint8, dev)
        _expect("oscales", oscales, (N // G, M_pad), sdt, dev)
        _expect("smooth_factor", smooth_factor, (N,), None, dev)
    if lora_down is not None:
        _expect("lora_down", lora_down, (N, lora_down.shape[1]), torch.bfloat16, dev)
        _expect("lora_act_out", lora_act_out, (M_pad, lora_down.shape[1]), torch.float32, dev)
    wgt_n = packing.native(wgt, "qweight", fp4)
    wsc_n = packing.native(wscales, "wscales", fp4)
    bias_n = packing.native(bias, "vector")
    wcs_n = packing.native(wcscales, "vector")
    if fp4 and lora_up is not None:
        packing.require_nonzero(wcs_n, "wcscales")
    up_n = packing.native(lora_up, "lora_up")
    nsm_n = packing.native(smooth_factor, "smooth_rcp") if qout is not None else None
    ndown_n = packing.native(lora_down, "lora_down")

    rot_n = None
    if rotary_emb is not None:
        rot_n = packing.native(rotary_emb, "rotemb")
        for name, t in (("norm_q", norm_q), ("norm_k", norm_k)):
            nv.require_gpu(t, name)
            if t.dtype != torch.bfloat16 or t.numel() != 128 or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous bf16 vector of 128 elements (one head)")
        if out_q is None and (out is None or out.shape[-1] != N):
            raise ValueError("rotary_emb needs a full-width `out`")
    qkv_strides = (0, 0, 0)
    if out_q is not None:
        if N % 384:
            raise ValueError("out_q / out_k / out_v need N to be three equal parts of 128-wide heads")
        for name, t in zip(("out_q", "out_k", "out_v"), qkv):
            if not t.is_cuda:
                raise RuntimeError(f"{name} must live on a GPU (got {t.device}); this path has no CPU implementation")
            if t.dtype != torch.float16 or t.device != dev or tuple(t.shape) != (1, N // 384, M_pad, 128) or t.stride(3) != 1 or t.stride(2) != 128:
                raise ValueError(
                    f"{name} must be float16 [1, {N // 384}, {M_pad}, 128] with contiguous rows (one batch: the reference places row "
                    f"block b of the GEMM at row block b of every head, epilogues.cuh:535), got {tuple(t.shape)} {t.dtype}")
        if not 0 <= attn_tokens <= M_pad:
            raise ValueError(f"attn_tokens must lie in [0, {M_pad}]")
        qkv_strides = tuple(t.stride(1) for t in qkv)

    vk_rows = 0
    if out_vk is not None:
        if N % 384:
            raise ValueError("out_vk needs N to be three equal parts of whole 128-column blocks")
        heads = N // 96
        if out_linearattn.dim() != 3 or out_vk.dim() != 4:
            raise ValueError("out_linearattn is [B, tokens_pad, N/3] and out_vk [B, heads, 33, 32]")
        B, vk_rows = out_linearattn.shape[0], out_linearattn.shape[1]
        _expect("out_linearattn", out_linearattn, (B, vk_rows, N // 3), torch.bfloat16, dev)
        _expect("out_vk", out_vk, (B, heads, 33, 32), torch.float32, dev)
        if vk_rows % 256 or B * vk_rows != M_pad:
            raise ValueError(f"out_linearattn holds {B} x {vk_rows} rows; the GEMM has {M_pad} (tokens are padded to a multiple of 256 per batch entry)")
        out = out_linearattn  # the q third is the plain store of this epilogue (epilogues.cuh:662-674)

    n_sc = max(1, math.ceil(rank_up / 16))
    sc = (ctypes.c_float * n_sc)(*[float(lora_scales[i]) if i < len(lora_scales) else 0.0 for i in range(n_sc)])
    M_out = 0 if out is None else out.numel() // out.shape[-1]
    N_out = 0 if out is None else out.shape[-1]
    args = nv.GemmArgs(
        act=act.data_ptr(), ascales=ascales.data_ptr(), wgt=wgt_n.data_ptr(), wscales=wsc_n.data_ptr(),
        colnorm=nv.ptr(wsc_n.colnorm), bias=nv.ptr(bias_n), wcscales=nv.ptr(wcs_n),
        lora_act_in=nv.ptr(lora_act_in), lora_up=nv.ptr(up_n), lora_scales=sc, out=nv.ptr(out),
        qout=nv.ptr(qout), oscales=nv.ptr(oscales), next_smooth_rcp=nv.ptr(nsm_n),
        next_lora_down=nv.ptr(ndown_n), next_lora_act_out=nv.ptr(lora_act_out),
        M_pad=M_pad, N=N, K=K, M_out=M_out, N_out=N_out, R_up=rank_up,
        R_down=0 if lora_down is None else lora_down.shape[1],
        alpha=float(alpha), act_unsigned=int(act_unsigned), fuse_silu=int(fuse_silu), fp4=int(fp4),
        norm_q=nv.ptr(norm_q), norm_k=nv.ptr(norm_k), rotary_emb=nv.ptr(rot_n),
        rot_rows=0 if rot_n is None else rot_n.shape[0], norm_eps=NORM_EPS, k_split=int(K_SPLIT or 0),
        out_q=nv.ptr(out_q), out_k=nv.ptr(out_k), out_v=nv.ptr(out_v), qkv_head_stride=(ctypes.c_int64 * 3)(*qkv_strides),
        attn_tokens=int(attn_tokens) if out_q is not None else 0, qkv_rows=M_pad if out_q is not None else 0,
        out_vk=nv.ptr(out_vk), vk_rows=vk_rows,
    )
    nv.launch(nv.lib().svdq_gemm_w4a4_noalloc if NO_ALLOC else nv.lib().svdq_gemm_w4a4, ctypes.byref(args), dev)


svdq_gemm_w4a4_cuda = svdq_gemm_w4a4
