"""Load-time repack of reference-format checkpoint tensors into the gfx950-native layouts, and the
inverse views the tests need to compare kernel outputs in logical order.

Reference formats: ``NunchakuWeightPacker`` (nunchaku/lora/flux/packer.py:187-398).  The byte
shuffling itself runs on the GPU behind the C ABI (``svdq_repack_*``); this module only allocates
the destination tensors and keeps a small cache so that an operator called with a reference-format
tensor (as nunchaku.ops callers do) repacks it once, not per call.
"""

from __future__ import annotations

import weakref

import torch

from . import _native as nv

NATIVE_ATTR = "_svdq_native"


def _tag(t: torch.Tensor, kind: str, **extra) -> torch.Tensor:
    setattr(t, NATIVE_ATTR, kind)
    for k, v in extra.items():
        setattr(t, k, v)
    return t


def is_native(t: torch.Tensor | None, kind: str) -> bool:
    return t is not None and getattr(t, NATIVE_ATTR, None) == kind


def repack_qweight(qweight: torch.Tensor, fp4: bool = False) -> torch.Tensor:
    """int8 [N, K/2] reference order -> int8 [N, K/2] native tiles (offset-binary INT4 codes)."""
    nv.require_gpu(qweight, "qweight")
    N, K2 = qweight.shape
    out = torch.empty_like(qweight)
    nv.check(nv.lib().svdq_repack_qweight(qweight.data_ptr(), out.data_ptr(), N, K2 * 2, int(fp4), nv.stream_ptr(qweight.device)))
    return _tag(out, "qweight")


def repack_wscales(wscales: torch.Tensor, fp4: bool = False) -> torch.Tensor:
    """bf16 [K/64, N] (or fp8 [K/16, N]) reference order -> fp16 column-normalised scales with the
    same element count (INT4: ``[K/64][N]``; NVFP4: ``[K/64][N][4]`` viewed as ``[K/16, N]``); the
    fp32 per-column factor that undoes the normalisation rides along as ``.colnorm``."""
    nv.require_gpu(wscales, "wscales")
    G, N = wscales.shape
    out = torch.empty(G, N, dtype=torch.float16, device=wscales.device)
    colnorm = torch.empty(N, dtype=torch.float32, device=wscales.device)
    fn = nv.lib().svdq_repack_wmscales if fp4 else nv.lib().svdq_repack_wscales
    K = G * (16 if fp4 else 64)
    nv.check(fn(wscales.data_ptr(), out.data_ptr(), colnorm.data_ptr(), N, K, nv.stream_ptr(wscales.device)))
    return _tag(out, "wscales", colnorm=colnorm)


def repack_vector(vec: torch.Tensor) -> torch.Tensor:
    """bias / wcscales / smooth_factor bf16 [N]: reference lane order -> channel order."""
    nv.require_gpu(vec, "vector")
    out = torch.empty_like(vec)
    nv.check(nv.lib().svdq_repack_vector(vec.data_ptr(), out.data_ptr(), vec.numel(), nv.stream_ptr(vec.device)))
    return _tag(out, "vector")


def repack_smooth(smooth: torch.Tensor) -> torch.Tensor:
    """smooth_factor bf16 [K] reference lane order -> fp32 [K] correctly rounded reciprocals."""
    nv.require_gpu(smooth, "smooth_factor")
    out = torch.empty(smooth.numel(), dtype=torch.float32, device=smooth.device)
    nv.check(nv.lib().svdq_repack_smooth(smooth.data_ptr(), out.data_ptr(), smooth.numel(), nv.stream_ptr(smooth.device)))
    return _tag(out, "smooth_rcp")


def repack_lora_down(proj_down: torch.Tensor) -> torch.Tensor:
    """bf16 [K, R] reference order -> native MFMA operand order (same shape and dtype)."""
    nv.require_gpu(proj_down, "proj_down")
    K, R = proj_down.shape
    out = torch.empty_like(proj_down)
    if R == 0:  # a layer without a low-rank branch
        return _tag(out, "lora_down")
    nv.check(nv.lib().svdq_repack_lora_down(proj_down.data_ptr(), out.data_ptr(), K, R, nv.stream_ptr(proj_down.device)))
    return _tag(out, "lora_down")


def repack_lora_up(proj_up: torch.Tensor) -> torch.Tensor:
    """bf16 [N, R] reference order -> row-major channel/rank order."""
    nv.require_gpu(proj_up, "proj_up")
    N, R = proj_up.shape
    out = torch.empty_like(proj_up)
    if R == 0:
        return _tag(out, "lora_up")
    nv.check(nv.lib().svdq_repack_lora_up(proj_up.data_ptr(), out.data_ptr(), N, R, nv.stream_ptr(proj_up.device)))
    return _tag(out, "lora_up")


def repack_rotemb(rotemb: torch.Tensor) -> torch.Tensor:
    """Rotary table fp32 [B, M, 128] (or [M, 128]) in the order written by ``pack_rotemb``
    (nunchaku/models/embeddings.py:88-120) -> the order the GEMM epilogue reads (same element count;
    ``include/svdq_amd.h``, ``svdq_gemm_args.rotary_emb``).  The row count must be a multiple of 32."""
    nv.require_gpu(rotemb, "rotary_emb")
    if rotemb.dtype != torch.float32 or not rotemb.is_contiguous():
        raise ValueError("rotary_emb must be a contiguous float32 tensor")
    rows = rotemb.numel() // rotemb.shape[-1]
    if rotemb.shape[-1] != 128:
        raise ValueError(f"rotary_emb must be [.., M, 128], got {tuple(rotemb.shape)}")
    out = torch.empty(rows, 128, dtype=torch.float32, device=rotemb.device)
    nv.check(nv.lib().svdq_repack_rotemb(rotemb.data_ptr(), out.data_ptr(), rows, nv.stream_ptr(rotemb.device)))
    return _tag(out, "rotemb")


_REPACKERS = {
    "qweight": repack_qweight,
    "wscales": repack_wscales,
    "vector": repack_vector,
    "smooth_rcp": repack_smooth,
    "lora_down": repack_lora_down,
    "lora_up": repack_lora_up,
    "rotemb": repack_rotemb,
}

# (data_ptr, version, shape, dtype, kind, fp4) -> (weakref to the source, native tensor)
_cache: dict[tuple, tuple[weakref.ref, torch.Tensor]] = {}


def native(t: torch.Tensor | None, kind: str, fp4: bool = False) -> torch.Tensor | None:
    """Return the native form of ``t``: ``t`` itself when it already is native, else a cached repack
    of the reference-format tensor (redone when the source is modified or replaced)."""
    if t is None or is_native(t, kind):
        return t
    key = (t.data_ptr(), t._version, tuple(t.shape), t.dtype, kind, fp4)
    hit = _cache.get(key)
    if hit is not None and hit[0]() is t:
        return hit[1]
    for k in [k for k, (ref, _) in _cache.items() if ref() is None]:
        del _cache[k]
    out = _REPACKERS[kind](t, fp4) if kind in ("qweight", "wscales") else _REPACKERS[kind](t)
    _cache[key] = (weakref.ref(t), out)
    return out


# ---------------------------------------------------------------------------------------------
# logical views of the kernels' private 4-bit tile layout (for tests and debugging)
# ---------------------------------------------------------------------------------------------


INT4_WORD_ROT = 2  # INT4 code words are stored rotated left by this many bits (csrc/svdq_common.h)


def act_to_logical(act: torch.Tensor, K: int, fp4: bool = False, unsigned: bool = False) -> torch.Tensor:
    """Native activation tiles u8 [M_pad, K/2] ([M_pad/32][K/64][32 rows][8 words]) -> one code per
    element, int8 [M_pad, K] in row/column order.  INT4 words are stored rotated left by 2 bits and
    signed codes offset-binary (code + 8); NVFP4 words are plain nibbles."""
    M_pad = act.shape[0]
    w = act.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    if not fp4:
        w = ((w >> INT4_WORD_ROT) | (w << (32 - INT4_WORD_ROT))) & 0xFFFFFFFF
    nib = torch.stack([(w >> (4 * e)) & 0xF for e in range(8)], dim=-1)  # [M_pad, K/8, 8] in tile order
    codes = nib.reshape(M_pad // 32, K // 64, 32, 64).permute(0, 2, 1, 3).reshape(M_pad, K)
    if not fp4 and not unsigned:
        codes = codes - 8
    return codes.to(torch.int8)


def logical_to_act(codes: torch.Tensor, fp4: bool = False, unsigned: bool = False) -> torch.Tensor:
    """Inverse of :func:`act_to_logical` (used by tests to feed hand-made codes to the GEMM)."""
    M_pad, K = codes.shape
    c = codes.to(torch.int64)
    if not fp4 and not unsigned:
        c = c + 8
    c = (c & 0xF).reshape(M_pad // 32, 32, K // 64, 8, 8).permute(0, 2, 1, 3, 4)  # tile, group, row, word, element
    w = sum(c[..., e] << (4 * e) for e in range(8))
    if not fp4:
        w = ((w << INT4_WORD_ROT) | (w >> (32 - INT4_WORD_ROT))) & 0xFFFFFFFF
    w = torch.where(w >= 2**31, w - 2**32, w).to(torch.int32)
    return w.contiguous().view(torch.uint8).reshape(M_pad, K // 2)


def scales_to_logical(scales: torch.Tensor, fp4: bool = False) -> torch.Tensor:
    """Activation scales as the kernels store them -> ``[K/G, M_pad]`` group-major.  INT4 scales are
    stored that way already; NVFP4 scales are stored ``[K/64][M_pad][4]``."""
    if not fp4:
        return scales
    G16, M_pad = scales.shape
    return scales.view(torch.uint8).reshape(G16 // 4, M_pad, 4).permute(0, 2, 1).reshape(G16, M_pad).contiguous().view(scales.dtype)


def logical_to_scales(scales: torch.Tensor, fp4: bool = False) -> torch.Tensor:
    """Inverse of :func:`scales_to_logical`."""
    if not fp4:
        return scales
    G16, M_pad = scales.shape
    return scales.view(torch.uint8).reshape(G16 // 4, 4, M_pad).permute(0, 2, 1).contiguous().reshape(G16, M_pad).view(scales.dtype)
