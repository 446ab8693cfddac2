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


FRAG_BYTES = 1536  # one fp6 MFMA operand: 32 rows x 64 codes x 6 bits (csrc/svdq_common.h)
ACT_BLOCK_ROWS, WGT_BLOCK_COLS = 128, 256


def repack_qweight(qweight: torch.Tensor, fp4: bool = False) -> torch.Tensor:
    """int8 [N, K/2] reference order -> native weights.  INT4: E2M3 fragments
    ``[ceil(N/256)][K/64][8]`` as int8 ``[ceil(N/256) * 256, 3K/4]`` (``.logical_shape`` = (N, K));
    NVFP4: int8 [N, K/2] nibble tiles."""
    nv.require_gpu(qweight, "qweight")
    N, K2 = qweight.shape
    K = K2 * 2
    if fp4:
        out = torch.empty_like(qweight)
    else:
        n_pad = (N + WGT_BLOCK_COLS - 1) // WGT_BLOCK_COLS * WGT_BLOCK_COLS
        out = torch.empty(n_pad, K * 3 // 4, dtype=torch.int8, device=qweight.device)
    nv.check(nv.lib().svdq_repack_qweight(qweight.data_ptr(), out.data_ptr(), N, K, int(fp4), nv.stream_ptr(qweight.device)))
    return _tag(out, "qweight", logical_shape=(N, K))


def repack_wscales(wscales: torch.Tensor, fp4: bool = False) -> torch.Tensor:
    """Reference-order group scales -> native.  INT4 (bf16 [K/64, N]): the factor operand
    ``[ceil(N/256)][K/64][256] x {bf16(64 s), 0, 0, 0}`` as int64 ``[ceil(N/256), K/64, 256]``.
    NVFP4 (fp8 [K/16, N]): fp16 column-normalised ``[K/64][N][4]`` viewed as ``[K/16, N]``, with the
    fp32 per-column factor that undoes the normalisation as ``.colnorm``."""
    nv.require_gpu(wscales, "wscales")
    G, N = wscales.shape
    if fp4:
        out = torch.empty(G, N, dtype=torch.float16, device=wscales.device)
        colnorm = torch.empty(N, dtype=torch.float32, device=wscales.device)
        nv.check(nv.lib().svdq_repack_wmscales(wscales.data_ptr(), out.data_ptr(), colnorm.data_ptr(), N, G * 16, nv.stream_ptr(wscales.device)))
        return _tag(out, "wscales", colnorm=colnorm)
    nblocks = (N + WGT_BLOCK_COLS - 1) // WGT_BLOCK_COLS
    out = torch.empty(nblocks, G, WGT_BLOCK_COLS, dtype=torch.int64, device=wscales.device)
    nv.check(nv.lib().svdq_repack_wscales(wscales.data_ptr(), out.data_ptr(), N, G * 64, nv.stream_ptr(wscales.device)))
    return _tag(out, "wscales", colnorm=None)


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


def tensor_version(t: torch.Tensor) -> int | None:
    """The in-place modification counter of ``t``, or None for tensors that keep none (those created
    under ``torch.inference_mode()``)."""
    try:
        return t._version
    except RuntimeError:
        return None


def native(t: torch.Tensor | None, kind: str, fp4: bool = False) -> torch.Tensor | None:
    """Return the native form of ``t``: ``t`` itself when it already is native, else a cached repack
    of the reference-format tensor.  The cache notices in-place operations on the tensor and its
    replacement (version counter, identity); a tensor without a version counter (inference mode) is
    repacked on every call, and writes through ``t.data`` are invisible to it: pass native tensors
    (``repack_*``) where that matters."""
    if t is None or is_native(t, kind):
        return t
    version = tensor_version(t)
    if version is None:
        return _REPACKERS[kind](t, fp4) if kind in ("qweight", "wscales") else _REPACKERS[kind](t)
    key = (t.data_ptr(), version, tuple(t.shape), t.dtype, kind, fp4)
    hit = _cache.get(key)
    if hit is not None and hit[0]() is t:
        return hit[1]
    for k in [k for k, (ref, _) in _cache.items() if ref() is None]:
        del _cache[k]
    out = _REPACKERS[kind](t, fp4) if kind in ("qweight", "wscales") else _REPACKERS[kind](t)
    _cache[key] = (weakref.ref(t), out)
    return out


def require_nonzero(t: torch.Tensor | None, what: str) -> None:
    """Raise if a native per-channel vector holds a zero.  The NVFP4 GEMM adds the low-rank term in units of
    the column factor (column normalisation x alpha x wcscales), i.e. divides by it: a zero there would silently
    drop the term.  Checked once per tensor object (the check reads the tensor back: one synchronisation)."""
    if t is None or getattr(t, "_svdq_nonzero", False):
        return
    if bool((t == 0).any()):
        raise ValueError(f"{what} holds a zero: the NVFP4 kernel adds the low-rank term in units of the per-channel factor "
                         "and cannot divide by it (the reference multiplies only)")
    t._svdq_nonzero = True


# ---------------------------------------------------------------------------------------------
# logical views of the kernels' private 4-bit tile layout (for tests and debugging)
# ---------------------------------------------------------------------------------------------


def act_nbytes_per_row(K: int, fp4: bool = False) -> int:
    """Bytes of quantized activations per row: 4 bits per element for NVFP4, 6 (E2M3) for INT4."""
    return K // 2 if fp4 else K * 3 // 4


# E2M3 pattern of code / 8 for code in [-15, 15] (csrc/svdq_common.h, int4_code_to_e2m3), and its inverse
def _e2m3_of_code(code: int) -> int:
    x = abs(code)
    m = x  # subnormals x / 8 and the first binade 1 + (x - 8) / 8: the five low bits are the magnitude
    return m | (32 if code < 0 else 0)


_E2M3_TO_CODE = torch.full((64,), 127, dtype=torch.int8)
for _c in range(-15, 16):
    _E2M3_TO_CODE[_e2m3_of_code(_c)] = _c
_E2M3_TO_CODE[32] = 0  # minus zero: what the hardware conversion makes of a value that rounds to -0.0
_CODE_TO_E2M3 = torch.tensor([_e2m3_of_code(c) for c in range(-16, 16)], dtype=torch.uint8)  # index code + 16


def act_to_logical(act: torch.Tensor, K: int, fp4: bool = False, unsigned: bool = False) -> torch.Tensor:
    """Quantized activations in the kernels' private layout -> one code per element, int8 [M_pad, K] in
    row/column order.  INT4: E2M3 fragments ``[M_pad/128][K/64][4]`` (u8 [M_pad, 3K/4]); NVFP4: nibble
    tiles ``[M_pad/32][K/64][32 rows][8 words]`` (u8 [M_pad, K/2])."""
    M_pad = act.shape[0]
    if fp4:
        w = act.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
        nib = torch.stack([(w >> (4 * e)) & 0xF for e in range(8)], dim=-1)  # [M_pad, K/8, 8] in tile order
        return nib.reshape(M_pad // 32, K // 64, 32, 64).permute(0, 2, 1, 3).reshape(M_pad, K).to(torch.int8)
    return _fragments_to_logical(act, M_pad, K, ACT_BLOCK_ROWS)


def _fragments_to_logical(buf: torch.Tensor, rows: int, K: int, block_rows: int) -> torch.Tensor:
    """E2M3 fragments ``[rows/block_rows][K/64][block_rows/32]`` -> int8 codes [rows, K]."""
    import numpy as np

    nf = block_rows // 32
    f = buf.contiguous().cpu().view(torch.uint8).reshape(rows // block_rows, K // 64, nf, FRAG_BYTES)
    strings = torch.cat([f[..., :1024].reshape(*f.shape[:3], 64, 16), f[..., 1024:].reshape(*f.shape[:3], 64, 8)], dim=-1)
    bits = np.unpackbits(strings.numpy(), axis=-1, bitorder="little").reshape(*f.shape[:3], 64, 32, 6)
    pat = (bits * np.array([1, 2, 4, 8, 16, 32], dtype=np.uint8)).sum(axis=-1).astype(np.int64)  # [blk, g, frag, slot, 32]
    codes = _E2M3_TO_CODE[torch.from_numpy(pat)]
    assert (codes != 127).all(), "a pattern that is not code / 8 for any INT4 code"
    # slot = row + 32 * half, element j of a half is column 32 * half + j
    codes = codes.reshape(rows // block_rows, K // 64, nf, 2, 32, 32).permute(0, 2, 4, 1, 3, 5)  # blk, frag, row, g, half, j
    return codes.reshape(rows, K).contiguous().to(buf.device)


def qweight_to_logical(qweight_native: torch.Tensor) -> torch.Tensor:
    """Native INT4 weights (``repack_qweight``) -> int8 codes [N, K] (tests and debugging)."""
    N, K = qweight_native.logical_shape
    return _fragments_to_logical(qweight_native, qweight_native.shape[0], K, WGT_BLOCK_COLS)[:N]


def wscales_to_logical(wscales_native: torch.Tensor, N: int) -> torch.Tensor:
    """Native INT4 weight scales (``repack_wscales``) -> fp32 [K/64, N] (the factor 64 taken out again)."""
    w = wscales_native.cpu()  # int64 [nblocks, G, 256], bf16 bits of 64 * scale in the low 16 bits
    assert ((w >> 16) == 0).all(), "the upper three 16-bit slots of a scale entry must be zero"
    v = (w.to(torch.int32) << 16).view(torch.float32) * (1.0 / 64.0)
    return v.permute(1, 0, 2).reshape(w.shape[1], -1)[:, :N].contiguous()


def logical_to_act(codes: torch.Tensor, fp4: bool = False, unsigned: bool = False) -> torch.Tensor:
    """Inverse of :func:`act_to_logical` (used by tests to feed hand-made codes to the GEMM)."""
    M_pad, K = codes.shape
    if fp4:
        c = (codes.to(torch.int64) & 0xF).reshape(M_pad // 32, 32, K // 64, 8, 8).permute(0, 2, 1, 3, 4)  # tile, group, row, word, element
        w = sum(c[..., e] << (4 * e) for e in range(8))
        w = torch.where(w >= 2**31, w - 2**32, w).to(torch.int32)
        return w.contiguous().view(torch.uint8).reshape(M_pad, K // 2)
    import numpy as np

    pat = _CODE_TO_E2M3[codes.cpu().to(torch.int64) + 16]
    pat = pat.reshape(M_pad // ACT_BLOCK_ROWS, 4, 32, K // 64, 2, 32).permute(0, 3, 1, 4, 2, 5)  # blk, g, frag, half, row, j
    pat = pat.reshape(M_pad // ACT_BLOCK_ROWS, K // 64, 4, 64, 32).numpy()
    bits = ((pat[..., None] >> np.arange(6, dtype=np.uint8)) & 1).astype(np.uint8).reshape(*pat.shape[:4], 192)
    strings = torch.from_numpy(np.packbits(bits, axis=-1, bitorder="little"))  # [blk, g, frag, slot, 24]
    f = torch.cat([strings[..., :16].reshape(*pat.shape[:3], 1024), strings[..., 16:].reshape(*pat.shape[:3], 512)], dim=-1)
    return f.reshape(M_pad, K * 3 // 4).contiguous().to(codes.device)


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
