"""Logical (layout-free) quantizers of the SVDQuant W4A4 path, restated in IEEE fp32 on the CPU.

Test infrastructure only (see ``oracle/__init__.py``).

All tensors here are *logical*: codes are one small integer per element (not nibble-packed, not
lane-permuted), scales are ``[groups, rows]`` exactly as the reference advertises their shapes.
"""

from __future__ import annotations

import numpy as np
import torch

INT4_GROUP = 64
NVFP4_GROUP = 16
SHIFT_GELU = 0.171875  # src/kernels/zgemm/gemm_w4a4_launch_impl.cuh:286

# fl32(1/7) and fl32(1/15): the reference multiplies by these constants instead of dividing
# (src/kernels/zgemm/gemm_w4a4.cuh:435-441,476-477).
RECIP_7 = np.float32(1.0) / np.float32(7.0)
RECIP_15 = np.float32(1.0) / np.float32(15.0)
RECIP_6 = np.float32(1.0) / np.float32(6.0)  # gemm_w4a4.cuh:91-92
assert RECIP_7.view(np.uint32) == 0x3E124925 and RECIP_15.view(np.uint32) == 0x3D888889

# E2M1 magnitudes by 3-bit pattern (exponent bias 1, one mantissa bit); bit 3 is the sign.
E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def bf16(x: torch.Tensor) -> torch.Tensor:
    """Round an fp32 tensor to bf16 (round-to-nearest-even) and return it as fp32."""
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float32)


def _smooth_divide(x: torch.Tensor, smooth: torch.Tensor | None, shift: float) -> torch.Tensor:
    """Steps 1-2 of the activation quantizer: ``bf16(bf16(x + shift) / smooth)``.

    Follows EpilogueQuantize::apply_quantize (gemm_w4a4.cuh:972-993): the tile is bf16, the shift is
    added in bf16, the division is done in fp32 (h2div, gemm_utils.cuh:337-343) and rounded back to
    bf16.  The reference's ``__fdividef`` is replaced by the correctly rounded IEEE quotient.
    """
    t = bf16(x.to(torch.float32) + torch.tensor(shift, dtype=torch.float32))
    if smooth is None:
        return t
    return bf16(t / smooth.to(torch.float32)[None, :])


def quantize_act_int4(
    x: torch.Tensor,
    smooth: torch.Tensor | None = None,
    unsigned: bool = False,
    shift: float = 0.0,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-64-group INT4 activation quantizer.

    Restates quantize_w4a4_from_fpsum_warp<use_unsigned> (gemm_w4a4.cuh:429-523) with IEEE fp32:
    ``amax`` over the group in bf16, ``s = f32(amax) * fl32(1/qmax)``, stored scale ``bf16(s)``,
    ``r = fl32(1/s)`` (the reference's ``rcp.approx.ftz`` is replaced by the exact reciprocal),
    ``code = sat(rne(f32(y) * r))`` (cvt.rni + cvt.pack.sat, gemm_utils.cuh:209-227).
    A group whose ``amax`` is zero yields codes 0 and scale 0.

    x: bf16 ``[M, K]`` (K a multiple of 64); smooth: bf16 ``[K]`` or None.
    Returns (codes int8 ``[M, K]`` in [-8, 7] or [0, 15], scales bf16 ``[K/64, M]``).
    """
    M, K = x.shape
    assert K % INT4_GROUP == 0
    y = _smooth_divide(x, smooth, shift).reshape(M, K // INT4_GROUP, INT4_GROUP)
    amax = y.abs().amax(dim=-1)  # exact: the maximum of bf16 values is a bf16 value
    recip = torch.tensor(float(RECIP_15 if unsigned else RECIP_7), dtype=torch.float32)
    s = amax * recip  # fp32 product, one rounding
    scales = s.to(torch.bfloat16)
    r = torch.tensor(1.0, dtype=torch.float32) / s  # IEEE reciprocal; inf where s == 0
    q = torch.round(y * r[..., None])  # fp32 product then round-half-even
    q = torch.where(s[..., None] == 0, torch.zeros_like(q), q)
    lo, hi = (0, 15) if unsigned else (-8, 7)
    codes = q.clamp_(lo, hi).to(torch.int8).reshape(M, K)
    return codes, scales.t().contiguous()


def e2m1_encode(v: torch.Tensor) -> torch.Tensor:
    """fp32 -> 4-bit E2M1 pattern, round-to-nearest-even, saturating (cvt.rn.satfinite.e2m1x2,
    gemm_utils.cuh:239-245).  Ties go to the pattern with an even low bit."""
    a = v.abs()
    grid = torch.tensor(E2M1_VALUES, dtype=torch.float32)
    mids = (grid[1:] + grid[:-1]) * 0.5  # 0.25 .75 1.25 1.75 2.5 3.5 5
    code = torch.zeros(a.shape, dtype=torch.int64)
    for i, m in enumerate(mids.tolist()):
        up = i + 1  # pattern just above midpoint i
        # strictly above the midpoint -> round up; exactly on it -> up only if `up` is even
        take = (a > m) | ((a == m) & (up % 2 == 0))
        code = torch.where(take, torch.full_like(code, up), code)
    sign = (torch.signbit(v) & (code >= 0)).to(torch.int64)
    return (code | (sign << 3)).to(torch.uint8)


def e2m1_decode(code: torch.Tensor) -> torch.Tensor:
    grid = torch.tensor(E2M1_VALUES, dtype=torch.float32)
    mag = grid[(code.to(torch.int64) & 7)]
    return torch.where((code.to(torch.int64) & 8) != 0, -mag, mag)


def quantize_act_nvfp4(x: torch.Tensor, smooth: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-16-group NVFP4 activation quantizer (quantize_w4a4_fp4_from_fpsum_warp,
    gemm_w4a4.cuh:85-187): ``s = min(f32(amax) * fl32(1/6), 448)``, stored scale
    ``e4m3_rn(s)``, codes from the *unrounded* s: ``e2m1_rn_sat(f32(y) * fl32(1/s))``.
    Zero groups give codes 0 / scale 0.

    Returns (codes uint8 ``[M, K]`` holding 4-bit E2M1 patterns, scales float8_e4m3fn ``[K/16, M]``).
    """
    M, K = x.shape
    assert K % NVFP4_GROUP == 0
    y = _smooth_divide(x, smooth, 0.0).reshape(M, K // NVFP4_GROUP, NVFP4_GROUP)
    amax = y.abs().amax(dim=-1)
    s = torch.minimum(amax * torch.tensor(float(RECIP_6), dtype=torch.float32), torch.tensor(448.0))
    scales = s.to(torch.float8_e4m3fn)
    r = torch.tensor(1.0, dtype=torch.float32) / s
    v = y * r[..., None]
    v = torch.where(s[..., None] == 0, torch.zeros_like(v), v)
    codes = e2m1_encode(v).reshape(M, K)
    return codes, scales.t().contiguous()


# ---------------------------------------------------------------------------------------------
# Weight-side synthetic quantizers.  The offline weight quantizer is not part of the reference
# tree; these only manufacture self-consistent (codes, scales) pairs for tests and the bench.
# ---------------------------------------------------------------------------------------------


def quantize_weight_int4(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-(row, 64-group) absmax INT4: ``ws = bf16(absmax / 7)``, ``wq = clamp(rne(w / ws), -7, 7)``.
    Returns (codes int8 ``[N, K]``, scales bf16 ``[K/64, N]``)."""
    N, K = w.shape
    g = w.to(torch.float32).reshape(N, K // INT4_GROUP, INT4_GROUP)
    ws = (g.abs().amax(dim=-1) / 7.0).to(torch.bfloat16)
    wsf = ws.to(torch.float32)
    q = torch.round(g / torch.where(wsf == 0, torch.ones_like(wsf), wsf)[..., None]).clamp_(-7, 7)
    return q.to(torch.int8).reshape(N, K), ws.t().contiguous()


def quantize_weight_nvfp4(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, float]:
    """Per-(row, 16-group) NVFP4 with a per-tensor fp32 scale chosen so group scales fit E4M3.
    Returns (E2M1 patterns uint8 ``[N, K]``, scales float8_e4m3fn ``[K/16, N]``, wtscale)."""
    N, K = w.shape
    g = w.to(torch.float32).reshape(N, K // NVFP4_GROUP, NVFP4_GROUP)
    amax = g.abs().amax(dim=-1)
    wt = float(amax.max() / 6.0 / 448.0)
    wt = wt if wt > 0 else 1.0
    ws = (amax / 6.0 / wt).clamp_(max=448.0).to(torch.float8_e4m3fn)
    wsf = ws.to(torch.float32) * wt
    v = g / torch.where(wsf == 0, torch.ones_like(wsf), wsf)[..., None]
    return e2m1_encode(v).reshape(N, K), ws.t().contiguous(), wt


# ---------------------------------------------------------------------------------------------
# Dequantizers and nibble packing (logical order: element 2b in the low nibble of byte b).
# ---------------------------------------------------------------------------------------------


def dequant_int4(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """codes ``[R, K]`` (any integer dtype), scales ``[K/64, R]`` -> fp32 ``[R, K]``."""
    R, K = codes.shape
    s = scales.to(torch.float32).t()  # [R, K/64]
    return (codes.to(torch.float32).reshape(R, K // INT4_GROUP, INT4_GROUP) * s[..., None]).reshape(R, K)


def dequant_nvfp4(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """E2M1 patterns ``[R, K]``, E4M3 scales ``[K/16, R]`` -> fp32 ``[R, K]`` (stored scale is used,
    as the GEMM does: gemm_w4a4.cuh:191-250)."""
    R, K = codes.shape
    s = scales.to(torch.float32).t()
    return (e2m1_decode(codes).reshape(R, K // NVFP4_GROUP, NVFP4_GROUP) * s[..., None]).reshape(R, K)


def pack_nibbles(codes: torch.Tensor) -> torch.Tensor:
    """``[R, K]`` 4-bit values (two's complement nibble for negatives) -> uint8 ``[R, K/2]``."""
    c = codes.to(torch.int16) & 0xF
    return (c[:, 0::2] | (c[:, 1::2] << 4)).to(torch.uint8)


def unpack_nibbles(packed: torch.Tensor, signed: bool) -> torch.Tensor:
    p = packed.to(torch.int16)
    lo, hi = p & 0xF, (p >> 4) & 0xF
    out = torch.stack([lo, hi], dim=-1).reshape(packed.shape[0], -1)
    if signed:
        out = torch.where(out >= 8, out - 16, out)
    return out.to(torch.int8)
