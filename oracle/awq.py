"""CPU restatement of the AWQ W4A16 GEMV path (AWQW4A16Linear, nunchaku/models/linear.py:138-208 ->
awq_gemv_w4a16_cuda, nunchaku/ops/gemv.py -> gemv_kernel, src/kernels/awq/gemv_awq.cu:84-215).

Test infrastructure only (see ``oracle/__init__.py``).

Weight storage, two independent statements:

* ``pack_w4``   follows the reshape/permute recipe of the reference's packer
  (nunchaku/models/text_encoders/tinychat_utils.py:76-106).
* ``w4_index``  is read off the kernel: which thread loads which 16 bytes (gemv_awq.cu:137-158), the
  nibble order of ``dequantize_s4_to_fp16x2`` (src/kernels/awq/dequantize.cuh:18-74: outputs 2p, 2p+1
  of a 32-bit word are its nibbles p and p + 4) and the shuffle that follows (gemv_awq.cu:168-180).

Arithmetic: ``w = bf16(code * scale + zero)`` (one rounding: ``__hfma2``, gemv_awq.cu:176; ``zero`` is the
stored tensor, i.e. minus the scaled zero point, tinychat_utils.py:187), ``out[m, n] = sum_k w[n, k] x[m, k]``
accumulated in fp32.  The reference rounds every product to bf16 first (``__hmul2``, gemv_awq.cu:197);
that is a loss of the reference's, not part of the definition: ``round_products=True`` reproduces it to
size the difference.  Parity status: the storage order and the scale / zero convention are pinned by golden vectors
written by the reference's own ``pack_w4`` and ``convert_to_tinychat_w4x16y16_linear_weight``
(tests/golden/awq_vectors.npz) and by the two derivations, the arithmetic by the library matmul; the reference holds
no output fixture of the GEMV kernel itself.
"""

from __future__ import annotations

import numpy as np
import torch


def pack_w4(codes: np.ndarray) -> np.ndarray:
    """tinychat_utils.py:76-106.  ``codes``: integers in [0, 15], shape [OC, IC], IC % 64 == 0, OC % 4 == 0.
    Returns int16 [OC/4, IC] (the module views it as int32 [OC/4, IC/2])."""
    oc, ic = codes.shape
    assert oc % 4 == 0 and ic % 64 == 0
    w = codes.astype(np.int64).reshape(-1, 4, 8)
    w = w[:, 0] | (w[:, 1] << 4) | (w[:, 2] << 8) | (w[:, 3] << 12)        # 32 codes -> 8 words of 16 bits
    w = w.reshape(oc // 4, 4, ic // 64, 16).transpose(0, 2, 1, 3).reshape(oc // 4, ic)
    return w.astype(np.uint16).view(np.int16)


def w4_index(oc: int, ic: int):
    """For every stored nibble, in storage order (32-bit words, nibble e in bits [4e, 4e+4)), its logical
    (n, k).  A 4-row group is ic/64 blocks of 128 bytes; thread slot u = 0..7 of a block (16 bytes) holds
    row (u / 2) and the 32 input channels 64 * block + 32 * (u % 2) + [0, 32) (gemv_awq.cu:137-141); word
    i2 of the 16 bytes, nibble p + 4 b, is channel 8 p + 2 i2 + b of those 32 (dequantize.cuh and the
    shuffle, gemv_awq.cu:168-180)."""
    g, blk, u, i2, nib = np.meshgrid(np.arange(oc // 4), np.arange(ic // 64), np.arange(8), np.arange(4), np.arange(8), indexing="ij")
    p, b = nib % 4, nib // 4
    n = 4 * g + u // 2
    k = 64 * blk + 32 * (u % 2) + 8 * p + 2 * i2 + b
    return n.reshape(-1), k.reshape(-1)


def unpack_w4(stored: np.ndarray) -> np.ndarray:
    """Inverse of :func:`pack_w4` through the closed form.  ``stored``: int16 [OC/4, IC] (or int32 [OC/4, IC/2])."""
    raw = np.ascontiguousarray(stored).view(np.uint8).reshape(-1)
    oc4 = stored.shape[0]
    ic = raw.size * 2 // (oc4 * 4)
    nibbles = np.stack((raw & 15, raw >> 4), axis=-1).reshape(-1)  # little endian: byte i holds nibbles 2i, 2i+1
    n, k = w4_index(oc4 * 4, ic)
    out = np.empty((oc4 * 4, ic), dtype=np.int64)
    out[n, k] = nibbles
    return out


def dequant(codes: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, group_size: int = 64) -> torch.Tensor:
    """bf16(code * scale + zero), one rounding (gemv_awq.cu:176).  codes int [OC, IC]; scales, zeros bf16
    [IC/G, OC] (the module's layout).  Returns bf16 [OC, IC]."""
    s = scales.t().to(torch.float64).repeat_interleave(group_size, dim=1)
    z = zeros.t().to(torch.float64).repeat_interleave(group_size, dim=1)
    return (codes.to(torch.float64) * s + z).to(torch.bfloat16)  # the fp64 sum is exact: one rounding


def gemv(x: torch.Tensor, codes: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, group_size: int = 64,
         round_products: bool = False) -> torch.Tensor:
    """x bf16 [M, IC] -> fp32 [M, OC]."""
    w = dequant(codes, scales, zeros, group_size)
    if round_products:
        prod = (x.float()[:, None, :] * w.float()[None, :, :]).to(torch.bfloat16)
        return prod.to(torch.float64).sum(-1).float()
    return (x.to(torch.float64) @ w.to(torch.float64).t()).float()


def make_layer(oc: int, ic: int, seed: int, group_size: int = 64):
    """Synthetic AWQ layer the way convert_to_tinychat_w4x16y16_linear_weight (tinychat_utils.py:109-189) builds
    one: asymmetric per-group quantization of N(0, 0.02) weights.  Returns (codes int [OC, IC], scales bf16
    [IC/G, OC], zeros bf16 [IC/G, OC] = -(zero point * scale), bias bf16 [OC])."""
    g = torch.Generator().manual_seed(seed)
    w = 0.02 * torch.randn(oc, ic, generator=g)
    wg = w.view(oc, ic // group_size, group_size)
    lo, hi = wg.min(-1).values, wg.max(-1).values
    scale = ((hi - lo) / 15).clamp_min(1e-8).to(torch.bfloat16)
    zero = (-lo).to(torch.bfloat16)  # pre-scaled zero: w + zero >= 0
    codes = ((wg + zero.float()[..., None]) / scale.float()[..., None]).round().clamp(0, 15).to(torch.int32).view(oc, ic)
    bias = (0.02 * torch.randn(oc, generator=g)).to(torch.bfloat16)
    return codes, scale.t().contiguous(), (-zero).t().contiguous(), bias
