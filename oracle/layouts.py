"""Reference checkpoint layouts of the W4A4 path: logical tensor <-> the byte order the reference
stores (and its CUDA kernels load).  Test infrastructure only (see ``oracle/__init__.py``).

Two independent statements of every layout are kept on purpose:

* ``pack_*``   follow the reshape/permute recipe of ``NunchakuWeightPacker``
  (nunchaku/lora/flux/packer.py:187-398), written with numpy axes.
* ``*_index``  are closed forms read off the CUDA loaders (which lane of a 32-lane warp loads which
  element: src/kernels/zgemm/gemm_base.cuh:100-112,265-340,474-489, lora.cuh:43-59,
  gemm_w4a4.cuh:46-83).  They give, for every *stored* position, the logical coordinates.

``tests/test_oracle_layouts.py`` checks that both agree, that the lane tables printed in the
reference's comments come out, and that the golden bytes written by the reference packer match.

Shapes: N out-features (multiple of 128), K in-features (multiple of 128), R rank (multiple of 16).
"""

from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------------------------
# qweight: 4-bit codes, logical int [N, K]  ->  stored int8 [N, K/2]
# --------------------------------------------------------------------------------------------


def pack_qweight(codes: np.ndarray) -> np.ndarray:
    """packer.py:187-239 (pack_weight, bits=4, warp_n=128).  ``codes``: integer array [N, K] with
    values in [-8, 15]; only the low 4 bits are kept."""
    N, K = codes.shape
    assert N % 128 == 0 and K % 128 == 0
    c = (codes.astype(np.int64) & 0xF).reshape(N // 128, 8, 2, 8, 1, K // 64, 1, 2, 4, 8)
    # axes: n_tile, n_pack, n_pack_size, n_lane, reg_n, k_tile, k_pack, k_pack_size, k_lane, reg_k
    c = c.transpose(0, 5, 6, 1, 3, 8, 2, 7, 4, 9)
    words = (c << (4 * np.arange(8, dtype=np.int64))).sum(axis=-1).astype(np.uint32)
    return np.ascontiguousarray(words).view(np.int8).reshape(N, K // 2)


def qweight_index(N: int, K: int):
    """For every stored nibble, in storage order, its logical (n, k).

    Storage = u32 words ``[N/128][K/64][j:8][lane:32][c:4]``, nibble e of a word in bits [4e,4e+4).
    With g = lane/4, t = lane%4 (gemm_base.cuh:278-294 + the mma.m16n8k64 B-fragment):
    n = 128*bn + 16*j + g + 8*(c>=2),  k = 64*kt + 32*(c odd) + 8*t + e.
    Returns (n_idx, k_idx), each int array of shape [N*K].
    """
    bn, kt, j, lane, c, e = np.meshgrid(
        np.arange(N // 128), np.arange(K // 64), np.arange(8), np.arange(32), np.arange(4), np.arange(8), indexing="ij"
    )
    g, t = lane // 4, lane % 4
    n = 128 * bn + 16 * j + g + 8 * (c >= 2)
    k = 64 * kt + 32 * (c % 2) + 8 * t + e
    return n.reshape(-1), k.reshape(-1)


def unpack_qweight(stored: np.ndarray, signed: bool = True) -> np.ndarray:
    """Inverse of :func:`pack_qweight` through the closed form.  Returns int8 [N, K]."""
    N, K2 = stored.shape
    K = K2 * 2
    b = stored.reshape(-1).view(np.uint8).astype(np.int16)
    nib = np.stack([b & 0xF, b >> 4], axis=-1).reshape(-1)
    n, k = qweight_index(N, K)
    out = np.zeros((N, K), dtype=np.int16)
    out[n, k] = nib
    if signed:
        out = np.where(out >= 8, out - 16, out)
    return out.astype(np.int8)


# --------------------------------------------------------------------------------------------
# per-channel vectors and per-group 16-bit scales: logical [G, N] -> stored [G, N]
# (bias, smooth_factor, wcscales are the G == 1 case, stored flat [N])
# --------------------------------------------------------------------------------------------


def pack_wscales(scales: np.ndarray) -> np.ndarray:
    """packer.py:241-301 (pack_scale, warp_n=128 -> s_pack_size 4, 32 lanes, 1 pack).
    ``scales``: logical [G, N] array of any 16-bit dtype (viewed as uint16)."""
    G, N = scales.shape
    assert N % 128 == 0
    s = np.ascontiguousarray(scales.T).reshape(N // 128, 1, 8, 2, 4, 2, G)
    s = s.transpose(0, 6, 1, 2, 4, 3, 5)
    return np.ascontiguousarray(s).reshape(G, N)


def wscales_index(G: int, N: int):
    """Stored order ``[N/128][G][lane:32][v:4]``; lane holds channels 16*(lane/4) + 2*(lane%4) +
    {0, 1, 8, 9} of its 128-block (gemm_base.cuh:100-112,474-489).  Returns (g_idx, n_idx)."""
    bn, g, lane, v = np.meshgrid(np.arange(N // 128), np.arange(G), np.arange(32), np.arange(4), indexing="ij")
    n = 128 * bn + 16 * (lane // 4) + 2 * (lane % 4) + (v % 2) + 8 * (v // 2)
    return g.reshape(-1), n.reshape(-1)


def unpack_wscales(stored: np.ndarray) -> np.ndarray:
    G, N = stored.shape
    g, n = wscales_index(G, N)
    out = np.zeros((G, N), dtype=stored.dtype)
    out[g, n] = stored.reshape(-1)
    return out


def pack_vector(vec: np.ndarray) -> np.ndarray:
    """bias / smooth_factor / wcscales: pack_scale with group_size=-1 (packer.py:301,
    nunchaku_converter.py:941-946)."""
    return pack_wscales(vec.reshape(1, -1)).reshape(-1)


def unpack_vector(stored: np.ndarray) -> np.ndarray:
    return unpack_wscales(stored.reshape(1, -1)).reshape(-1)


# --------------------------------------------------------------------------------------------
# NVFP4 micro-scales: logical fp8 [K/16, N] -> stored fp8 [K/16, N]
# --------------------------------------------------------------------------------------------


def pack_wmscales(scales: np.ndarray) -> np.ndarray:
    """packer.py:303-360 (pack_micro_scale).  ``scales``: logical [K/16, N] of a 1-byte dtype."""
    G, N = scales.shape
    assert N % 128 == 0 and G % 4 == 0
    s = np.ascontiguousarray(scales.T).reshape(N // 128, 1, 4, 4, 8, G // 4, 4)
    s = s.transpose(0, 5, 1, 4, 3, 2, 6)
    return np.ascontiguousarray(s).reshape(G, N)


def wmscales_index(G: int, N: int):
    """Stored order ``[N/128][K/64][lane:32][p:4][byte:4]``: word p of lane L is channel
    32*p + 8*(L%4) + L/4 of the 128-block, its 4 bytes the 4 groups of 16 inside the 64-wide k tile
    (gemm_w4a4.cuh:46-61,75-83).  Returns (g_idx, n_idx)."""
    bn, kt, lane, p, b = np.meshgrid(
        np.arange(N // 128), np.arange(G // 4), np.arange(32), np.arange(4), np.arange(4), indexing="ij"
    )
    n = 128 * bn + 32 * p + 8 * (lane % 4) + lane // 4
    g = 4 * kt + b
    return g.reshape(-1), n.reshape(-1)


def unpack_wmscales(stored: np.ndarray) -> np.ndarray:
    G, N = stored.shape
    g, n = wmscales_index(G, N)
    out = np.zeros((G, N), dtype=stored.dtype)
    out[g, n] = stored.reshape(-1)
    return out


# --------------------------------------------------------------------------------------------
# low-rank weights: proj_down logical [K, R] -> stored [K, R]; proj_up logical [N, R] -> stored [N, R]
# --------------------------------------------------------------------------------------------


def pack_lora(w: np.ndarray, down: bool) -> np.ndarray:
    """packer.py:362-398 (pack_lowrank_weight).  ``down``: w is the logical down projection given as
    [K, R] (the packer itself takes it transposed, [R, K]); else w is the up projection [N, R]."""
    C, R = w.shape
    assert C % 16 == 0 and R % 16 == 0
    if down:
        # packer input is [R, K]: view(r_packs,16,c_packs,16).permute(2,0,1,3)
        x = np.ascontiguousarray(w.T).reshape(R // 16, 16, C // 16, 16).transpose(2, 0, 1, 3)
    else:
        x = w.reshape(C // 16, 16, R // 16, 16).transpose(0, 2, 1, 3)
    # (c_packs, r_packs, pack_n, pack_k) -> split pack_n=(n_pack_size 2, n_lane 8, reg_n 1), pack_k=(2, 4, 2)
    x = np.ascontiguousarray(x).reshape(C // 16, R // 16, 2, 8, 1, 2, 4, 2)
    x = x.transpose(0, 1, 3, 6, 2, 5, 4, 7)
    return np.ascontiguousarray(x).reshape(C, R)


def lora_index(C: int, R: int, down: bool):
    """Stored order ``[C/16][R/16][lane:32][d:4][h:2]`` of 16-bit values (lora.cuh:43-59).
    down: channel = 16c + 2t + h + 8*(d odd), rank = 16r + g + 8*(d>=2);
    up:   channel = 16c + g + 8*(d>=2),       rank = 16r + 2t + h + 8*(d odd);  g=lane/4, t=lane%4.
    Returns (channel_idx, rank_idx)."""
    c, r, lane, d, h = np.meshgrid(
        np.arange(C // 16), np.arange(R // 16), np.arange(32), np.arange(4), np.arange(2), indexing="ij"
    )
    g, t = lane // 4, lane % 4
    if down:
        ch = 16 * c + 2 * t + h + 8 * (d % 2)
        rk = 16 * r + g + 8 * (d // 2)
    else:
        ch = 16 * c + g + 8 * (d // 2)
        rk = 16 * r + 2 * t + h + 8 * (d % 2)
    return ch.reshape(-1), rk.reshape(-1)


def unpack_lora(stored: np.ndarray, down: bool) -> np.ndarray:
    C, R = stored.shape
    ch, rk = lora_index(C, R, down)
    out = np.zeros((C, R), dtype=stored.dtype)
    out[ch, rk] = stored.reshape(-1)
    return out


# --------------------------------------------------------------------------------------------
# rotary table: logical fp32 [M, D] ((sin, cos) of pair i at [2i], [2i+1])  ->  packed fp32 [M, D]
# --------------------------------------------------------------------------------------------


def pack_rotemb(rotemb: np.ndarray) -> np.ndarray:
    """pack_rotemb, nunchaku/models/embeddings.py:88-120, for one batch entry: the reshape/permute
    recipe, written with numpy axes.  ``rotemb``: fp32 [M, D] with M % 16 == 0 and D % 8 == 0."""
    M, D = rotemb.shape
    assert M % 16 == 0 and D % 8 == 0
    r = rotemb.reshape(M // 16, 16, D // 8, 8).transpose(0, 2, 1, 3)      # [M/16][D/8][16 rows][8 floats]
    r = r.reshape(M // 16, D // 8, 2, 8, 4, 2).transpose(0, 1, 3, 4, 2, 5)  # rows -> (half, g), floats -> (t, s)
    return np.ascontiguousarray(r).reshape(M, D)


def rotemb_index(M: int, D: int):
    """For every stored float, in storage order, its logical (row, float index), read off the loader
    EpilogueRMSNormRope::load_rotemb and the use of the loaded float4 in ``apply``
    (src/kernels/zgemm/epilogues.cuh:282-305,383-401): storage = float4 ``[M/16][D/8][lane:32]``;
    lane = 4 g + t holds, for the m16n8 accumulator tile j of the head, (sin, cos) of rows g and
    g + 8 (float4 .xy and .zw) for the pair at columns 8 j + 2 t, 8 j + 2 t + 1."""
    mb, j, lane, half, s = np.meshgrid(np.arange(M // 16), np.arange(D // 8), np.arange(32), np.arange(2), np.arange(2), indexing="ij")
    g, t = lane // 4, lane % 4
    row = 16 * mb + g + 8 * half
    col = 8 * j + 2 * t + s
    return row.reshape(-1), col.reshape(-1)


def unpack_rotemb(stored: np.ndarray) -> np.ndarray:
    """Inverse of :func:`pack_rotemb` through the closed form."""
    M, D = stored.shape
    row, col = rotemb_index(M, D)
    out = np.empty_like(stored)
    out[row, col] = stored.reshape(-1)
    return out
