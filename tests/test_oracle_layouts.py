"""Pins oracle/layouts.py: golden bytes written by the reference's own packer
(tests/golden/packer_vectors.npz, made by tests/golden/make_packer_vectors.py), agreement of the two
independent derivations, and the lane tables printed in the reference's comments."""

from pathlib import Path

import numpy as np
import pytest

from oracle import layouts as L

GOLD = Path(__file__).parent / "golden" / "packer_vectors.npz"


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


def test_golden_qweight(gold):
    assert np.array_equal(L.pack_qweight(gold["codes"]), gold["qweight"])
    assert np.array_equal(L.unpack_qweight(gold["qweight"]), gold["codes"])


def test_golden_wscales_and_vector(gold):
    assert np.array_equal(L.pack_wscales(gold["wscales_logical"]), gold["wscales_packed"])
    assert np.array_equal(L.unpack_wscales(gold["wscales_packed"]), gold["wscales_logical"])
    assert np.array_equal(L.pack_vector(gold["vec_logical"]), gold["vec_packed"].reshape(-1))
    assert np.array_equal(L.unpack_vector(gold["vec_packed"].reshape(-1)), gold["vec_logical"])


def test_golden_micro_scales(gold):
    assert np.array_equal(L.pack_wmscales(gold["mscales_logical"]), gold["mscales_packed"])
    assert np.array_equal(L.unpack_wmscales(gold["mscales_packed"]), gold["mscales_logical"])


def test_golden_lowrank(gold):
    assert np.array_equal(L.pack_lora(gold["down_logical"], True), gold["down_packed"])
    assert np.array_equal(L.pack_lora(gold["up_logical"], False), gold["up_packed"])
    assert np.array_equal(L.unpack_lora(gold["down_packed"], True), gold["down_logical"])
    assert np.array_equal(L.unpack_lora(gold["up_packed"], False), gold["up_logical"])


@pytest.mark.parametrize("N,K", [(128, 128), (256, 384), (384, 128)])
def test_two_derivations_agree(N, K):
    rng = np.random.default_rng(N * 1000 + K)
    codes = rng.integers(-8, 8, (N, K))
    assert np.array_equal(L.unpack_qweight(L.pack_qweight(codes)), codes)
    s = rng.integers(0, 65536, (K // 64, N)).astype(np.uint16)
    assert np.array_equal(L.unpack_wscales(L.pack_wscales(s)), s)
    m = rng.integers(0, 256, (K // 16, N)).astype(np.uint8)
    assert np.array_equal(L.unpack_wmscales(L.pack_wmscales(m)), m)
    for down in (True, False):
        w = rng.integers(0, 65536, (K if down else N, 32)).astype(np.uint16)
        assert np.array_equal(L.unpack_lora(L.pack_lora(w, down), down), w)


def test_lane_tables_from_reference_comments():
    # nunchaku/lora/flux/packer.py:286-298: scale store order "0 1 8 9 / 2 3 10 11 / ... / 118 119 126 127"
    v = L.pack_vector(np.arange(128, dtype=np.uint16))
    assert v[:4].tolist() == [0, 1, 8, 9]
    assert v[4:8].tolist() == [2, 3, 10, 11]
    assert v[16:20].tolist() == [16, 17, 24, 25]
    assert v[28:32].tolist() == [22, 23, 30, 31]
    assert v[112:116].tolist() == [112, 113, 120, 121]
    assert v[124:128].tolist() == [118, 119, 126, 127]
    # packer.py:346-357: micro scale store order "0 32 64 96 / 8 40 72 104 / ... / 31 63 95 127"
    m = L.pack_wmscales(np.tile(np.arange(128, dtype=np.uint8)[None, :], (4, 1))).reshape(-1)
    words = m.reshape(-1, 4)[:, 0].reshape(32, 4)  # lane x word, first byte of each word
    assert words[0].tolist() == [0, 32, 64, 96]
    assert words[1].tolist() == [8, 40, 72, 104]
    assert words[3].tolist() == [24, 56, 88, 120]
    assert words[4].tolist() == [1, 33, 65, 97]
    assert words[28].tolist() == [7, 39, 71, 103]
    assert words[31].tolist() == [31, 63, 95, 127]


def test_qweight_first_words_by_hand():
    # lane 0 of tile 0 holds row 0, columns 0..7 in its first word (mma.m16n8k64 B fragment,
    # src/kernels/zgemm/gemm_base.cuh:278-294); second word: columns 32..39; third: row 8
    codes = np.zeros((128, 128), dtype=np.int64)
    codes[0, :8] = np.arange(8)
    codes[0, 32:40] = 7
    codes[8, :8] = 3
    w = L.pack_qweight(codes).reshape(-1).view(np.uint32)
    assert w[0] == 0x76543210 and w[1] == 0x77777777 and w[2] == 0x33333333 and w[3] == 0


def test_rotemb_two_derivations_agree():
    """The permute recipe of pack_rotemb (embeddings.py:88-120) against the closed form read off the
    kernel's loader (epilogues.cuh:282-305,383-401), and pack / unpack as inverses."""
    rng = np.random.default_rng(0)
    for M, D in ((16, 8), (32, 128), (48, 64)):
        logical = rng.standard_normal((M, D)).astype(np.float32)
        packed = L.pack_rotemb(logical)
        row, col = L.rotemb_index(M, D)
        assert np.array_equal(packed.reshape(-1), logical[row, col])
        assert np.array_equal(L.unpack_rotemb(packed), logical)


def test_rotemb_known_positions():
    """Hand-evaluated positions of the m16n8 fp32 accumulator fragment (the table named in
    embeddings.py:109-113): thread 4g+t holds c0,c1 = row g, columns 2t, 2t+1 and c2,c3 = row g+8."""
    M, D = 16, 8
    logical = (np.arange(M)[:, None] * 100 + np.arange(D)[None, :]).astype(np.float32)
    packed = L.pack_rotemb(logical).reshape(-1)
    # lane 0: rows 0 and 8, columns 0, 1
    assert packed[0:4].tolist() == [0.0, 1.0, 800.0, 801.0]
    # lane 5 = (g 1, t 1): rows 1 and 9, columns 2, 3
    assert packed[20:24].tolist() == [102.0, 103.0, 902.0, 903.0]
    # lane 31 = (g 7, t 3): rows 7 and 15, columns 6, 7
    assert packed[124:128].tolist() == [706.0, 707.0, 1506.0, 1507.0]
