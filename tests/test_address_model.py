"""Host-side model of every global address the INT4 GEMM kernel and the quantize kernel form, checked against the sizes of
the buffers the operators are given (CPU only; nothing here touches a GPU).

The model restates the index arithmetic of ``csrc/gemm6_kernel.h`` (tile numbering, k-parts, the schedule of the
asynchronous copies with its look-ahead, parked partial sums, output stores) and of ``csrc/quantize.hip`` (the row buffer
whose size ends at the last valid row, code / scale / projection stores) for whole grids, over the shape distribution of
``tests/test_gpu_shape_sweep.py`` and of the randomized loop that once ended in a GPU fault (M = 100, K = 3072, N = 768,
rank 0, three k-parts among them).  It guards the arithmetic; the fault itself came from the compiler keeping a carry flag
alive across an inline-asm statement that overwrote it (``tests/test_build_guard.py`` checks the generated code for that).
"""

import random

import pytest

FRAG = 1536
BM, BN = 128, 256
SLOT_BYTES = 32 * 256 * 4 * 4


def choose_kparts(ntiles, kgroups, ncu=256):
    """csrc/gemm.hip::choose_kparts"""
    if ntiles > ncu:
        return 1
    best, best_t = 1, 0.55 * kgroups + 4.4
    for k in (2, 3, 4, 6, 8):
        units, g = ntiles * k, (kgroups + k - 1) // k
        if g < 12 or units > 2 * ncu:
            break
        shared = units > ncu
        t = g * (0.95 if shared else 0.55) + 4.4 + (11.5 if k == 4 else 5.3 + 2.6 * (k - 1)) * (1.5 if shared else 1.0)
        if t < (0.90 if best == 1 else 0.95) * best_t:
            best, best_t = k, t
    return best


def gemm6_grid(M_pad, N, K, k_split=0):
    mblocks, nblocks, kgroups = M_pad // BM, (N + BN - 1) // BN, K // 64
    ntiles = mblocks * nblocks
    kparts = min(k_split, kgroups) if k_split > 0 else choose_kparts(ntiles, kgroups)
    nbands = (mblocks + 9) // 10
    band = (mblocks + nbands - 1) // nbands
    return mblocks, nblocks, kgroups, ntiles, kparts, band


def check_gemm6(M_pad, N, K, M_out, N_out, k_split=0):
    mblocks, nblocks, kgroups, ntiles, kparts, BAND = gemm6_grid(M_pad, N, K, k_split)
    act_bytes = M_pad * K * 3 // 4
    wgt_bytes = nblocks * BN * K * 3 // 4
    wsc_bytes = nblocks * kgroups * 2048
    asc_bytes = kgroups * M_pad * 2
    part_bytes = ntiles * kparts * SLOT_BYTES if kparts > 1 else 0
    total = ntiles * kparts
    seen = {}
    for bid in range(total):
        v = (bid % 8) * (total // 8) + bid // 8 if total % 8 == 0 else bid
        assert 0 <= v < total
        tile, part = divmod(v, kparts)
        band = tile // (BAND * nblocks)
        in_band = tile - band * BAND * nblocks
        band_rows = min(mblocks - band * BAND, BAND)
        assert band_rows > 0
        mb, nb = band * BAND + in_band % band_rows, in_band // band_rows
        assert 0 <= mb < mblocks and 0 <= nb < nblocks, (tile, mb, nb)
        gb = kgroups * part // kparts
        ng = kgroups * (part + 1) // kparts - gb
        assert ng >= 1
        assert (mb, nb, part) not in seen
        seen[(mb, nb, part)] = True
        # the copy schedule: which k-groups get their weights (W) and the rest (R) requested
        w_req, r_req = [0], [0]
        if ng > 1:
            w_req.append(1)
            r_req.append(1)
        if ng > 2:
            w_req.append(2)
        l = 0
        while l + 3 < ng:  # MODE 2
            r_req.append(l + 2)
            w_req.append(l + 3)
            l += 1
        if l + 2 < ng:  # MODE 1
            r_req.append(l + 2)
            l += 1
        assert w_req == list(range(ng)) and r_req == list(range(ng)), (ng, w_req, r_req)
        for wave in range(4):
            for g in range(ng):
                # three 1 KB weight chunks, 16 bytes per lane
                src_w = (nb * kgroups + gb + g) * 8 * FRAG + wave * 3072
                assert src_w + 2048 + 63 * 16 + 16 <= wgt_bytes
                src_a = (mb * kgroups + gb + g) * 4 * FRAG + wave * 1024
                assert src_a + 63 * 16 + 16 <= act_bytes
                if wave < 2:
                    src_x = (mb * kgroups + gb + g) * 4 * FRAG + (4 + wave) * 1024
                    assert src_x + 63 * 16 + 16 <= act_bytes
                else:
                    src_x = (nb * kgroups + gb + g) * 2048 + (wave - 2) * 1024
                    assert src_x + 63 * 16 + 16 <= wsc_bytes
                src_q = ((gb + g) * M_pad + mb * BM) * 2
                assert src_q + 63 * 4 + 4 <= asc_bytes
        if kparts > 1:
            slot = (tile * kparts + part) * SLOT_BYTES
            assert slot + ((7 * 4 + 3) * 256 + 255) * 16 + 16 <= part_bytes
            assert tile * 4 + 4 <= ntiles * 4  # arrival counter
        # output stores: rows below M_out, 16-byte pieces below N_out
        for wm in range(2):
            for wn in range(2):
                for mt in range(2):
                    for rr in (0, 31):
                        for cc in (0, 120):
                            m, n = mb * BM + wm * 64 + mt * 32 + rr, nb * BN + wn * 128 + cc
                            if m < M_out and n < N_out:
                                assert (m * N_out + n) * 2 + 16 <= M_out * N_out * 2
    assert len(seen) == total
    return kparts


def sweep_shapes():
    """The distribution of the seeded sweep and of the randomized loop (test_gpu_shape_sweep.py), INT4 cases."""
    shapes = {(100, 3072, 768, 0), (100, 3072, 768, 3)}
    for seed in (1, 2, 3):
        rng = random.Random(seed)
        for _ in range(400):
            fp4 = rng.random() < 0.3
            M = rng.choice([1, 17, 100, 255, 256, 257, 300, 511, 640, 900, 1300])
            K = 128 * rng.randint(1, 9) if rng.random() < 0.7 else rng.choice([2048, 3072, 4096, 6144])
            N = 128 * rng.randint(1, 11)
            rng.choice([0, 16, 32, 32, 48, 64, 96, 128])
            rng.random(), rng.random(), rng.choice([1.0, 1.0, 0.5, 1.7]) if not fp4 else None, rng.random()
            ks = rng.choice([None, None, None, 1, 2, 3, 5]) if not fp4 else rng.choice([None, None, 1, 2])
            if not fp4:
                shapes.add((M, K, N, ks or 0))
    return sorted(shapes)


def test_gemm6_addresses_stay_inside_their_buffers():
    shapes = sweep_shapes()
    assert (100, 3072, 768, 0) in shapes
    for M, K, N, ks in shapes:
        M_pad = (M + 255) // 256 * 256
        check_gemm6(M_pad, N, K, M, N, ks)
    # the case that faulted: six tiles, by the library's own choice split in three parts then and in four now
    assert check_gemm6(256, 768, 3072, 100, 768, 0) == 4
    assert check_gemm6(256, 768, 3072, 100, 768, 3) == 3


def test_gemm6_addresses_large_shapes():
    for M_pad, N, K in ((4608, 12288, 3072), (4608, 3072, 12288), (4608, 9216, 3072), (256, 3072, 3072)):
        check_gemm6(M_pad, N, K, M_pad, N, 0)


@pytest.mark.parametrize("glu", [False, True])
def test_quantize_row_buffer_cuts_exactly_at_the_last_row(glu):
    """The kernel reads x through a raw buffer whose size (num_records) ends with the workgroup's last valid row, and
    carries the 128-column chunk in the scalar offset.  The hardware's range check for a raw buffer compares the lane
    offset plus the access size with num_records and ignores the scalar offset, so a lane reads memory if and only
    if its row is valid (and the chunk exists: past the last chunk the kernel sets bit 31 of the lane offset)."""
    XW = 2 if glu else 1
    PPR, RPI = 16 * XW, 64 // (16 * XW)
    for K in (128, 256, 1152, 3072, 12288):
        ld = XW * K
        nchunks = K // 128
        for MT in (1, 2):
            for rows_valid in (0, 1, 5, 15, 16, 17, 31, 32):
                rv = min(rows_valid, 16 * MT)
                num_records = rv * ld * 2
                for c in (0, nchunks - 1, nchunks, nchunks + 3):
                    beyond = 0 if c < nchunks else 0x80000000
                    soffset = c * 256 * XW
                    for mt in range(MT):
                        for i in range(4 * XW):
                            for lane in range(64):
                                row = 16 * mt + RPI * i + lane // PPR
                                voff = ((lane // PPR) * ld * 2 + (lane % PPR) * 16) | beyond
                                voff += (16 * mt + RPI * i) * ld * 2
                                in_range = voff + 16 <= num_records
                                assert in_range == (row < rv and c < nchunks), (K, MT, rows_valid, c, mt, i, lane)
                                if in_range:  # the bytes a lane in range touches belong to its row and chunk
                                    first = voff + soffset
                                    assert row * ld * 2 + c * 256 * XW <= first and first + 16 <= row * ld * 2 + (c + 1) * 256 * XW


def test_quantize_store_addresses():
    for M, K, R in ((1, 128, 0), (100, 3072, 32), (257, 1152, 160), (300, 256, 1024), (4608, 3072, 32)):
        M_pad = (M + 255) // 256 * 256
        kgroups = K // 64
        act_bytes, asc_elems, lora_elems = M_pad * K * 3 // 4, kgroups * M_pad, M_pad * R
        for row in (0, 31, 127, 128, M_pad - 1):
            for c in (0, K // 128 - 1):
                for q in range(4):
                    g = 2 * c + (q >> 1)
                    frag = ((row // 128 * kgroups + g) * 4 + (row % 128) // 32) * FRAG
                    slot = row % 32 + 32 * (q & 1)
                    assert frag + slot * 16 + 16 <= act_bytes and frag + 1024 + slot * 8 + 8 <= act_bytes
                    assert g * M_pad + row < asc_elems
            if R:
                for rt_base in range(0, R // 16, 8):
                    rts = min(R // 16 - rt_base, 8)
                    for rank in (0, 16 * rts - 1):
                        assert row * R + 16 * rt_base + rank < lora_elems
