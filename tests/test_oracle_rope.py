"""Pins oracle.linear.rmsnorm_rope: the RMS norm against the library routine, the rotation against
complex multiplication, the q / k / v split, and invariants a dropped term or a swapped sin / cos
would break."""

import torch

from oracle import linear as olin


def _table(M, seed):
    g = torch.Generator().manual_seed(seed)
    ang = torch.rand(M, 64, generator=g, dtype=torch.float64) * 6.283
    return torch.stack((torch.sin(ang), torch.cos(ang)), dim=-1).reshape(M, 128).float(), ang


def test_identity_rotation_is_library_rms_norm():
    M, N = 8, 768
    g = torch.Generator().manual_seed(1)
    x = torch.randn(M, N, generator=g)
    wq, wk = torch.randn(128, generator=g), torch.randn(128, generator=g)
    rot = torch.zeros(M, 128)
    rot[:, 1::2] = 1.0  # sin 0, cos 1
    got = olin.rmsnorm_rope(x, wq, wk, rot)
    want_q = torch.nn.functional.rms_norm(x[:, :256].double().reshape(M, 2, 128), (128,), wq.double(), 1e-6).reshape(M, 256)
    want_k = torch.nn.functional.rms_norm(x[:, 256:512].double().reshape(M, 2, 128), (128,), wk.double(), 1e-6).reshape(M, 256)
    assert torch.allclose(got[:, :256].double(), want_q, rtol=1e-6, atol=1e-6)
    assert torch.allclose(got[:, 256:512].double(), want_k, rtol=1e-6, atol=1e-6)
    assert torch.equal(got[:, 512:], x[:, 512:])  # v passes through


def test_rotation_is_complex_multiplication():
    M, N = 4, 384
    g = torch.Generator().manual_seed(2)
    x = torch.randn(M, N, generator=g)
    ones = torch.ones(128)
    rot, ang = _table(M, 3)
    got = olin.rmsnorm_rope(x, ones, ones, rot).double()
    for part in range(2):
        h = x[:, part * 128:(part + 1) * 128].double()
        h = h * torch.rsqrt((h * h).mean(dim=-1, keepdim=True) + 1e-6)
        z = torch.complex(h[:, 0::2], h[:, 1::2]) * torch.polar(torch.ones_like(ang), ang)
        want = torch.stack((z.real, z.imag), dim=-1).reshape(M, 128)
        assert torch.allclose(got[:, part * 128:(part + 1) * 128], want, rtol=1e-6, atol=1e-6)


def test_rotation_keeps_the_norm_and_quarter_turn_swaps():
    M, N = 4, 384
    x = torch.randn(M, N, generator=torch.Generator().manual_seed(4))
    ones = torch.ones(128)
    rot, _ = _table(M, 5)
    got = olin.rmsnorm_rope(x, ones, ones, rot)
    # after the norm every head has mean square 1 (up to eps); a rotation keeps it
    assert torch.allclose((got[:, :128] ** 2).mean(-1), torch.ones(M), atol=1e-4)
    quarter = torch.zeros(M, 128)
    quarter[:, 0::2] = 1.0  # sin 1, cos 0: (x, y) -> (-y, x)
    q = olin.rmsnorm_rope(x, ones, ones, quarter)
    base = olin.rmsnorm_rope(x, ones, ones, torch.stack((torch.zeros(M, 64), torch.ones(M, 64)), -1).reshape(M, 128))
    assert torch.allclose(q[:, 0:256:2], -base[:, 1:256:2], atol=1e-6)
    assert torch.allclose(q[:, 1:256:2], base[:, 0:256:2], atol=1e-6)


def test_pack_qkv_literal_answers():
    """Two heads, four rows, three tokens.  Which column goes to which tensor and head, the two roundings and
    the mask values are written out by hand."""
    from oracle import linear as olin

    out = torch.zeros(4, 768)
    out[0, 0] = 1.0            # q, head 0, dim 0
    out[0, 128 + 5] = 2.0      # q, head 1, dim 5
    out[1, 256 + 7] = 3.0      # k, head 0, dim 7
    out[2, 384 + 127] = -4.0   # k, head 1, dim 127
    out[2, 512] = 5.0          # v, head 0, dim 0
    out[0, 640 + 64] = 1.00390625   # v, head 1: 1 + 2^-8 is a bf16 tie, rounds to 1.0 although fp16 could hold it
    out[1, 640] = 70000.0      # bf16 70144, beyond fp16: +inf
    out[1, 1] = 2.0**-25       # the midpoint of the fp16 subnormals 0 and 2^-24: ties to even, 0 ...
    out[1, 2] = 1.5 * 2.0**-24  # ... and the midpoint of 2^-24 and 2 * 2^-24 goes to 2 * 2^-24
    out[3] = 9.0               # row 3 is padding
    q, k, v = olin.pack_qkv(out, attn_tokens=3)
    assert q.shape == k.shape == v.shape == (1, 2, 4, 128) and q.dtype == torch.float16
    assert q[0, 0, 0, 0] == 1.0 and q[0, 1, 0, 5] == 2.0 and q[0, 0, 0].abs().sum() == 1.0
    assert k[0, 0, 1, 7] == 3.0 and k[0, 1, 2, 127] == -4.0
    assert v[0, 0, 2, 0] == 5.0 and v[0, 1, 0, 64] == 1.0
    assert torch.isinf(v[0, 1, 1, 0]) and v[0, 1, 1, 0] > 0
    assert q[0, 0, 1, 1] == 0.0 and q[0, 0, 1, 2].item() == 2.0**-23
    assert (q[0, :, 3] == 0).all() and (v[0, :, 3] == 0).all() and torch.isnan(k[0, :, 3]).all()
    assert not torch.isnan(k[0, :, :3]).any()
