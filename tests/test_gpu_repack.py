"""Load-time repack on the GPU against the oracle's statement of the reference layouts, including
the golden bytes written by the reference packer."""

from pathlib import Path

import numpy as np
import pytest
import torch

from conftest import announce
from oracle import layouts as L

pytestmark = pytest.mark.gpu
GOLD = Path(__file__).parent / "golden" / "packer_vectors.npz"


def _bf16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_repack_golden_vectors(dev):
    from nunchaku_amd import packing

    z = np.load(GOLD)
    announce("repack golden qweight/wscales/vector/lora N=K=256 R=32")
    qn = packing.repack_qweight(torch.from_numpy(z["qweight"]).to(dev))
    N, K = z["codes"].shape
    # E2M3 fragments of code / 8, decoded back to one code per element
    assert torch.equal(packing.qweight_to_logical(qn).cpu(), torch.from_numpy(z["codes"]))

    ws = packing.repack_wscales(_bf16(z["wscales_packed"]).to(dev))
    logical = _bf16(z["wscales_logical"]).float()
    assert torch.equal(packing.wscales_to_logical(ws, N), logical)  # the factor 4 is a power of two: exact

    v = packing.repack_vector(_bf16(z["vec_packed"].reshape(-1)).to(dev))
    assert torch.equal(v.cpu().view(torch.int16), _bf16(z["vec_logical"]).view(torch.int16))

    r = packing.repack_smooth(_bf16(z["vec_packed"].reshape(-1)).to(dev))
    want = (1.0 / _bf16(z["vec_logical"]).float())
    assert torch.equal(r.cpu(), want)

    up = packing.repack_lora_up(_bf16(z["up_packed"]).to(dev))
    assert torch.equal(up.cpu().view(torch.int16), _bf16(z["up_logical"]).view(torch.int16))

    dn = packing.repack_lora_down(_bf16(z["down_packed"]).to(dev)).cpu().view(torch.int16)
    logical = _bf16(z["down_logical"]).view(torch.int16)  # [K, R]
    R = logical.shape[1]
    dn = dn.reshape(K // 128, 4, R // 16, 64, 8)
    c, i, rt, lane, j = np.meshgrid(np.arange(K // 128), np.arange(4), np.arange(R // 16), np.arange(64), np.arange(8), indexing="ij")
    k = 128 * c + 32 * (lane // 16) + 8 * i + j
    rk = 16 * rt + lane % 16
    assert torch.equal(dn, logical[torch.from_numpy(k), torch.from_numpy(rk)])


def test_repack_micro_scales(dev):
    from nunchaku_amd import packing

    z = np.load(GOLD)
    announce("repack golden nvfp4 micro scales")
    src = torch.from_numpy(z["mscales_packed"]).view(torch.float8_e4m3fn).to(dev)
    ws = packing.repack_wscales(src, fp4=True)
    logical = torch.from_numpy(z["mscales_logical"]).view(torch.float8_e4m3fn).float()
    G16, N = logical.shape
    got = ws.float().cpu().reshape(G16 // 4, N, 4).permute(0, 2, 1).reshape(G16, N)  # [K/64][N][4] -> [K/16][N]
    assert torch.equal(got * ws.colnorm.cpu()[None, :], logical)


def test_repack_random_larger(dev):
    from nunchaku_amd import packing

    rng = np.random.default_rng(5)
    N, K = 384, 640
    announce(f"repack random N={N} K={K}")
    codes = rng.integers(-8, 8, (N, K)).astype(np.int8)
    qn = packing.repack_qweight(torch.from_numpy(L.pack_qweight(codes)).to(dev))
    assert torch.equal(packing.qweight_to_logical(qn).cpu(), torch.from_numpy(codes))
    assert qn.shape == (512, K * 3 // 4), "N = 384 is padded to two blocks of 256 columns"
    pad = packing._fragments_to_logical(qn, 512, K, 256)[N:]
    assert (pad == 0).all(), "columns beyond N must hold zero codes"
    ws = rng.random((K // 64, N)).astype(np.float32) + 0.01
    wsb = torch.from_numpy(ws).to(torch.bfloat16)
    wn = packing.repack_wscales(torch.from_numpy(L.pack_wscales(wsb.view(torch.int16).numpy().view(np.uint16)).view(np.int16).copy()).view(torch.bfloat16).to(dev))
    assert torch.equal(packing.wscales_to_logical(wn, N), wsb.float())
    assert (wn.cpu()[1, :, 128:] == 0).all(), "scales of the columns beyond N must be zero"
    pat = rng.integers(0, 16, (N, K)).astype(np.int8)
    qf = packing.repack_qweight(torch.from_numpy(L.pack_qweight(pat)).to(dev), fp4=True)
    assert torch.equal(packing.act_to_logical(qf.view(torch.uint8).cpu(), K, fp4=True), torch.from_numpy(pat))
