"""Writes ``packer_vectors.npz``: small inputs and the bytes the reference's own
``NunchakuWeightPacker`` (nunchaku/lora/flux/packer.py) produces for them.

Run once in the development container, where the reference tree is mounted:

    python tests/golden/make_packer_vectors.py /root/reference

The reference package cannot be imported as a package here (its ``__init__`` needs libraries that
are not installed), so the three pure-torch files the packer consists of are loaded by file path
under their real module names; nothing of the reference is copied or stubbed.  Only the resulting
vectors (plain arrays) are committed; the tests read the ``.npz`` and never the reference.
"""

import importlib.util
import sys
import types
from pathlib import Path

import numpy as np
import torch


def _load(ref: Path):
    for name in ("nunchaku", "nunchaku.lora", "nunchaku.lora.flux"):
        mod = types.ModuleType(name)
        mod.__path__ = [str(ref / name.replace(".", "/"))]
        sys.modules[name] = mod
    for name in ("nunchaku.utils", "nunchaku.lora.flux.utils", "nunchaku.lora.flux.packer"):
        path = ref / (name.replace(".", "/") + ".py")
        spec = importlib.util.spec_from_file_location(name, path)
        mod = importlib.util.module_from_spec(spec)
        sys.modules[name] = mod
        spec.loader.exec_module(mod)
    return sys.modules["nunchaku.lora.flux.packer"]


def main():
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    packer_mod = _load(ref)
    packer = packer_mod.NunchakuWeightPacker(bits=4)
    g = torch.Generator().manual_seed(1234)
    N, K, R = 256, 256, 32

    codes = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int32)
    qweight = packer.pack_weight(codes.clone())

    wscales = torch.randn(N, K // 64, generator=g).to(torch.bfloat16)  # packer takes [N, groups]
    wscales_packed = packer.pack_scale(wscales.clone(), group_size=64)

    vec = torch.randn(N, generator=g).to(torch.bfloat16)
    vec_packed = packer.pack_scale(vec.clone().view(-1, 1), group_size=-1)

    mscales = (torch.rand(N, K // 16, generator=g) * 400).to(torch.bfloat16)
    mscales_packed = packer.pack_micro_scale(mscales.clone(), group_size=16)

    down = torch.randn(R, K, generator=g).to(torch.bfloat16)  # packer takes the down projection as [R, K]
    down_packed = packer.pack_lowrank_weight(down.clone(), down=True)
    up = torch.randn(N, R, generator=g).to(torch.bfloat16)
    up_packed = packer.pack_lowrank_weight(up.clone(), down=False)

    def u16(t):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)

    out = Path(__file__).with_name("packer_vectors.npz")
    np.savez_compressed(
        out,
        codes=codes.numpy().astype(np.int8),
        qweight=qweight.numpy(),
        wscales_logical=u16(wscales.t()),  # logical [groups, N]
        wscales_packed=u16(wscales_packed),
        vec_logical=u16(vec),
        vec_packed=u16(vec_packed),
        mscales_logical=mscales.t().contiguous().to(torch.float8_e4m3fn).view(torch.uint8).numpy(),
        mscales_packed=mscales_packed.contiguous().view(torch.uint8).numpy(),
        down_logical=u16(down.t()),  # logical [K, R]
        down_packed=u16(down_packed),
        up_logical=u16(up),
        up_packed=u16(up_packed),
    )
    print("wrote", out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
