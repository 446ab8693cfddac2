"""Writes ``awq_vectors.npz``: small inputs and what the reference's own TinyChat packer
(nunchaku/models/text_encoders/tinychat_utils.py: ``pack_w4``, ``convert_to_tinychat_w4x16y16_linear_weight``)
makes of them.

Run once in the development container, where the reference tree is mounted:

    python tests/golden/make_awq_vectors.py /root/reference

The file is pure torch and is loaded by its path (the reference package itself cannot be imported here: its
``__init__`` needs libraries that are not installed); nothing of the reference is copied or stubbed.  Only the
resulting vectors (plain arrays) are committed; the tests read the ``.npz`` and never the reference.
"""

import importlib.util
import sys
from pathlib import Path

import numpy as np
import torch


def main():
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    spec = importlib.util.spec_from_file_location("tinychat_utils", ref / "nunchaku/models/text_encoders/tinychat_utils.py")
    tc = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(tc)

    g = torch.Generator().manual_seed(4321)
    oc, ic, gs = 16, 192, 64
    codes = torch.randint(0, 16, (oc, ic), generator=g, dtype=torch.int32)
    packed = tc.pack_w4(codes.clone())

    # a weight that quantizes exactly: (code - zero_point) * scale with scale a power of two, so that the converter's
    # round() has no ties to decide and its codes are known
    ng = ic // gs
    scale = torch.tensor([0.5, 0.25, 2.0]).repeat(oc, 1)[:, :ng] * (1 + torch.arange(oc).view(oc, 1) % 2)  # [oc, ng]
    zero_point = torch.randint(0, 16, (oc, ng), generator=g).float()
    w = ((codes.view(oc, ng, gs).float() - zero_point.view(oc, ng, 1)) * scale.view(oc, ng, 1)).view(oc, ic).to(torch.bfloat16)
    assert torch.equal(w.float(), ((codes.view(oc, ng, gs).float() - zero_point.view(oc, ng, 1)) * scale.view(oc, ng, 1)).view(oc, ic))
    # the converter quantizes (w + zero) / scale with zero in weight units: zero = zero_point * scale
    qweight, qscale, qzero = tc.convert_to_tinychat_w4x16y16_linear_weight(
        w.clone(), scale.to(torch.bfloat16), (zero_point * scale).to(torch.bfloat16), group_size=gs)

    out = Path(__file__).with_name("awq_vectors.npz")
    np.savez_compressed(
        out,
        codes=codes.numpy().astype(np.int8), packed=packed.numpy(),
        weight_bits=w.view(torch.int16).numpy(), scale_bits=scale.to(torch.bfloat16).view(torch.int16).numpy(),
        zero_point=zero_point.numpy().astype(np.int8),
        qweight=qweight.numpy(), qscale_bits=qscale.view(torch.int16).numpy(), qzero_bits=qzero.view(torch.int16).numpy(),
    )
    print(f"wrote {out}: packed {tuple(packed.shape)} {packed.dtype}, qweight {tuple(qweight.shape)}, qscale {tuple(qscale.shape)}, qzero {tuple(qzero.shape)}")


if __name__ == "__main__":
    main()
