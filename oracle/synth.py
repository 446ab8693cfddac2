"""Seeded synthetic layers and activations shaped like the benchmark configurations.

Test infrastructure only (see ``oracle/__init__.py``).  Everything is produced as *logical*
tensors on the CPU; ``to_reference_checkpoint`` turns a layer into the tensors a reference
checkpoint would hold (reference storage layouts, ``layouts.py``).
"""

from __future__ import annotations

import dataclasses
import math

import numpy as np
import torch

from . import layouts, quant


@dataclasses.dataclass
class LogicalLayer:
    N: int
    K: int
    R: int
    wq: torch.Tensor  # int8 codes / uint8 E2M1 patterns [N, K]
    ws: torch.Tensor  # bf16 [K/64, N]  or  float8_e4m3fn [K/16, N]
    smooth: torch.Tensor  # bf16 [K]
    proj_down: torch.Tensor  # bf16 [K, R]
    proj_up: torch.Tensor  # bf16 [N, R]
    bias: torch.Tensor | None  # bf16 [N]
    fp4: bool = False
    wtscale: float = 1.0
    wcscales: torch.Tensor | None = None


def make_activations(M: int, K: int, seed: int, outlier_frac: float = 0.01, outlier_mul: float = 20.0) -> torch.Tensor:
    """bf16 ~N(0,1) with ``ceil(frac*K)`` channels multiplied by ``outlier_mul``."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    n_out = math.ceil(outlier_frac * K)
    idx = torch.randperm(K, generator=g)[:n_out]
    x[:, idx] *= outlier_mul
    return x.to(torch.bfloat16)


def make_layer(N: int, K: int, R: int, seed: int, fp4: bool = False, bias: bool = True) -> LogicalLayer:
    g = torch.Generator().manual_seed(seed + 1000)
    w = 0.02 * torch.randn(N, K, generator=g)
    smooth = (0.5 + 1.5 * torch.rand(K, generator=g)).to(torch.bfloat16)
    proj_down = (0.02 * torch.randn(K, R, generator=g)).to(torch.bfloat16)
    proj_up = (0.02 * torch.randn(N, R, generator=g)).to(torch.bfloat16)
    b = (0.02 * torch.randn(N, generator=g)).to(torch.bfloat16) if bias else None
    if fp4:
        wq, ws, wt = quant.quantize_weight_nvfp4(w)
        return LogicalLayer(N, K, R, wq, ws, smooth, proj_down, proj_up, b, True, wt, None)
    wq, ws = quant.quantize_weight_int4(w)
    return LogicalLayer(N, K, R, wq, ws, smooth, proj_down, proj_up, b)


def _u16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def to_reference_checkpoint(layer: LogicalLayer) -> dict[str, torch.Tensor]:
    """The state-dict tensors of one SVDQW4A4Linear in the reference's storage layouts
    (nunchaku/models/linear.py:38-72 for names/shapes/dtypes, packer.py for the byte order)."""
    sd = {
        "qweight": torch.from_numpy(layouts.pack_qweight(layer.wq.numpy())),
        "smooth_factor": _bf16(layouts.pack_vector(_u16(layer.smooth))),
        "smooth_factor_orig": torch.ones(layer.K, dtype=torch.bfloat16),
        "proj_down": _bf16(layouts.pack_lora(_u16(layer.proj_down), down=True)),
        "proj_up": _bf16(layouts.pack_lora(_u16(layer.proj_up), down=False)),
    }
    if layer.bias is not None:
        sd["bias"] = _bf16(layouts.pack_vector(_u16(layer.bias)))
    if layer.fp4:
        ws8 = layer.ws.contiguous().view(torch.uint8).numpy()
        sd["wscales"] = torch.from_numpy(layouts.pack_wmscales(ws8)).view(torch.float8_e4m3fn)
        sd["wtscale"] = torch.tensor([layer.wtscale], dtype=torch.bfloat16)
        wc = layer.wcscales if layer.wcscales is not None else torch.ones(layer.N, dtype=torch.bfloat16)
        sd["wcscales"] = _bf16(layouts.pack_vector(_u16(wc)))
    else:
        sd["wscales"] = _bf16(layouts.pack_wscales(_u16(layer.ws)))
    return sd


# (M, K, N, R, seed) of the benchmark configurations; the two-layer ones list both layers.
CONFIGS = {
    "c1": dict(M=256, K=3072, N=3072, R=32, seed=0),
    "c2_qkv": dict(M=4608, K=3072, N=9216, R=32, seed=1),
    "c3_fc1": dict(M=4608, K=3072, N=12288, R=32, seed=2),
    "c3_fc2": dict(M=4608, K=12288, N=3072, R=32, seed=2),
    "c4_qkv_mlp": dict(M=4608, K=3072, N=21504, R=32, seed=3, fp4=True),
    "c4_out": dict(M=4608, K=15360, N=3072, R=32, seed=3, fp4=True),
    "c5": dict(M=18432, K=3072, N=12288, R=128, seed=4),
}


# ---------------------------------------------------------------------------------------------
# A small checkpoint with the reference's key names, for the ingestion tests.
# ---------------------------------------------------------------------------------------------

# (checkpoint module name inside a block, N, K) of a toy double-stream block and a toy single-stream block;
# the names are those a reference checkpoint holds BEFORE convert_flux_state_dict
# (nunchaku/models/transformers/transformer_flux_v2.py:395-450)
TOY_BLOCK_LAYERS = {
    "transformer_blocks.0": (("qkv_proj", 384, 128), ("qkv_proj_context", 384, 128), ("out_proj", 128, 128), ("out_proj_context", 128, 128),
                             ("mlp_fc1", 256, 128), ("mlp_fc2", 128, 256), ("mlp_context_fc1", 256, 128), ("mlp_context_fc2", 128, 256)),
    "single_transformer_blocks.0": (("qkv_proj", 384, 128), ("mlp_fc1", 256, 128), ("mlp_fc2", 128, 256), ("out_proj", 128, 128)),
}


def toy_checkpoint(rank: int = 16, fp4_blocks: tuple[str, ...] = ()) -> tuple[dict[str, torch.Tensor], dict[str, LogicalLayer]]:
    """State dict in the reference's checkpoint naming (``lora_down``, ``lora_up``, ``smooth``,
    ``smooth_orig``, block-local module names) and the logical layers it was made from, keyed by the
    checkpoint prefix.  NVFP4 layers come without ``wtscale`` / ``wcscales`` when their seed is even, as
    older checkpoints do."""
    sd: dict[str, torch.Tensor] = {}
    layers: dict[str, LogicalLayer] = {}
    seed = 100
    for block, specs in TOY_BLOCK_LAYERS.items():
        for name, n, k in specs:
            seed += 1
            fp4 = block in fp4_blocks
            layer = make_layer(n, k, rank, seed=seed, fp4=fp4, bias=name != "mlp_fc2")
            if fp4 and seed % 2 == 0:
                layer.wtscale = 1.0
            ref = to_reference_checkpoint(layer)
            prefix = f"{block}.{name}"
            for key, value in ref.items():
                ck = {"proj_down": "lora_down", "proj_up": "lora_up", "smooth_factor": "smooth", "smooth_factor_orig": "smooth_orig"}.get(key, key)
                if fp4 and seed % 2 == 0 and key in ("wtscale", "wcscales"):
                    continue
                sd[f"{prefix}.{ck}"] = value
            layers[prefix] = layer
        sd[f"{block}.norm_q.weight"] = torch.ones(128, dtype=torch.bfloat16)
        sd[f"{block}.norm_k.weight"] = torch.ones(128, dtype=torch.bfloat16)
    sd["x_embedder.weight"] = torch.zeros(4, 4, dtype=torch.bfloat16)  # an unquantized tensor passes through
    return sd, layers
