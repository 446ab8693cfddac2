"""Checkpoint ingestion for the quantized linear layers: a reference ``.safetensors`` file (or state
dict) -> ``SVDQW4A4Linear`` / ``AWQW4A16Linear`` modules whose tensors have been converted once into the
layouts the gfx950 kernels read, plus the low-rank hot-swap helpers.

What the reference does, and where:

* key renames from the checkpoint's names to the module tree's names: ``convert_flux_state_dict``,
  nunchaku/models/transformers/transformer_flux_v2.py:395-450 (``lora_down -> proj_down``,
  ``lora_up -> proj_up``, ``smooth -> smooth_factor``, ``smooth_orig -> smooth_factor_orig``, and the
  block-local module names);
* per-tensor / per-channel scales that a checkpoint does not hold are ones: the same file, :264-269;
* a user LoRA is merged by concatenating its ranks behind the layer's own low-rank branch
  (nunchaku/lora/flux/nunchaku_converter.py: ``to_nunchaku`` -> packed ``lora_down`` / ``lora_up``), the
  layer's rank grows with whatever is loaded (src/Linear.cpp:124-134, ``lora_scales`` reset to ones, one
  per 16 ranks) and ``setLoraScale(skip_ranks, scale)`` scales the ranks behind the first ``skip_ranks``
  (nunchaku/csrc/flux.h:177-196).

Everything above the layers (the transformer, its attention, its pipelines) is out of this package's
scope: the functions here return the quantized layers keyed by their module path.
"""

from __future__ import annotations

from pathlib import Path

import torch

from .models.linear import AWQW4A16Linear, SVDQW4A4Linear

# (old, new) replacements inside a double-stream block ("transformer_blocks.N.") and a single-stream block
# ("single_transformer_blocks.N."), tried in order, first match wins
_DOUBLE_BLOCK_RENAMES = (
    (".mlp_context_fc1.", ".ff_context.net.0.proj."),
    (".mlp_context_fc2.", ".ff_context.net.2."),
    (".mlp_fc1.", ".ff.net.0.proj."),
    (".mlp_fc2.", ".ff.net.2."),
    (".qkv_proj_context.", ".attn.add_qkv_proj."),
    (".qkv_proj.", ".attn.to_qkv."),
    (".norm_q.", ".attn.norm_q."),
    (".norm_k.", ".attn.norm_k."),
    (".norm_added_q.", ".attn.norm_added_q."),
    (".norm_added_k.", ".attn.norm_added_k."),
    (".out_proj_context.", ".attn.to_add_out."),
    (".out_proj.", ".attn.to_out.0."),
)
_SINGLE_BLOCK_RENAMES = (
    (".qkv_proj.", ".attn.to_qkv."),
    (".out_proj.", ".attn.to_out."),
    (".norm_q.", ".attn.norm_q."),
    (".norm_k.", ".attn.norm_k."),
)


def _rename_tensor(key: str) -> str:
    key = key.replace(".lora_down", ".proj_down").replace(".lora_up", ".proj_up")
    if ".smooth_orig" in key:
        return key.replace(".smooth_orig", ".smooth_factor_orig")
    if ".smooth" in key and ".smooth_factor" not in key:
        return key.replace(".smooth", ".smooth_factor")
    return key


def convert_flux_state_dict(state_dict: dict[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    """Checkpoint key names -> module-tree key names (transformer_flux_v2.py:395-450).  Keys outside the
    transformer blocks pass through unchanged."""
    out = {}
    for key, value in state_dict.items():
        if "single_transformer_blocks." in key:
            table = _SINGLE_BLOCK_RENAMES
        elif "transformer_blocks." in key:
            table = _DOUBLE_BLOCK_RENAMES
        else:
            out[key] = value
            continue
        new_key = key
        for old, new in table:
            # (a norm_q / norm_k key carries both renames of its pair in the reference; one applies)
            if old in key:
                new_key = key.replace(old, new)
                break
        out[_rename_tensor(new_key)] = value
    return out


def load_state_dict_in_safetensors(path: str | Path, device: str | torch.device = "cpu") -> tuple[dict[str, torch.Tensor], dict[str, str]]:
    """Tensors and metadata of a ``.safetensors`` file (nothing is executed from the file)."""
    from safetensors import safe_open

    tensors = {}
    with safe_open(str(path), framework="pt", device=str(device)) as f:
        metadata = dict(f.metadata() or {})
        for key in f.keys():
            tensors[key] = f.get_tensor(key)
    return tensors, metadata


def build_quantized_layers(
    state_dict: dict[str, torch.Tensor], device: str | torch.device, convert_names: bool = True, act_unsigned_suffixes: tuple[str, ...] = (".ff.net.2", ".ff_context.net.2", ".mlp_fc2"),
) -> dict[str, torch.nn.Module]:
    """Every quantized linear layer found in ``state_dict`` as a loaded module on ``device``, keyed by its
    module path, with its native tensors already converted (one repack per layer, here, at load time).

    A layer is recognised by its ``qweight``: int8 ``[N, K/2]`` with ``wscales`` ``[K/G, N]`` is an
    ``SVDQW4A4Linear`` (NVFP4 when the scales are fp8; rank from ``proj_down``), int32 ``[N/4, K/2]`` with
    ``wzeros`` an ``AWQW4A16Linear``.  ``wtscale`` / ``wcscales`` missing from an NVFP4 checkpoint are ones
    (transformer_flux_v2.py:264-269).  Layers whose path ends in one of ``act_unsigned_suffixes`` take
    unsigned activations: the second MLP layers, fed by the fused GELU epilogue
    (``net[2].act_unsigned = net[2].precision != "nvfp4"``, nunchaku/models/attention.py:34;
    ``mlp_fc2`` of the single-stream block, transformer_flux_v2.py:180).
    """
    sd = convert_flux_state_dict(state_dict) if convert_names else dict(state_dict)
    prefixes = sorted(k[: -len(".qweight")] for k in sd if k.endswith(".qweight"))
    layers: dict[str, torch.nn.Module] = {}
    for prefix in prefixes:
        own = {k[len(prefix) + 1:]: v for k, v in sd.items() if k.startswith(prefix + ".")}
        qweight = own["qweight"]
        if qweight.dtype == torch.int32:
            if "wzeros" not in own or "wscales" not in own:
                raise ValueError(f"{prefix}: an int32 qweight needs wscales and wzeros (AWQ W4A16)")
            n, k = qweight.shape[0] * 4, qweight.shape[1] * 2
            module = AWQW4A16Linear(k, n, bias="bias" in own, group_size=k // own["wscales"].shape[0], device=device)
        elif qweight.dtype == torch.int8:
            n, k = qweight.shape[0], qweight.shape[1] * 2
            if "wscales" not in own or "proj_down" not in own or "proj_up" not in own or "smooth_factor" not in own:
                raise ValueError(f"{prefix}: an int8 qweight needs wscales, smooth, lora_down and lora_up (SVDQuant W4A4)")
            fp4 = own["wscales"].dtype == torch.float8_e4m3fn
            precision = "nvfp4" if fp4 else "int4"
            module = SVDQW4A4Linear(
                k, n, rank=own["proj_down"].shape[1], bias="bias" in own, precision=precision,
                act_unsigned=(not fp4) and prefix.endswith(act_unsigned_suffixes), device=device,
            )
            if "smooth_factor_orig" not in own:
                own["smooth_factor_orig"] = torch.ones_like(own["smooth_factor"])
            if fp4:
                own.setdefault("wtscale", torch.ones(1, dtype=torch.bfloat16))
                own.setdefault("wcscales", torch.ones(n, dtype=torch.bfloat16))
        else:
            raise ValueError(f"{prefix}.qweight has dtype {qweight.dtype}: not a quantized linear layer of this path")
        module.load_state_dict(own, strict=True)
        if isinstance(module, SVDQW4A4Linear):
            module.native_tensors()
        layers[prefix] = module
    return layers


def load_quantized_layers(path: str | Path, device: str | torch.device) -> tuple[dict[str, torch.nn.Module], dict[str, str]]:
    """``build_quantized_layers`` on a ``.safetensors`` file; also returns the file's metadata (the
    reference keeps ``quantization_config`` there, transformer_flux_v2.py:249-250)."""
    tensors, metadata = load_state_dict_in_safetensors(path)
    return build_quantized_layers(tensors, device), metadata


def concat_lowrank(base: torch.Tensor, extra: torch.Tensor) -> torch.Tensor:
    """Append the ranks of ``extra`` behind those of ``base``; both are low-rank weights ``[C, R]`` in the
    reference's packed order (down or up projection alike: 16 x 16 fragments, channel fragment major, rank
    fragment minor, each fragment 256 consecutive values: packer.py:362-398), so appending ranks is a
    concatenation of fragments."""
    if base.shape[0] != extra.shape[0] or base.shape[0] % 16 or base.shape[1] % 16 or extra.shape[1] % 16:
        raise ValueError("both tensors must be [C, R] with the same C, C and R multiples of 16")
    c = base.shape[0]
    joined = torch.cat((base.reshape(c // 16, base.shape[1] // 16, 256), extra.to(base.dtype).reshape(c // 16, extra.shape[1] // 16, 256)), dim=1)
    return joined.reshape(c, base.shape[1] + extra.shape[1]).contiguous()
