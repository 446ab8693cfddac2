"""Checkpoint ingestion, host side (no GPU): the key renames against the names spelled out by hand from
nunchaku/models/transformers/transformer_flux_v2.py:395-450, rank concatenation in the packed order against
the oracle's unpack -> concatenate -> pack, and the per-16-rank factors."""

import numpy as np
import pytest
import torch

from nunchaku_amd import checkpoint
from oracle import layouts as L
from oracle import synth


def test_key_renames_literal():
    keys = [
        "transformer_blocks.3.mlp_fc1.qweight", "transformer_blocks.3.mlp_fc2.lora_down", "transformer_blocks.3.mlp_context_fc1.smooth",
        "transformer_blocks.3.mlp_context_fc2.smooth_orig", "transformer_blocks.3.qkv_proj.lora_up", "transformer_blocks.3.qkv_proj_context.wscales",
        "transformer_blocks.3.out_proj.bias", "transformer_blocks.3.out_proj_context.qweight", "transformer_blocks.3.norm_q.weight",
        "transformer_blocks.3.norm_added_k.weight", "transformer_blocks.3.norm1.linear.qweight",
        "single_transformer_blocks.7.qkv_proj.smooth", "single_transformer_blocks.7.out_proj.lora_down", "single_transformer_blocks.7.mlp_fc1.lora_up",
        "single_transformer_blocks.7.norm_k.weight", "x_embedder.weight",
    ]
    want = [
        "transformer_blocks.3.ff.net.0.proj.qweight", "transformer_blocks.3.ff.net.2.proj_down", "transformer_blocks.3.ff_context.net.0.proj.smooth_factor",
        "transformer_blocks.3.ff_context.net.2.smooth_factor_orig", "transformer_blocks.3.attn.to_qkv.proj_up", "transformer_blocks.3.attn.add_qkv_proj.wscales",
        "transformer_blocks.3.attn.to_out.0.bias", "transformer_blocks.3.attn.to_add_out.qweight", "transformer_blocks.3.attn.norm_q.weight",
        "transformer_blocks.3.attn.norm_added_k.weight", "transformer_blocks.3.norm1.linear.qweight",
        "single_transformer_blocks.7.attn.to_qkv.smooth_factor", "single_transformer_blocks.7.attn.to_out.proj_down", "single_transformer_blocks.7.mlp_fc1.proj_up",
        "single_transformer_blocks.7.attn.norm_k.weight", "x_embedder.weight",
    ]
    got = checkpoint.convert_flux_state_dict({k: torch.zeros(1) for k in keys})
    assert list(got.keys()) == want


def test_toy_checkpoint_names_convert_to_module_paths():
    sd, layers = synth.toy_checkpoint(rank=16)
    conv = checkpoint.convert_flux_state_dict(sd)
    assert "transformer_blocks.0.ff.net.2.qweight" in conv and "single_transformer_blocks.0.attn.to_out.proj_up" in conv
    assert not any(".lora_down" in k or ".lora_up" in k or k.endswith(".smooth") or k.endswith(".smooth_orig") for k in conv)
    assert len([k for k in conv if k.endswith(".qweight")]) == len(layers) == 12


def test_concat_lowrank_is_rank_concatenation():
    rng = np.random.default_rng(0)

    def bf(a):
        return torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16)

    def packed(t, down):
        return torch.from_numpy(L.pack_lora(t.view(torch.int16).numpy().view(np.uint16), down=down).view(np.int16).copy()).view(torch.bfloat16)

    for down, C in ((True, 256), (False, 384)):
        a, b = bf(rng.standard_normal((C, 32))), bf(rng.standard_normal((C, 48)))
        got = checkpoint.concat_lowrank(packed(a, down), packed(b, down))
        want = packed(torch.cat((a, b), dim=1), down)
        assert got.shape == (C, 80) and torch.equal(got.view(torch.int16), want.view(torch.int16))
    with pytest.raises(ValueError):
        checkpoint.concat_lowrank(torch.zeros(256, 32, dtype=torch.bfloat16), torch.zeros(128, 16, dtype=torch.bfloat16))


def test_lora_scales_per_16_ranks():
    from nunchaku_amd.models.linear import SVDQW4A4Linear

    m = SVDQW4A4Linear(128, 128, rank=32)
    assert m.lora_scales is None
    m.update_lora(torch.zeros(128, 64, dtype=torch.bfloat16), torch.zeros(128, 64, dtype=torch.bfloat16))
    assert m.rank == 64 and m.lora_scales is None and tuple(m.proj_down.shape) == (128, 64)
    m.set_lora_scale(32, 0.7)  # the layer's own 32 ranks keep 1, the appended 32 get 0.7 (flux.h:177-196)
    assert m.lora_scales == [1.0, 1.0, 0.7, 0.7]
    with pytest.raises(ValueError):
        m.set_lora_scale(24, 0.5)
    with pytest.raises(ValueError):
        m.update_lora(torch.zeros(128, 24, dtype=torch.bfloat16), torch.zeros(128, 24, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        m.update_lora(torch.zeros(64, 32, dtype=torch.bfloat16), torch.zeros(128, 32, dtype=torch.bfloat16))
    # the rank grows with what is loaded (src/Linear.cpp:124-134): a rank-128 LoRA behind the layer's own 32 ranks
    m.update_lora(torch.zeros(128, 160, dtype=torch.bfloat16), torch.zeros(128, 160, dtype=torch.bfloat16))
    m.set_lora_scale(32, 0.5)
    assert m.rank == 160 and m.lora_scales == [1.0, 1.0] + [0.5] * 8
    with pytest.raises(ValueError):  # the reference's MAX_RANK (lora.cuh:22)
        m.update_lora(torch.zeros(128, 1040, dtype=torch.bfloat16), torch.zeros(128, 1040, dtype=torch.bfloat16))


def test_safetensors_round_trip(tmp_path):
    from safetensors.torch import save_file

    sd, _ = synth.toy_checkpoint(rank=16)
    path = tmp_path / "toy.safetensors"
    save_file({k: v.contiguous() for k, v in sd.items()}, str(path), metadata={"quantization_config": '{"rank": 16}'})
    tensors, meta = checkpoint.load_state_dict_in_safetensors(path)
    assert meta["quantization_config"] == '{"rank": 16}'
    assert set(tensors) == set(sd) and all(torch.equal(tensors[k].view(torch.uint8), sd[k].contiguous().view(torch.uint8)) for k in sd)
