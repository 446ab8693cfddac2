"""Checkpoint ingestion end to end on the GPU: a small multi-layer ``.safetensors`` file with the
reference's key names and storage layouts (written by ``oracle/synth.py``) -> layers -> outputs against the
oracle layer by layer; the low-rank hot swap (rank growth, per-16-rank factors) on a loaded layer."""

import numpy as np
import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_oracle
from oracle import layouts as L
from oracle import linear as olin
from oracle import synth

pytestmark = pytest.mark.gpu


def _module_path(prefix):
    from nunchaku_amd import checkpoint

    return next(iter(checkpoint.convert_flux_state_dict({prefix + ".qweight": None}))).rsplit(".qweight", 1)[0]


@pytest.mark.parametrize("fp4_blocks", [(), ("single_transformer_blocks.0",)])
def test_load_toy_checkpoint_and_run_every_layer(dev, tmp_path, fp4_blocks):
    from safetensors.torch import save_file

    from nunchaku_amd import checkpoint
    from nunchaku_amd.models.linear import SVDQW4A4Linear
    from nunchaku_amd.ops import fused_gelu_mlp

    sd, logical = synth.toy_checkpoint(rank=16, fp4_blocks=fp4_blocks)
    path = tmp_path / "toy.safetensors"
    save_file({k: v.contiguous() for k, v in sd.items()}, str(path), metadata={"quantization_config": '{"rank": 16}'})
    announce(f"checkpoint: load {path.name} ({len(logical)} quantized layers, nvfp4 blocks {fp4_blocks})")
    layers, meta = checkpoint.load_quantized_layers(path, dev)
    assert meta["quantization_config"] == '{"rank": 16}'
    assert set(layers) == {_module_path(p) for p in logical}
    M = 200
    for prefix, layer in logical.items():
        mod = layers[_module_path(prefix)]
        assert isinstance(mod, SVDQW4A4Linear) and mod.rank == 16 and mod.precision == ("nvfp4" if layer.fp4 else "int4")
        assert mod.act_unsigned == (prefix.endswith("fc2") and not layer.fp4)
        if prefix.endswith("fc2"):
            continue  # run below, behind its first layer
        announce(f"checkpoint: layer {prefix} N={layer.N} K={layer.K}")
        x = synth.make_activations(M, layer.K, seed=layer.N + layer.K)
        ref = make_oracle(layer)
        if layer.fp4:
            ref.wtscale = float(torch.tensor(layer.wtscale).to(torch.bfloat16))
        y = mod(x.to(dev).view(1, M, layer.K))[0]
        torch.cuda.synchronize()
        check_output(y, ref.forward(x))
    for fc1_prefix in [p for p in logical if p.endswith("fc1")]:
        fc2_prefix = fc1_prefix[:-1] + "2"
        announce(f"checkpoint: fused mlp {fc1_prefix} -> {fc2_prefix}")
        l1, l2 = logical[fc1_prefix], logical[fc2_prefix]
        r1, r2 = make_oracle(l1), make_oracle(l2, act_unsigned=not l2.fp4)
        for r, l in ((r1, l1), (r2, l2)):
            if l.fp4:
                r.wtscale = float(torch.tensor(l.wtscale).to(torch.bfloat16))
        x = synth.make_activations(M, l1.K, seed=7)
        y = fused_gelu_mlp(x.to(dev).view(1, M, l1.K), layers[_module_path(fc1_prefix)], layers[_module_path(fc2_prefix)])[0]
        torch.cuda.synchronize()
        want, _ = olin.fused_gelu_mlp(x, r1, r2)
        # (the second layer quantizes the first one's bf16 output: a flipped rounding there moves a code by one)
        got = y.float().cpu()
        rel = ((got - want.to(torch.bfloat16).float()).norm() / want.norm()).item()
        assert rel <= 2e-2, rel


@pytest.mark.parametrize("R2", [16, 128, 224])  # a rank-128 user LoRA behind a stock rank-32 branch is rank 160
def test_lora_hot_swap_rank_growth_and_scales(dev, R2):
    from nunchaku_amd import checkpoint
    from nunchaku_amd.models.linear import SVDQW4A4Linear

    N, K, R, M = 256, 256, 32, 300
    announce(f"lora hot swap N={N} K={K} rank {R} + {R2}")
    layer = synth.make_layer(N, K, R, seed=21)
    mod = SVDQW4A4Linear(K, N, rank=R, device=dev)
    mod.load_state_dict(synth.to_reference_checkpoint(layer))
    x = synth.make_activations(M, K, seed=22)
    y0 = mod(x.to(dev).view(1, M, K))[0].clone()
    check_output(y0, make_oracle(layer).forward(x))

    g = torch.Generator().manual_seed(23)
    extra_down = (0.05 * torch.randn(K, R2, generator=g)).to(torch.bfloat16)
    extra_up = (0.05 * torch.randn(N, R2, generator=g)).to(torch.bfloat16)

    def packed(t, down):
        return torch.from_numpy(L.pack_lora(t.view(torch.int16).numpy().view(np.uint16), down=down).view(np.int16).copy()).view(torch.bfloat16)

    mod.update_lora(checkpoint.concat_lowrank(mod.proj_down.data.cpu(), packed(extra_down, True)),
                    checkpoint.concat_lowrank(mod.proj_up.data.cpu(), packed(extra_up, False)))
    assert mod.rank == R + R2
    for strength in (1.0, 0.7, 0.0):
        mod.set_lora_scale(R, strength)
        y = mod(x.to(dev).view(1, M, K))[0]
        torch.cuda.synchronize()
        grown = synth.LogicalLayer(N, K, R + R2, layer.wq, layer.ws, layer.smooth, torch.cat((layer.proj_down, extra_down), 1),
                                   torch.cat((layer.proj_up, extra_up), 1), layer.bias)
        ref = make_oracle(grown)
        codes, scales, lora = ref.quantize(x)
        from oracle import quant

        want = olin.gemm_w4a4(quant.dequant_int4(codes, scales), ref.w_deq, bias=ref.bias, lora_act_in=lora, lora_up=ref.proj_up,
                              lora_scales=[1.0, 1.0] + [strength] * (R2 // 16))[:M]
        check_output(y, want)
        if strength == 0.0:
            assert torch.equal(y, y0)  # the appended ranks switched off: the original layer, bit for bit
        else:
            assert not torch.equal(y, y0)
