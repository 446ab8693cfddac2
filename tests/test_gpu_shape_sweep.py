"""A seeded sweep over shapes and epilogue options of the two operators against the oracle: ragged token counts, N that is
not a multiple of the INT4 kernel's 256-column tile, ranks from 0 to 128 and a few up to 1024 (the reference's limit,
lora.cuh:22), with and without bias, per-channel scales, alpha, low-rank scale factors, tiles split along K, both
precisions.  Every case is small enough for the CPU oracle to check every element.  Every buffer the two operators write
lies between bands of a byte pattern, which must be intact afterwards."""

import random

import numpy as np
import pytest
import torch

from conftest import announce
from gpu_util import Guarded, check_output, make_module, make_oracle
from oracle import layouts as L
from oracle import synth

pytestmark = pytest.mark.gpu


def _cases():
    rng = random.Random(20240607)
    cases = []
    for i in range(28):
        fp4 = i % 4 == 3
        M = rng.choice([1, 17, 100, 255, 256, 257, 300, 511, 640, 900])
        K = 128 * rng.randint(1, 9)
        N = 128 * rng.randint(1, 11)
        R = rng.choice([0, 16, 32, 32, 48, 64, 96, 128])
        opts = dict(bias=rng.random() < 0.7, scales=rng.random() < 0.4, alpha=rng.choice([1.0, 1.0, 0.5, 1.7]) if not fp4 else None,
                    lora_scales=rng.random() < 0.4, k_split=rng.choice([None, None, 1, 2, 3]) if not fp4 else rng.choice([None, 1]))
        cases.append((i, M, K, N, R, fp4, opts))
    # long K with few tiles: the shapes where the library splits tiles along K by its own choice (INT4: in 2 to 8 parts;
    # NVFP4: parties of equal size)
    rng = random.Random(77)
    for i in range(100, 112):
        fp4 = i % 4 == 3
        M = rng.choice([100, 256, 300, 640])
        K = rng.choice([2048, 3072, 4096, 6144])
        N = 128 * rng.randint(1, 8)
        R = rng.choice([16, 32, 32, 64])
        opts = dict(bias=rng.random() < 0.7, scales=rng.random() < 0.4, alpha=rng.choice([1.0, 0.5]) if not fp4 else None,
                    lora_scales=rng.random() < 0.4, k_split=None)
        cases.append((i, M, K, N, R, fp4, opts))
    # ranks above 128 (a stock rank-32 branch with a rank-128 user LoRA appended is 160): the quantize operator
    # projects in windows of 128 ranks, the GEMM's up projection walks all of them
    rng = random.Random(99)
    for i, R in zip(range(200, 208), [160, 256, 160, 272, 1024, 256, 144, 512]):
        fp4 = i % 4 == 3
        M = rng.choice([100, 256, 300, 640])
        K = 128 * rng.randint(1, 6)
        N = 128 * rng.randint(1, 6)
        opts = dict(bias=rng.random() < 0.7, scales=rng.random() < 0.4, alpha=rng.choice([1.0, 0.5]) if not fp4 else None,
                    lora_scales=i % 2 == 0, k_split=None)
        cases.append((i, M, K, N, R, fp4, opts))
    return cases


@pytest.mark.parametrize("i,M,K,N,R,fp4,opts", _cases())
def test_layer_sweep(dev, i, M, K, N, R, fp4, opts, monkeypatch):
    from nunchaku_amd.ops import gemm as gemm_mod
    from nunchaku_amd.ops import svdq_gemm_w4a4

    announce(f"sweep {i}: M={M} K={K} N={N} R={R} fp4={fp4} {opts}")
    g = torch.Generator().manual_seed(1000 + i)
    layer = synth.make_layer(N, K, R, seed=500 + i, fp4=fp4, bias=opts["bias"])
    if opts["scales"]:
        layer.wcscales = (0.5 + torch.rand(N, generator=g)).to(torch.bfloat16)
    elif fp4:
        layer.wcscales = None
    x = synth.make_activations(M, K, seed=700 + i)
    m = make_module(layer, dev)
    ref = make_oracle(layer)
    alpha = float(torch.tensor(layer.wtscale).to(torch.bfloat16)) if fp4 else opts["alpha"]
    ref.wtscale = alpha
    ref.wcscales = layer.wcscales
    lora_scales = None
    if opts["lora_scales"] and R:
        lora_scales = [float(v) for v in (0.25 + 1.5 * torch.rand((R + 15) // 16, generator=g)).tolist()]
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_quantize_w4a4_act_fuse_lora

    t = m.native_tensors()
    M_pad = (M + 255) // 256 * 256
    G = 16 if fp4 else 64
    g_qx = Guarded((M_pad, packing.act_nbytes_per_row(K, fp4)), torch.uint8, dev)
    g_asc = Guarded((K // G, M_pad), torch.float8_e4m3fn if fp4 else torch.bfloat16, dev)
    g_la = Guarded((M_pad, R), torch.float32, dev)
    g_out = Guarded((M, N), torch.bfloat16, dev)
    qx, asc, la = svdq_quantize_w4a4_act_fuse_lora(x.to(dev), output=g_qx.t, oscales=g_asc.t, lora_down=t["proj_down"],
                                                   lora_act_out=g_la.t, smooth=t["smooth_factor"], fp4=fp4)
    out = g_out.t
    out.fill_(float("nan"))
    monkeypatch.setattr(gemm_mod, "K_SPLIT", opts["k_split"])
    wcs = None
    if fp4:
        wcs = t["wcscales"]  # part of an NVFP4 layer's checkpoint (ones when the layer has none)
    elif layer.wcscales is not None:
        # an INT4 module has no such parameter: the operator takes the reference's packed vector
        packed = L.pack_vector(layer.wcscales.view(torch.int16).numpy().view(np.uint16))
        wcs = torch.from_numpy(packed.view(np.int16).copy()).view(torch.bfloat16).to(dev)
    kw = dict(act=qx, wgt=t["qweight"], out=out, ascales=asc, wscales=t["wscales"], bias=t["bias"], fp4=fp4, alpha=alpha,
              wcscales=wcs, lora_scales=lora_scales)
    if R:
        kw.update(lora_act_in=la, lora_up=t["proj_up"])
    svdq_gemm_w4a4(**kw)
    torch.cuda.synchronize()
    for name, gd in (("quantized activations", g_qx), ("activation scales", g_asc), ("lora_act", g_la), ("out", g_out)):
        gd.check(name)
    assert not torch.isnan(out.float()).any()
    codes, scales, lora = ref.quantize(x)
    from oracle import linear as olin
    from oracle import quant

    a = quant.dequant_nvfp4(codes, scales) if fp4 else quant.dequant_int4(codes, scales)
    want = olin.gemm_w4a4(a, ref.w_deq, bias=layer.bias, lora_act_in=lora if R else None, lora_up=layer.proj_up if R else None,
                          lora_scales=lora_scales, alpha=alpha, wcscales=layer.wcscales)[:M]
    check_output(out, want)
