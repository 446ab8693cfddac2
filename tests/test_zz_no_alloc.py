"""``svdq_gemm_w4a4_noalloc``: the GEMM for callers that cannot allocate.  Calls that need a workspace (tiles
split along K, the next layer's low-rank sums) take it from a fixed array in device memory; the results
must equal those of ``svdq_gemm_w4a4`` bit for bit (same kernels, same order of the partial sums), also on
the second of two calls in a row that uses less of the array than the first (what the first call left
there must not leak into it)."""

import pytest
import torch

from conftest import announce
from gpu_util import make_module
from oracle import synth

pytestmark = pytest.mark.gpu


def _run(dev, gemm_mod, m, M, K, N, R, seed, no_alloc, k_split, monkeypatch):
    from nunchaku_amd import packing

    monkeypatch.setattr(gemm_mod, "NO_ALLOC", no_alloc)
    monkeypatch.setattr(gemm_mod, "K_SPLIT", k_split)
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(-8, 8, (M, K), generator=g).to(torch.int8)
    scales = (torch.rand(K // 64, M, generator=g) * 0.5 + 0.01).to(torch.bfloat16)
    lora_act = torch.randn(M, R, generator=g) * 3
    t = m.native_tensors()
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    gemm_mod.svdq_gemm_w4a4(act=packing.logical_to_act(codes).to(dev), wgt=t["qweight"], out=out, ascales=scales.to(dev),
                            wscales=t["wscales"], lora_act_in=lora_act.to(dev), lora_up=t["proj_up"], bias=t["bias"])
    torch.cuda.synchronize()
    return out


def test_noalloc_split_tiles_two_calls_in_a_row(dev, monkeypatch):
    from nunchaku_amd.ops import gemm as gemm_mod

    big = dict(M=512, K=1024, N=768, R=32)    # 12 tiles x 8 parts: 12.6 MB of partial sums
    small = dict(M=256, K=512, N=256, R=16)   # 2 tiles x 4 parts
    mods = {}
    for name, c in (("big", big), ("small", small)):
        mods[name] = make_module(synth.make_layer(c["N"], c["K"], c["R"], seed=c["K"]), dev)
    announce("noalloc split tiles: reference results through svdq_gemm_w4a4")
    want_big = _run(dev, gemm_mod, mods["big"], **big, seed=1, no_alloc=False, k_split=8, monkeypatch=monkeypatch)
    want_small = _run(dev, gemm_mod, mods["small"], **small, seed=2, no_alloc=False, k_split=4, monkeypatch=monkeypatch)
    announce("noalloc split tiles: big call, then a smaller one, through svdq_gemm_w4a4_noalloc")
    got_big = _run(dev, gemm_mod, mods["big"], **big, seed=1, no_alloc=True, k_split=8, monkeypatch=monkeypatch)
    got_small = _run(dev, gemm_mod, mods["small"], **small, seed=2, no_alloc=True, k_split=4, monkeypatch=monkeypatch)
    assert not torch.isnan(got_big.float()).any() and not torch.isnan(got_small.float()).any()
    assert torch.equal(got_big, want_big)
    assert torch.equal(got_small, want_small)
    # and once more in the other order
    assert torch.equal(_run(dev, gemm_mod, mods["small"], **small, seed=2, no_alloc=True, k_split=4, monkeypatch=monkeypatch), want_small)
    assert torch.equal(_run(dev, gemm_mod, mods["big"], **big, seed=1, no_alloc=True, k_split=8, monkeypatch=monkeypatch), want_big)


def test_noalloc_next_layer_sums_two_calls_in_a_row(dev, monkeypatch):
    """The fused MLP's first GEMM (next layer's quantized input and low-rank sums) through the fixed array,
    for a larger and then a smaller layer pair."""
    from nunchaku_amd.ops import fused_gelu_mlp
    from nunchaku_amd.ops import gemm as gemm_mod

    results = {}
    for no_alloc in (False, True):
        monkeypatch.setattr(gemm_mod, "NO_ALLOC", no_alloc)
        for name, (M, K, N1, R) in (("big", (700, 256, 1024, 32)), ("small", (200, 128, 256, 16))):
            announce(f"noalloc fused mlp {name} no_alloc={no_alloc}")
            fc1 = make_module(synth.make_layer(N1, K, R, seed=11), dev)
            fc2 = make_module(synth.make_layer(K, N1, R, seed=12), dev, act_unsigned=True)
            x = synth.make_activations(M, K, seed=13).to(dev).view(1, M, K)
            y = fused_gelu_mlp(x, fc1, fc2)
            torch.cuda.synchronize()
            results[(name, no_alloc)] = y
    for name in ("big", "small"):
        assert not torch.isnan(results[(name, True)].float()).any()
        assert torch.equal(results[(name, True)], results[(name, False)])


def test_noalloc_refuses_what_does_not_fit(dev, monkeypatch):
    from nunchaku_amd.ops import gemm as gemm_mod

    c = dict(M=2048, K=1024, N=2048, R=16)  # 128 tiles x 16 parts x 128 KB = 268 MB of partial sums
    m = make_module(synth.make_layer(c["N"], c["K"], c["R"], seed=3), dev)
    with pytest.raises(NotImplementedError, match="fixed scratch"):
        _run(dev, gemm_mod, m, **c, seed=3, no_alloc=True, k_split=16, monkeypatch=monkeypatch)


def test_noalloc_forward_in_a_graph(dev, monkeypatch):
    """What the entry point is for: the layer's forward (quantize, then a GEMM split along K whose parked sums and
    arrival counters live in the fixed array) captured into a graph and replayed, with eager work of the same layer
    between the replays; every replay gives the eager result."""
    from nunchaku_amd.ops import gemm as gemm_mod

    announce("forward through svdq_gemm_w4a4_noalloc captured into a graph")
    monkeypatch.setattr(gemm_mod, "NO_ALLOC", True)
    monkeypatch.setattr(gemm_mod, "K_SPLIT", None)
    M, K, N, R = 256, 3072, 512, 32
    m = make_module(synth.make_layer(N, K, R, seed=9), dev)
    xs = [synth.make_activations(M, K, seed=100 + i).to(dev).view(1, M, K) for i in range(3)]
    eager = [m(x).clone() for x in xs]
    torch.cuda.synchronize()
    static_x = xs[0].clone()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            m(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = m(static_x)
    for _ in range(2):
        for i, x in enumerate(xs):
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            z = m(x)
            torch.cuda.synchronize()
            assert torch.equal(y, eager[i]) and torch.equal(z, eager[i])
