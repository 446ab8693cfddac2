"""The workspace policy of ``svdq_gemm_w4a4`` (``csrc/gemm.hip``): one block per (device, stream) pair for the launches that
need one; a block that a launch has been given is never freed or moved by a later call (a pair that comes to need more
gets a new, larger block and the old one stays allocated); a call that would have to allocate while its stream is being
captured is refused with an error code instead of an allocation inside the capture; ``svdq_release_workspaces`` frees
everything, after which calls allocate again.

A captured graph keeps the addresses it was recorded with: the test records a split GEMM into a graph, makes the pair
outgrow its block with a larger eager call, and replays the graph, which must still give the eager result."""

import pytest
import torch

from conftest import announce
from gpu_util import make_module
from oracle import synth

pytestmark = pytest.mark.gpu


def _layer_call(dev, gemm_mod, m, M, K, R, seed):
    from nunchaku_amd import packing

    M_pad = (M + 255) // 256 * 256
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(-8, 8, (M_pad, K), generator=g).to(torch.int8)
    act = packing.logical_to_act(codes).to(dev)
    sc = (torch.rand(K // 64, M_pad, generator=g) * 0.5 + 0.01).to(torch.bfloat16).to(dev)
    la = (torch.randn(M_pad, R, generator=g) * 3).to(dev)
    t = m.native_tensors()

    def run(out):
        gemm_mod.svdq_gemm_w4a4(act=act, wgt=t["qweight"], out=out, ascales=sc, wscales=t["wscales"], lora_act_in=la,
                                lora_up=t["proj_up"], bias=t["bias"])
        return out

    return run


def test_a_pair_outgrows_its_block_and_a_graph_recorded_before_still_replays(dev, monkeypatch):
    from nunchaku_amd import _native as nv
    from nunchaku_amd.ops import gemm as gemm_mod

    announce("workspace: growth behind a recorded graph, refusal under capture, release")
    monkeypatch.setattr(gemm_mod, "NO_ALLOC", False)
    small = dict(M=256, K=1024, N=512, R=16)    # 4 tiles x 4 parts: 2 MB of parked sums
    big = dict(M=512, K=2048, N=1024, R=16)     # 16 tiles x 8 parts: 16 MB
    m_small = make_module(synth.make_layer(small["N"], small["K"], small["R"], seed=31), dev)
    m_big = make_module(synth.make_layer(big["N"], big["K"], big["R"], seed=32), dev)
    run_small = _layer_call(dev, gemm_mod, m_small, small["M"], small["K"], small["R"], seed=1)
    run_big = _layer_call(dev, gemm_mod, m_big, big["M"], big["K"], big["R"], seed=2)
    out_small = torch.empty(small["M"], small["N"], dtype=torch.bfloat16, device=dev)
    out_big = torch.empty(big["M"], big["N"], dtype=torch.bfloat16, device=dev)

    # what the two calls give without any workspace (whole tiles); a split sum may differ from it by a bf16 ulp, so the
    # split results are compared with themselves bit for bit and with this one closely
    monkeypatch.setattr(gemm_mod, "K_SPLIT", 1)
    whole_small, whole_big = run_small(torch.empty_like(out_small)).clone(), run_big(torch.empty_like(out_big)).clone()
    torch.cuda.synchronize()

    side = torch.cuda.Stream(device=dev)
    # (1) a stream whose pair has no block yet: the call is refused under capture, nothing is allocated, nothing is launched
    monkeypatch.setattr(gemm_mod, "K_SPLIT", 4)
    refused = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="captured"):
        with torch.cuda.graph(refused, stream=side):
            run_small(out_small)
    torch.cuda.synchronize()

    # (2) the same call made once before the capture gives the pair its block; then it can be recorded
    with torch.cuda.stream(side):
        eager_small = run_small(out_small).clone()
    torch.cuda.synchronize()
    assert torch.allclose(eager_small.float(), whole_small.float(), rtol=2e-2, atol=2e-2)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run_small(out_small)
    out_small.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out_small, eager_small)

    # (3) a larger call on the same stream: the pair outgrows its block; the recorded graph goes on using the old one
    monkeypatch.setattr(gemm_mod, "K_SPLIT", 8)
    with torch.cuda.stream(side):
        eager_big = run_big(out_big).clone()
    torch.cuda.synchronize()
    assert torch.allclose(eager_big.float(), whole_big.float(), rtol=2e-2, atol=2e-2)
    for _ in range(3):
        out_small.zero_()
        graph.replay()
        with torch.cuda.stream(side):  # eager work of the pair's new block between the replays
            run_big(out_big)
        torch.cuda.synchronize()
        assert torch.equal(out_small, eager_small), "a replay after the pair's block was replaced gives another result"
        assert torch.equal(out_big, eager_big)

    # (4) release: the graph must not be replayed any more; calls allocate again and give the same results
    del graph, refused
    torch.cuda.synchronize()
    assert nv.lib().svdq_release_workspaces() == 0
    monkeypatch.setattr(gemm_mod, "K_SPLIT", 4)
    with torch.cuda.stream(side):
        again = run_small(out_small).clone()
    torch.cuda.synchronize()
    assert torch.equal(again, eager_small)
