"""GEMM epilogue that prepares the next layer (GELU -> shift/smooth/quantize unsigned + low-rank down
projection) and the fused MLP built on it, against the oracle."""

import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_module, make_oracle
from oracle import linear as olin
from oracle import quant, synth

pytestmark = pytest.mark.gpu


def _mlp(dev, M, K1, N1, N2, R, seed):
    fc1 = synth.make_layer(N1, K1, R, seed=seed)
    fc2 = synth.make_layer(N2, N1, R, seed=seed + 1)
    x = synth.make_activations(M, K1, seed=seed)
    m1 = make_module(fc1, dev)
    m2 = make_module(fc2, dev, act_unsigned=True)
    return fc1, fc2, x, m1, m2


@pytest.mark.parametrize("M,K1,N1,N2,R", [(256, 256, 512, 256, 32), (300, 384, 1024, 384, 16), (512, 3072, 1536, 256, 64)])
def test_next_layer_epilogue(dev, M, K1, N1, N2, R):
    """GEMM with `out` and `qout`: the stored post-GELU bf16 tile is within tolerance of the oracle,
    and the codes / scales / low-rank projection produced next to it are exactly (resp. to fp32
    tolerance) what the oracle derives from that very tile."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4

    announce(f"gemm next-layer epilogue M={M} K1={K1} N1={N1} R={R}")
    fc1, fc2, x, m1, m2 = _mlp(dev, M, K1, N1, N2, R, seed=M + N1)
    t1, t2 = m1.native_tensors(), m2.native_tensors()
    qx, asc, la = m1.quantize(x.to(dev))
    M_pad = qx.shape[0]
    out = torch.empty(M_pad, N1, dtype=torch.bfloat16, device=dev)
    qout = torch.empty(M_pad, N1 * 3 // 4, dtype=torch.uint8, device=dev)
    osc = torch.empty(N1 // 64, M_pad, dtype=torch.bfloat16, device=dev)
    la2 = torch.full((M_pad, R), float("nan"), dtype=torch.float32, device=dev)
    svdq_gemm_w4a4(act=qx, wgt=t1["qweight"], out=out, qout=qout, ascales=asc, wscales=t1["wscales"], oscales=osc,
                   lora_act_in=la, lora_up=t1["proj_up"], lora_down=t2["proj_down"], lora_act_out=la2, bias=t1["bias"],
                   smooth_factor=t2["smooth_factor"])
    torch.cuda.synchronize()
    ref1 = make_oracle(fc1)
    codes, scales, lora = ref1.quantize(x)
    want_h = ref1.forward_quant(codes, scales, lora, gelu=True)
    check_output(out, want_h)
    # the quantizer part, bit-exact given the bf16 tile the kernel itself stored
    h = out.cpu()
    want_codes, want_scales = quant.quantize_act_int4(h, fc2.smooth, unsigned=True, shift=quant.SHIFT_GELU)
    got_codes = packing.act_to_logical(qout.cpu(), N1, unsigned=True)
    assert torch.equal(got_codes, want_codes), f"{(got_codes != want_codes).sum().item()} codes differ"
    assert torch.equal(osc.cpu().view(torch.int16), want_scales.view(torch.int16))
    want_la2 = (h.double() @ fc2.proj_down.double()).float()
    assert (la2.cpu() - want_la2).abs().max().item() <= 3e-5 * want_la2.abs().max().item() + 1e-6


@pytest.mark.parametrize("M,K1,N1,N2,R", [(256, 256, 512, 256, 32), (150, 512, 2048, 512, 32), (256, 3072, 512, 256, 32)])
def test_fused_gelu_mlp(dev, M, K1, N1, N2, R):
    from nunchaku_amd.ops import fused_gelu_mlp

    announce(f"fused_gelu_mlp M={M} K1={K1} N1={N1} N2={N2} R={R}")
    fc1, fc2, x, m1, m2 = _mlp(dev, M, K1, N1, N2, R, seed=N1 + N2)
    y = fused_gelu_mlp(x.to(dev).view(1, M, K1), m1, m2)
    torch.cuda.synchronize()
    assert y.shape == (1, M, N2)
    want, _ = olin.fused_gelu_mlp(x, make_oracle(fc1), make_oracle(fc2, act_unsigned=True))
    # The intermediate is re-quantized to 4 bits: an element of the post-GELU tile that rounds to the
    # neighbouring bf16 value (different fp32 summation order) can move a code, so the chain is
    # compared at 5e-3; the exact step-by-step check is test_next_layer_epilogue.
    got = y[0].float().cpu()
    rel = ((got - want.to(torch.bfloat16).float()).norm() / want.norm()).item()
    assert rel <= 5e-3, rel


def test_mlp_flux_shape(dev):
    """FLUX MLP pair at full size (M=4608, 3072 -> 12288 -> 3072): step-by-step exactness on a row
    sample plus the whole chain on the same sample."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import fused_gelu_mlp, svdq_gemm_w4a4

    c1, c2 = synth.CONFIGS["c3_fc1"], synth.CONFIGS["c3_fc2"]
    announce(f"flux mlp pair {c1} {c2}")
    M = c1["M"]
    fc1 = synth.make_layer(c1["N"], c1["K"], c1["R"], seed=c1["seed"])
    fc2 = synth.make_layer(c2["N"], c2["K"], c2["R"], seed=c2["seed"] + 1)
    x = synth.make_activations(M, c1["K"], seed=c1["seed"])
    m1, m2 = make_module(fc1, dev), make_module(fc2, dev, act_unsigned=True)
    y = fused_gelu_mlp(x.to(dev).view(1, M, c1["K"]), m1, m2)[0]
    # redo fc1 with `out` to look at the intermediate
    t1, t2 = m1.native_tensors(), m2.native_tensors()
    qx, asc, la = m1.quantize(x.to(dev))
    out = torch.empty(M, c1["N"], dtype=torch.bfloat16, device=dev)
    qout = torch.empty(M, c1["N"] * 3 // 4, dtype=torch.uint8, device=dev)
    osc = torch.empty(c1["N"] // 64, M, dtype=torch.bfloat16, device=dev)
    la2 = torch.empty(M, c2["R"], dtype=torch.float32, device=dev)
    svdq_gemm_w4a4(act=qx, wgt=t1["qweight"], out=out, qout=qout, ascales=asc, wscales=t1["wscales"], oscales=osc,
                   lora_act_in=la, lora_up=t1["proj_up"], lora_down=t2["proj_down"], lora_act_out=la2, bias=t1["bias"],
                   smooth_factor=t2["smooth_factor"])
    torch.cuda.synchronize()
    # The low-rank input of fc2 is summed over 48 column blocks whose workgroups finish in no fixed order: the shares
    # are added in ascending order afterwards, so a second launch must reproduce the sums, and with them the layer
    # output, bit for bit.
    la2_first, y_first = la2.clone(), y.clone()
    for _ in range(3):
        la2.fill_(float("nan"))
        svdq_gemm_w4a4(act=qx, wgt=t1["qweight"], out=out, qout=qout, ascales=asc, wscales=t1["wscales"], oscales=osc,
                       lora_act_in=la, lora_up=t1["proj_up"], lora_down=t2["proj_down"], lora_act_out=la2, bias=t1["bias"],
                       smooth_factor=t2["smooth_factor"])
        y_again = fused_gelu_mlp(x.to(dev).view(1, M, c1["K"]), m1, m2)[0]
        torch.cuda.synchronize()
        assert torch.equal(la2, la2_first), "the next layer's low-rank input changed between two launches"
        assert torch.equal(y_again, y_first), "the fused MLP's output changed between two launches"
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(3))[:128]
    h = out.cpu()[rows]
    want_codes, want_scales = quant.quantize_act_int4(h, fc2.smooth, unsigned=True, shift=quant.SHIFT_GELU)
    assert torch.equal(packing.act_to_logical(qout.cpu(), c1["N"], unsigned=True)[rows], want_codes)
    assert torch.equal(osc.cpu()[:, rows].view(torch.int16), want_scales.view(torch.int16))
    want_la2 = (h.double() @ fc2.proj_down.double()).float()
    assert (la2.cpu()[rows] - want_la2).abs().max().item() <= 3e-5 * want_la2.abs().max().item()
    # fc2 on the kernel's own intermediate
    ref2 = make_oracle(fc2, act_unsigned=True)
    want_y = ref2.forward_quant(want_codes, want_scales, want_la2)
    check_output(y[rows], want_y)


def test_side_streams_give_the_same_bits(dev):
    """The library launches on the caller's current stream and keeps one workspace per (device, stream): the fused
    MLP whose first GEMM is split along K (parked sums, arrival counters) and leaves low-rank shares, run in turn on
    two side streams, gives what the default stream gave."""
    from nunchaku_amd.ops import fused_gelu_mlp

    M, K1, N1, N2, R = 256, 3072, 512, 256, 32
    announce(f"fused_gelu_mlp on side streams M={M} K1={K1} N1={N1} N2={N2}")
    fc1, fc2, x, m1, m2 = _mlp(dev, M, K1, N1, N2, R, seed=77)
    xd = x.to(dev).view(1, M, K1)
    want = fused_gelu_mlp(xd, m1, m2)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]
    outs = []
    for s in streams + streams:
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            outs.append(fused_gelu_mlp(xd, m1, m2))
    torch.cuda.synchronize()
    for got in outs:
        assert torch.equal(got, want)
