"""SVDQW4A4Linear end to end on the GPU: reference-format state dict -> load-time repack -> quantize
-> GEMM, against the oracle, at the CPU-reference configuration and through size-independent
properties at the FLUX shapes."""

import pytest
import torch

from conftest import announce
from gpu_util import check_output, make_module, make_oracle
from oracle import quant, synth

pytestmark = pytest.mark.gpu


def test_config1_full_layer(dev):
    """M=256, K=N=3072, rank 32, seed 0: the reference's own CPU-runnable case."""
    from nunchaku_amd import packing

    cfg = synth.CONFIGS["c1"]
    announce(f"linear config 1 {cfg}")
    layer = synth.make_layer(cfg["N"], cfg["K"], cfg["R"], seed=cfg["seed"])
    x = synth.make_activations(cfg["M"], cfg["K"], seed=cfg["seed"])
    m = make_module(layer, dev)
    ref = make_oracle(layer)
    y = m(x.to(dev).view(1, cfg["M"], cfg["K"]))
    torch.cuda.synchronize()
    assert y.shape == (1, cfg["M"], cfg["N"]) and y.dtype == torch.bfloat16
    qx, asc, la = m.quantize(x.to(dev))
    codes, scales, lora = ref.quantize(x)
    assert torch.equal(packing.act_to_logical(qx.cpu(), cfg["K"]), codes)
    assert torch.equal(asc.cpu().view(torch.int16), scales.view(torch.int16))
    want = ref.forward_quant(codes, scales, lora)[: cfg["M"]]
    rel = check_output(y[0], want)
    print(f"config 1 rel-L2 {rel:.2e}")


def test_ragged_tokens_3d_input(dev):
    announce("linear ragged tokens B=2 S=75")
    layer = synth.make_layer(256, 256, 32, seed=21)
    x = synth.make_activations(150, 256, seed=21)
    m = make_module(layer, dev)
    y = m(x.to(dev).view(2, 75, 256))
    torch.cuda.synchronize()
    want = make_oracle(layer).forward(x)
    check_output(y.reshape(150, 256), want)


def test_ops_accept_reference_layout_directly(dev):
    """nunchaku.ops callers pass checkpoint tensors as they are; they are repacked once and cached."""
    from nunchaku_amd import packing
    from nunchaku_amd.ops import svdq_gemm_w4a4, svdq_quantize_w4a4_act_fuse_lora

    announce("ops with reference-layout tensors")
    layer = synth.make_layer(256, 256, 32, seed=22)
    sd = {k: v.to(dev) for k, v in synth.to_reference_checkpoint(layer).items()}
    x = synth.make_activations(256, 256, seed=22)
    qx, asc, la = svdq_quantize_w4a4_act_fuse_lora(x.to(dev), lora_down=sd["proj_down"], smooth=sd["smooth_factor"])
    out = torch.empty(256, 256, dtype=torch.bfloat16, device=dev)
    for _ in range(2):
        svdq_gemm_w4a4(act=qx, wgt=sd["qweight"], out=out, ascales=asc, wscales=sd["wscales"], lora_act_in=la,
                       lora_up=sd["proj_up"], bias=sd["bias"])
    torch.cuda.synchronize()
    assert len(packing._cache) >= 5
    check_output(out, make_oracle(layer).forward(x))


def _full_shape_properties(dev, name, sample_rows=192, linearity=True):
    """One layer at a full-size configuration: the quantizer bit-exact against the oracle on all rows,
    the GEMM on a random sample of output rows, plus linearity in the bias."""
    from nunchaku_amd import packing

    cfg = synth.CONFIGS[name]
    announce(f"linear {name} {cfg}")
    M, K, N, R, fp4 = cfg["M"], cfg["K"], cfg["N"], cfg["R"], bool(cfg.get("fp4"))
    layer = synth.make_layer(N, K, R, seed=cfg["seed"], fp4=fp4)
    x = synth.make_activations(M, K, seed=cfg["seed"])
    m = make_module(layer, dev)
    ref = make_oracle(layer)
    if fp4:
        ref.wtscale = float(torch.tensor(layer.wtscale).to(torch.bfloat16))  # the checkpoint stores wtscale as bf16
    qx, asc, la = m.quantize(x.to(dev))
    y = m.forward_quant(qx, asc, la)[:M]
    torch.cuda.synchronize()
    codes, scales, lora = ref.quantize(x)
    if fp4:
        assert torch.equal(packing.act_to_logical(qx.cpu(), K, fp4=True).to(torch.uint8), codes)
        assert torch.equal(packing.scales_to_logical(asc.cpu(), True).view(torch.uint8), scales.view(torch.uint8))
    else:
        assert torch.equal(packing.act_to_logical(qx.cpu(), K), codes)
        assert torch.equal(asc.cpu().view(torch.int16), scales.view(torch.int16))
    assert (la.cpu()[:M] - lora[:M]).abs().max().item() <= 2e-5 * lora.abs().max().item()
    assert not torch.isnan(y.float()).any()
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(0))[:sample_rows]
    want = ref.forward_quant(codes[rows], scales[:, rows], lora[rows])
    check_output(y[rows], want)
    # Every tile of the output, through two checksums: the sum of each row and the sum of each column, against the same
    # sums of the oracle's formula taken before the matrix product (weights summed over the output channels, activations
    # over the rows).  A tile that is missing, stale or from the wrong place moves 128 column sums or 256 row sums by
    # about sqrt(128) .. sqrt(256) typical magnitudes; the bf16 rounding of the summed elements moves them by
    # sqrt(count) * 2^-9 of one.
    a = (quant.dequant_nvfp4(codes, scales) if fp4 else quant.dequant_int4(codes, scales))[:M].double()
    w = ref.w_deq.double()
    cf = torch.full((N,), float(ref.wtscale), dtype=torch.float64)
    if ref.wcscales is not None:
        cf = cf * ref.wcscales.double()
    lora_b = lora[:M].to(torch.bfloat16).double()
    up = layer.proj_up.double()
    bias = layer.bias.double()
    want_rows = a @ (w * cf[:, None]).sum(0) + bias.sum() + lora_b @ up.sum(0)
    want_cols = cf * (w @ a.sum(0)) + M * bias + up @ lora_b.sum(0)
    yd = y.double()
    rms = yd.pow(2).mean().sqrt().item()
    got_rows, got_cols = yd.sum(1).cpu(), yd.sum(0).cpu()
    assert (got_rows - want_rows).abs().max().item() <= 6 * N**0.5 * 2.0**-9 * rms, "row checksums"
    assert (got_cols - want_cols).abs().max().item() <= 6 * M**0.5 * 2.0**-9 * rms, "column checksums"
    if linearity:
        # bias linearity: y(bias) - y(0) == bias up to bf16 rounding of the two outputs
        m0 = make_module(synth.LogicalLayer(**{**layer.__dict__, "bias": torch.zeros_like(layer.bias)}), dev)
        y0 = m0.forward_quant(qx, asc, la)[:M]
        d = (y.float() - y0.float()).cpu() - layer.bias.float()[None, :]
        assert d.abs().max().item() <= 2 * 2.0**-7 * max(1.0, y.float().abs().max().item())


@pytest.mark.parametrize("name", ["c2_qkv", "c3_fc1"])
def test_flux_shapes_properties(dev, name):
    """Full FLUX shapes (INT4, rank 32)."""
    _full_shape_properties(dev, name)


@pytest.mark.parametrize("name", ["c4_qkv_mlp", "c4_out"])
def test_nvfp4_flux_shapes_properties(dev, name):
    """The NVFP4 configurations at full size: M=4608 with (K=3072, N=21504) and (K=15360, N=3072)."""
    _full_shape_properties(dev, name)


def test_batched_rank128_shape_properties(dev):
    """M=18432 (4 x 4608 tokens), K=3072, N=12288, rank 128: several batches of tiles per workgroup and
    four rounds of the low-rank up projection."""
    _full_shape_properties(dev, "c5", sample_rows=128)


@pytest.mark.parametrize("fp4", [False, True])
def test_forward_equals_the_two_operators(dev, fp4):
    """``forward`` goes through argument blocks prepared once per layer; the operator wrappers check and build
    everything per call.  Same bits, for row counts that change from call to call, a caller's output buffer,
    per-rank factors assigned as an attribute and a low-rank swap in between."""
    announce(f"forward against quantize + forward_quant, fp4={fp4}")
    layer = synth.make_layer(384, 256, 32, seed=31, fp4=fp4)
    m = make_module(layer, dev)
    for rows in (300, 75, 512):
        x = synth.make_activations(rows, 256, seed=rows).to(dev)
        want = m._forward_by_operators(x, None)
        got = m(x.view(1, rows, 256))
        assert torch.equal(got[0], want[:rows])  # (forward_quant without an output returns the padded rows)
    buf = torch.full((2, 75, 384), 7.0, dtype=torch.bfloat16, device=dev)
    x = synth.make_activations(150, 256, seed=5).to(dev)
    assert m(x.view(2, 75, 256), buf).data_ptr() == buf.data_ptr()
    assert torch.equal(buf.view(150, 384), m._forward_by_operators(x, None)[:150])
    m.lora_scales = [1.0, 0.25]
    assert torch.equal(m(x.view(1, 150, 256))[0], m._forward_by_operators(x, None)[:150])
    m.lora_scales = None
    from nunchaku_amd.checkpoint import concat_lowrank

    m.update_lora(concat_lowrank(m.proj_down.data, m.proj_down.data), concat_lowrank(m.proj_up.data, -m.proj_up.data))  # rank 64
    m.set_lora_scale(32, 0.5)
    assert torch.equal(m(x.view(1, 150, 256))[0], m._forward_by_operators(x, None)[:150])
    with pytest.raises(ValueError):
        m(x.view(1, 150, 256)[:, :, :128])
    with pytest.raises(ValueError):
        m(x.view(1, 150, 256), torch.empty(150, 385, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError):
        m(x.cpu().view(1, 150, 256))


def test_forward_refuses_a_parameter_of_the_wrong_shape(dev):
    announce("forward with a hand-assigned parameter of the wrong shape")
    layer = synth.make_layer(256, 256, 32, seed=33)
    m = make_module(layer, dev)
    x = synth.make_activations(256, 256, seed=33).to(dev).view(1, 256, 256)
    m(x)
    m.proj_up = torch.nn.Parameter(m.proj_up.data[:128].clone(), requires_grad=False)
    with pytest.raises(ValueError):
        m(x)


def test_one_layer_from_two_threads(dev):
    """A layer's prepared argument blocks are shared by the threads that call it: each call fills them and launches
    under the layer's lock, so concurrent forwards with different row counts give what they give alone."""
    import threading

    announce("one layer called from two threads")
    layer = synth.make_layer(384, 3072, 32, seed=35)  # (K = 3072 with few tiles: the GEMM takes the split path and its workspace)
    m = make_module(layer, dev)
    xs = {rows: synth.make_activations(rows, 3072, seed=rows).to(dev).view(1, rows, 3072) for rows in (100, 300)}
    want = {rows: m(x).clone() for rows, x in xs.items()}
    torch.cuda.synchronize()
    errors = []

    def work(rows):
        try:
            for _ in range(50):
                y = m(xs[rows])
                torch.cuda.synchronize()
                if not torch.equal(y, want[rows]):
                    errors.append(f"rows={rows}: a forward differs")
                    return
        except Exception as e:  # (an exception in a thread would otherwise pass unnoticed)
            errors.append(repr(e))

    threads = [threading.Thread(target=work, args=(rows,)) for rows in xs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
