"""Benchmark of the SVDQuant W4A4 + low-rank linear hot path on one MI355X.

One step = one forward of the layer on inputs already resident in HBM: the quantize + low-rank-down
kernel followed by the W4A4 GEMM kernel (bias and low-rank up fused).  Workload: FLUX.1-dev MLP fc1,
M=4608 tokens, K=3072, N=12288, rank 32, INT4 group 64, bf16 in/out, synthetic seeded data.

Prints ONE JSON line:  metric = effective TOPS of the fused layer, (2MNK + 2MR(K+N)) / step time;
`roofline` describes the GEMM kernel (the dominant one), timed with events on the launch stream;
`cpu_baseline` is the CPU oracle (PyTorch fake-quant layer) timed on this machine's host cores on a
bounded row sample of the same layer.
"""

from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import subprocess
import sys
import threading
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

WORKLOADS = {
    "flux_mlp_fc1": dict(M=4608, K=3072, N=12288, R=32, seed=2),
    "flux_qkv": dict(M=4608, K=3072, N=9216, R=32, seed=1),
    "flux_mlp_fc2": dict(M=4608, K=12288, N=3072, R=32, seed=2),
    "qwen_batched_r128": dict(M=18432, K=3072, N=12288, R=128, seed=4),
    "c1_small": dict(M=256, K=3072, N=3072, R=32, seed=0),
    # NVFP4 variant of the FLUX single-block layers: fused QKV + MLP-in projection, and the output projection
    "flux_single_nvfp4": dict(M=4608, K=3072, N=21504, R=32, seed=3, fp4=True),
    "flux_single_out_nvfp4": dict(M=4608, K=15360, N=3072, R=32, seed=3, fp4=True),
}
INT8_PEAK_TOPS = 5000.0  # MI355X dense INT8 MFMA, the peak the metric is quoted against
# HBM-side bytes per GEMM launch: rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (KiB per dispatch, mean of the launches of
# `bench.py --only gemm --workload W --steps 3`), each scaled by what the same counter reads for a device copy of known size
# (`bench.py --only copy`: FETCH_SIZE reads 131085 for 262144 KiB, factor 2.0; WRITE_SIZE reads 262144, factor 1.0).  The
# commands and the readings are in profiles/w4a4_gemm_hbm_traffic_all_workloads.md; a workload that is not in the table (a
# custom --shape, --qkv-rope) reports null.
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0
PROFILED_GEMM_FETCH_WRITE_KIB = {
    "flux_mlp_fc1": (143432.6, 110593.0),
    "flux_qkv": (103458.7, 82944.7),
    "flux_mlp_fc2": (154337.3, 27648.0),
    "qwen_batched_r128": (696300.5, 442369.8),
    "c1_small": (12905.7, 13827.8),
    "flux_single_nvfp4": (146101.8, 197586.7),
    "flux_single_out_nvfp4": (121730.6, 28944.1),
}
PROFILED_GEMM_TRAFFIC_BYTES = {w: (FETCH_SCALE * f + WRITE_SCALE * wr) * 1024 for w, (f, wr) in PROFILED_GEMM_FETCH_WRITE_KIB.items()}
HBM_PEAK_GBS = 8000.0


class Sensors:
    """Shader clock and package power as `rocm-smi` reports them, sampled by a thread while a timed loop runs."""

    def __init__(self):
        self.samples, self.stop = [], threading.Event()

    def _run(self):
        while not self.stop.is_set():
            try:
                txt = subprocess.run(["rocm-smi", "--showclocks", "--showpower", "--json"], capture_output=True, text=True, timeout=10).stdout
                card = next(iter(json.loads(txt).values()))
                clk = [float(re.search(r"(\d+)\s*Mhz", v, re.I).group(1)) for k, v in card.items() if k.lower().startswith("sclk") and re.search(r"(\d+)\s*Mhz", str(v), re.I)]
                pw = [float(v) for k, v in card.items() if "power" in k.lower() and re.fullmatch(r"[\d.]+", str(v).strip())]
                self.samples.append((clk[0] if clk else None, pw[0] if pw else None))
            except Exception:  # no tool, no permission, another output format: the timings stand without it
                return

    def __enter__(self):
        self.thread = threading.Thread(target=self._run, daemon=True)
        self.thread.start()
        return self

    def __exit__(self, *exc):
        self.stop.set()
        self.thread.join(timeout=15)

    def text(self):
        clk = [c for c, _ in self.samples[1:] if c]  # (the first sample may predate the loop)
        pw = [w for _, w in self.samples[1:] if w]
        if not clk and not pw:
            return "no sensor samples"
        return (f"sclk median {statistics.median(clk):.0f} MHz of {len(clk)} samples" if clk else "no clock samples") + \
               (f", package power median {statistics.median(pw):.0f} W" if pw else "")


def cpu_baseline(layer, x, rows: int, iters: int = 20):
    """The oracle's fake-quant layer on the host cores, on the first `rows` rows of the workload."""
    import torch

    from oracle import linear as olin

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    ref = olin.FakeQuantLinear(layer.wq, layer.ws, layer.smooth, layer.proj_down, layer.proj_up, layer.bias,
                               fp4=layer.fp4, wtscale=float(torch.tensor(layer.wtscale).to(torch.bfloat16)) if layer.fp4 else 1.0,
                               wcscales=layer.wcscales)
    xs = x[:rows].contiguous()
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        y = ref.forward(xs, double=False).to(torch.bfloat16)
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    ops = 2.0 * rows * layer.N * layer.K + 2.0 * rows * layer.R * (layer.K + layer.N)
    return {
        "value": ops / t / 1e12, "unit": "TOPS", "cores": cores, "kind": "port",
        "sample": f"first {rows} of {x.shape[0]} rows of the same layer, fp32 matmul, median of {iters}",
        "seconds_per_pass": t,
    }, y


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="flux_mlp_fc1", choices=sorted(WORKLOADS))
    ap.add_argument("--shape", default=None, help="M,K,N,R of an INT4 layer to time instead of a named workload (seed 9)")
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="keep the GPU busy with the same step for this long before the warm-up steps: after an idle period "
                         "(the seconds of synthetic-data preparation on the host) the first ~100 ms of work run 10-28 %% slower "
                         "while the power management settles; 0 measures from cold")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=4608)
    ap.add_argument("--qkv-rope", action="store_true",
                    help="time the GEMM with the RMS-norm + rotary epilogue of fused_qkv_norm_rottary (workload flux_qkv); "
                         "the CPU comparison is skipped")
    ap.add_argument("--only", choices=["gemm", "quantize", "copy", "awq-gemv", "fused-mlp", "litela", "power"], default=None,
                    help="profiling aid: launch only one of the two kernels in the timed loops (prints no JSON); "
                         "'copy' launches a plain device copy of 256 MiB, the yardstick for the HBM traffic counters; "
                         "'awq-gemv' times the AWQ W4A16 GEMV at the modulation shape (1 row, K=3072, N=18432); "
                         "'fused-mlp' times fused_gelu_mlp on the FLUX MLP pair (M=4608, 3072 -> 12288 -> 3072); "
                         "'litela' times the linear-attention pair (QKV projection with the q / vk epilogue, then vk times q) at "
                         "4096 tokens, K=2304, 72 heads of 32; "
                         "'power' times the workload's GEMM kernel launched back to back on its synthetic activations and on all-zero "
                         "activations (same weights, same launches), and the vendor library's dense GEMM of the same "
                         "M, K, N (fp16 and bf16 through torch.matmul, int8 through torch._int_mm) on random and on zero operands: "
                         "a kernel whose time follows the operands' bit activity at equal work runs against the power limit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    if args.only == "fused-mlp":
        from nunchaku_amd.models.linear import SVDQW4A4Linear
        from nunchaku_amd.ops import fused_gelu_mlp
        from oracle import synth

        dev = torch.device("cuda:0")
        M, K, N, R = 4608, 3072, 12288, 32
        mods = []
        for (n, k, unsigned, seed) in ((N, K, False, 2), (K, N, True, 3)):
            mod = SVDQW4A4Linear(k, n, rank=R, act_unsigned=unsigned, device=dev)
            mod.load_state_dict(synth.to_reference_checkpoint(synth.make_layer(n, k, R, seed=seed)))
            mod.native_tensors()
            mods.append(mod)
        x = synth.make_activations(M, K, seed=2).to(dev).view(1, M, K)
        for _ in range(20):
            fused_gelu_mlp(x, mods[0], mods[1])
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fused_gelu_mlp(x, mods[0], mods[1])
        e1.record()
        torch.cuda.synchronize()
        print(f"fused-mlp M={M} {K}->{N}->{K} rank {R}: {e0.elapsed_time(e1) * 1e3 / args.steps:.1f} us per call "
              "(quantize + fc1 with GELU / next-layer quantize / low-rank-down epilogue + fc2)")
        return
    if args.only == "litela":
        from nunchaku_amd.models.linear import SVDQW4A4Linear
        from nunchaku_amd.ops import linearattn_vk_mul_q, svdq_gemm_w4a4
        from oracle import synth

        dev = torch.device("cuda:0")
        T, K, heads, R = 4096, 2304, 72, 32
        N = heads * 96
        mod = SVDQW4A4Linear(K, N, rank=R, device=dev)
        mod.load_state_dict(synth.to_reference_checkpoint(synth.make_layer(N, K, R, seed=1)))
        t = mod.native_tensors()
        qx, asc, la = mod.quantize(synth.make_activations(T, K, seed=1).to(dev))
        out = torch.empty(T, N, dtype=torch.bfloat16, device=dev)
        q = torch.empty(1, T, N // 3, dtype=torch.bfloat16, device=dev)
        vk = torch.empty(1, heads, 33, 32, dtype=torch.float32, device=dev)
        base = dict(act=qx, wgt=t["qweight"], ascales=asc, wscales=t["wscales"], lora_act_in=la, lora_up=t["proj_up"], bias=t["bias"])
        for name, fn in (("plain layer of the shape", lambda: svdq_gemm_w4a4(**base, out=out)),
                         ("projection with relu(q) and vk sums", lambda: svdq_gemm_w4a4(**base, out_vk=vk, out_linearattn=q)),
                         ("vk times q", lambda: linearattn_vk_mul_q(q, vk))):
            for _ in range(20):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(args.steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            print(f"litela T={T} K={K} heads={heads} rank {R}: {name}: {e0.elapsed_time(e1) * 1e3 / args.steps:.1f} us per call")
        return
    if args.only == "awq-gemv":
        from nunchaku_amd.ops import awq_gemv_w4a16

        K, N = 3072, 18432
        dev = torch.device("cuda:0")
        gen = torch.Generator().manual_seed(0)
        qw = torch.randint(-2**31, 2**31 - 1, (N // 4, K // 2), generator=gen, dtype=torch.int32).to(dev)
        sc = (0.001 + 0.002 * torch.rand(K // 64, N, generator=gen)).to(torch.bfloat16).to(dev)
        zr = (-0.02 * torch.rand(K // 64, N, generator=gen)).to(torch.bfloat16).to(dev)
        bias = (0.02 * torch.randn(N, generator=gen)).to(torch.bfloat16).to(dev)
        for rows in (1, 4, 8):
            x = torch.randn(rows, K, generator=gen).to(torch.bfloat16).to(dev)
            for _ in range(20):
                awq_gemv_w4a16(x, qw, sc, zr, rows, N, K, bias=bias)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(args.steps):
                awq_gemv_w4a16(x, qw, sc, zr, rows, N, K, bias=bias)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / args.steps
            nbytes = N * K / 2 + 2 * 2 * (K // 64) * N + 2 * N + rows * (K + N) * 2  # codes, scales + zeros, bias, x and out
            print(f"awq-gemv rows={rows} K={K} N={N}: {us:.2f} us per launch (back to back), {nbytes / us / 1e3:.0f} GB/s of {nbytes / 1e6:.1f} MB")
        return
    if args.only == "copy":
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(f"copy: {args.steps} device copies of {src.numel()} bytes (reads {src.numel()}, writes {src.numel()})")
        return

    from nunchaku_amd.models.linear import SVDQW4A4Linear
    from oracle import synth

    cfg = WORKLOADS[args.workload]
    if args.shape:
        m_, k_, n_, r_ = (int(v) for v in args.shape.split(","))
        cfg = dict(M=m_, K=k_, N=n_, R=r_, seed=9)
        args.workload = f"custom_{m_}x{k_}x{n_}_r{r_}"
    M, K, N, R = cfg["M"], cfg["K"], cfg["N"], cfg["R"]
    dev = torch.device("cuda:0")
    fp4 = bool(cfg.get("fp4"))
    layer = synth.make_layer(N, K, R, seed=cfg["seed"], fp4=fp4)
    x = synth.make_activations(M, K, seed=cfg["seed"])
    mod = SVDQW4A4Linear(K, N, rank=R, precision="nvfp4" if fp4 else "int4", device=dev)
    mod.load_state_dict(synth.to_reference_checkpoint(layer))
    mod.native_tensors()  # load-time repack happens once, outside the timed region
    xd = x.to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    M_pad = (M + 255) // 256 * 256
    from nunchaku_amd import packing

    qx = torch.empty(M_pad, packing.act_nbytes_per_row(K, fp4), dtype=torch.uint8, device=dev)
    asc = torch.empty(K // 16, M_pad, dtype=torch.float8_e4m3fn, device=dev) if fp4 else torch.empty(K // 64, M_pad, dtype=torch.bfloat16, device=dev)
    la = torch.empty(M_pad, R, dtype=torch.float32, device=dev)
    t = mod.native_tensors()
    from nunchaku_amd.ops import svdq_quantize_w4a4_act_fuse_lora

    gemm = lambda: mod.forward_quant(qx, asc, la, out)  # noqa: E731
    if args.qkv_rope:
        if N % 384 != 0:
            sys.exit("--qkv-rope needs a QKV-shaped workload (N three equal parts of 128-wide heads): use --workload flux_qkv")
        from nunchaku_amd import packing
        from nunchaku_amd.ops import svdq_gemm_w4a4

        args.no_cpu = True
        gen = torch.Generator().manual_seed(cfg["seed"])
        ang = torch.rand(M_pad, 64, generator=gen) * 6.283
        # (sin, cos) pairs stay adjacent in the reference's packed order, so a table of random angles is as
        # good a packed table as any: taken as written by pack_rotemb and converted like a caller's table
        rot = packing.repack_rotemb(torch.stack((torch.sin(ang), torch.cos(ang)), dim=-1).reshape(M_pad, 128).to(dev))
        nq = (1.0 + 0.2 * torch.randn(128, generator=gen)).to(torch.bfloat16).to(dev)
        nk = (1.0 + 0.2 * torch.randn(128, generator=gen)).to(torch.bfloat16).to(dev)

        def gemm():
            svdq_gemm_w4a4(act=qx, wgt=t["qweight"], out=out, ascales=asc, wscales=t["wscales"], lora_act_in=la,
                           lora_up=t["proj_up"], bias=t["bias"], norm_q=nq, norm_k=nk, rotary_emb=rot)

    def step():
        svdq_quantize_w4a4_act_fuse_lora(xd, output=qx, oscales=asc, lora_down=t["proj_down"], lora_act_out=la, smooth=t["smooth_factor"], fp4=fp4)
        gemm()

    if args.only == "power":
        def b2b(fn, n=args.steps, sensors=None):
            for _ in range(max(10, args.warmup)):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            if sensors is not None:
                sensors.__enter__()
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            if sensors is not None:
                sensors.__exit__()
            return e0.elapsed_time(e1) * 1e3 / n

        t_settle = time.perf_counter()  # the first loop would otherwise run while the power management still ramps up
        while (time.perf_counter() - t_settle) * 1e3 < max(args.settle_ms, 500.0):
            for _ in range(10):
                gemm()
            torch.cuda.synchronize()

        ops = 2.0 * M * N * K
        for name, xs in (("synthetic activations", xd), ("all-zero activations", torch.zeros_like(xd)), ("synthetic activations again", xd)):
            svdq_quantize_w4a4_act_fuse_lora(xs, output=qx, oscales=asc, lora_down=t["proj_down"], lora_act_out=la, smooth=t["smooth_factor"], fp4=fp4)
            sens = Sensors()
            us = b2b(gemm, sensors=sens)
            print(f"power {args.workload}: W4A4 GEMM kernel, {name}: {us:.1f} us per launch, {ops / us / 1e6:.0f} TOPS ({sens.text()})", flush=True)
        for dt in (torch.float16, torch.bfloat16, torch.int8):
            for kind in ("random", "zero"):
                if dt == torch.int8:
                    a = torch.randint(-127, 128, (M_pad, K), device=dev, dtype=torch.int8) if kind == "random" else torch.zeros(M_pad, K, device=dev, dtype=torch.int8)
                    b = torch.randint(-127, 128, (K, N), device=dev, dtype=torch.int8) if kind == "random" else torch.zeros(K, N, device=dev, dtype=torch.int8)
                    try:
                        sens = Sensors()
                        us = b2b(lambda: torch._int_mm(a, b), sensors=sens)
                    except Exception as exc:  # the library has no such kernel for the shape
                        print(f"power {args.workload}: vendor int8 GEMM unavailable: {type(exc).__name__}: {exc}", flush=True)
                        break
                else:
                    a = (torch.randn(M_pad, K, device=dev) if kind == "random" else torch.zeros(M_pad, K, device=dev)).to(dt)
                    b = (torch.randn(N, K, device=dev) if kind == "random" else torch.zeros(N, K, device=dev)).to(dt)
                    o = torch.empty(M_pad, N, device=dev, dtype=dt)
                    sens = Sensors()
                    us = b2b(lambda: torch.matmul(a, b.t(), out=o), sensors=sens)
                print(f"power {args.workload}: vendor dense GEMM {str(dt).split('.')[-1]} M={M_pad} K={K} N={N}, {kind} operands: {us:.1f} us per launch, "
                      f"{2.0 * M_pad * N * K / us / 1e6:.0f} T(FL)OPS ({sens.text()})", flush=True)
        return
    if args.only:
        svdq_quantize_w4a4_act_fuse_lora(xd, output=qx, oscales=asc, lora_down=t["proj_down"], lora_act_out=la, smooth=t["smooth_factor"], fp4=fp4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            if args.only == "gemm":
                gemm()
            else:
                svdq_quantize_w4a4_act_fuse_lora(xd, output=qx, oscales=asc, lora_down=t["proj_down"], lora_act_out=la, smooth=t["smooth_factor"], fp4=fp4)
        torch.cuda.synchronize()
        print(f"{args.only}: {(time.perf_counter() - t0) * 1e6 / args.steps:.1f} us per launch (host clock, {args.steps} launches)")
        return

    # settle phase: not part of the warm-up count, reported in the output
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # whole-step time: exactly `steps` steps between two synchronisations
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    # the same loop timed by events on the launch stream: what the GPU spent, without the host's share
    s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s0.record()
    for _ in range(args.steps):
        step()
    s1.record()
    torch.cuda.synchronize()
    ms_per_step_events = s0.elapsed_time(s1) / args.steps

    # per-kernel durations with events on the stream the kernels are launched on
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    for e in evs:
        e[0].record()
        svdq_quantize_w4a4_act_fuse_lora(xd, output=qx, oscales=asc, lora_down=t["proj_down"], lora_act_out=la, smooth=t["smooth_factor"], fp4=fp4)
        e[1].record()
        gemm()
        e[2].record()
    torch.cuda.synchronize()
    tq_us = statistics.mean(e[0].elapsed_time(e[1]) for e in evs) * 1e3
    tg_us = statistics.mean(e[1].elapsed_time(e[2]) for e in evs) * 1e3
    # the short kernel again, launched back to back: events around ONE launch of a 15 us kernel include the
    # launch gap (about 4 us), which the kernel's own duration (rocprofv3 kernel trace) does not
    b0, b1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    b0.record()
    for _ in range(args.steps):
        svdq_quantize_w4a4_act_fuse_lora(xd, output=qx, oscales=asc, lora_down=t["proj_down"], lora_act_out=la, smooth=t["smooth_factor"], fp4=fp4)
    b1.record()
    torch.cuda.synchronize()
    tq_b2b_us = b0.elapsed_time(b1) * 1e3 / args.steps
    # The GEMM kernel's duration.  Three readings, all from events on the launch stream: (1) the interval between an
    # event after the quantize kernel and one after the GEMM (above): an event between two kernels adds about 4 us of
    # gap to the interval after it; (2) launches that follow each other directly (below): the chip is power-bound in
    # this kernel and runs 3-6 % slower when nothing memory-bound separates the launches; (3) the step's duration
    # minus the quantize kernel's: the kernel as it runs in the measured step, launch gaps charged to it.  (3) is what
    # the roofline uses; it is the reading that agrees with the rocprofv3 kernel trace of this command.
    g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    g0.record()
    for _ in range(args.steps):
        gemm()
    g1.record()
    torch.cuda.synchronize()
    tg_b2b_us = g0.elapsed_time(g1) * 1e3 / args.steps
    tg_step_us = ms_per_step_events * 1e3 - tq_b2b_us
    # The shader clock while the step runs (outside the timed region: about a second of the same steps with a thread
    # reading `rocm-smi`).  The GEMM is bound by the chip's power limit: the clock the power management grants on these
    # operands, against the 2400 MHz that the published peaks assume, is part of what `roofline.frac` measures.  Not
    # under a profiler, whose preloaded tool would load into the child processes too.
    clock = None
    profiled = any("rocprof" in os.environ.get(k, "").lower() for k in ("LD_PRELOAD", "ROCP_TOOL_LIBRARIES", "HSA_TOOLS_LIB", "ROCPROFILER_LIBRARY_PATH"))
    if not profiled:
        sens = Sensors()
        with sens:
            t_clk = time.perf_counter()
            while time.perf_counter() - t_clk < 1.0:
                for _ in range(20):
                    step()
                torch.cuda.synchronize()
        clk = [c for c, _ in sens.samples[1:] if c]
        if clk:
            clock = {"sclk_mhz_median_during_steps": statistics.median(clk), "samples": len(clk), "published_peak_clock_mhz": 2400,
                     "source": "rocm-smi --showclocks, sampled for one second of the same steps after the timed region"}

    ops_layer = 2.0 * M * N * K + 2.0 * M * R * (K + N)
    ops_gemm = 2.0 * M * N * K + 2.0 * M * R * N
    bytes_quant = 2.0 * M * K + M * K / 2 + (M * K / 16 if fp4 else 2.0 * M * K / 64) + 4.0 * M * R + 2.0 * K * R + 2.0 * K
    value = ops_layer / (ms_per_step * 1e-3) / 1e12
    gemm_tops = ops_gemm / (tg_step_us * 1e-6) / 1e12
    res = {
        "metric": "effective TOPS of fused W4A4+LoRA linear at FLUX M=4608; % of MFMA peak",
        "value": value, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "settle_ms": args.settle_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if fp4 else "e2m3 x e2m3 -> f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: SVDQW4A4Linear forward M={M} K={K} N={N} rank={R} {'NVFP4 g16' if fp4 else 'INT4 g64'} bf16 in/out"
                               + (" + RMS norm and rotary embedding on q, k in the GEMM epilogue" if args.qkv_rope else ""),
                   "M": M, "K": K, "N": N, "rank": R},
        "pct_of_int8_mfma_peak": 100.0 * value / INT8_PEAK_TOPS,
        "clock": clock,
        "us_per_layer": ms_per_step * 1e3,
        "us_per_layer_events": ms_per_step_events * 1e3,
        "kernels": {
            "quantize_fuse_lora_us": tq_us, "gemm_us": tg_step_us, "gemm_us_back_to_back": tg_b2b_us, "gemm_us_with_event_gap": tg_us,
            "quantize_fuse_lora_us_back_to_back": tq_b2b_us,
            "quantize_GBps": bytes_quant / (tq_b2b_us * 1e-6) / 1e9,
            "quantize_frac_of_hbm_peak": bytes_quant / (tq_b2b_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "gemm_main_term_TOPS": 2.0 * M * N * K / (tg_step_us * 1e-6) / 1e12,
        },
        "roofline": {
            "kernel": (f"gemm_w4a4_kernel<{'true' if args.qkv_rope else 'false'}>" if fp4 else f"g6::gemm6_kernel<{'true' if args.qkv_rope else 'false'}>"),
            "bound": "mfma", "achieved": gemm_tops, "peak": INT8_PEAK_TOPS,
            "unit": "TFLOP/s", "frac": gemm_tops / INT8_PEAK_TOPS, "traffic": None if args.qkv_rope else PROFILED_GEMM_TRAFFIC_BYTES.get(args.workload),
            "peak_basis": "dense INT8 MFMA (the metric's peak)" + ("; the NVFP4 kernel issues fp16 MFMA, dense peak 2500" if fp4 else
                          "; the INT4 kernel issues one fp6 MFMA (dense peak 10100) and one small bf16 MFMA per 32x32 tile and k-group"),
        },
    }
    if not args.no_cpu:
        cb, y_cpu = cpu_baseline(layer, x, min(args.cpu_rows, M))
        # the same rows from the GPU must agree with the CPU oracle (checker, not the thing measured)
        got = out[: y_cpu.shape[0]].float().cpu()
        rel = ((got - y_cpu.float()).norm() / y_cpu.float().norm()).item()
        cb["gpu_vs_cpu_rel_l2"] = rel
        res["cpu_baseline"] = cb
    print(json.dumps(res))


if __name__ == "__main__":
    main()
