"""``SVDQW4A4Linear`` with the constructor, parameter names/shapes/dtypes and methods of
nunchaku/models/linear.py:9-135, so that a reference checkpoint's state dict loads unchanged.

The parameters keep the reference storage layout (that is what checkpoints hold).  The first use
after loading converts them once into the gfx950-native layouts (``native_tensors``); the converted
tensors are what the kernels read.
"""

from __future__ import annotations

import ctypes
import threading

import torch
from torch import nn

from .. import _native as nv
from .. import packing
from ..ops import gemm as _gemm_op
from ..ops.gemm import svdq_gemm_w4a4
from ..ops.quantize import svdq_quantize_w4a4_act_fuse_lora


class _LayerCall:
    """The argument blocks of a layer's two C-ABI calls with everything filled in that does not change from one
    forward to the next (the layer's own tensors and sizes); ``SVDQW4A4Linear.forward`` only sets the pointers and
    row counts of the call.  The layer's tensors were checked when they were converted; the per-call tensors are
    allocated by ``forward`` itself, so the checks of the operator wrappers have nothing left to find."""

    def __init__(self, mod: "SVDQW4A4Linear", t: dict):
        fp4 = mod.precision == "nvfp4"
        K, N, R = mod.in_features, mod.out_features, mod.rank
        # the kernels read every element these sizes promise: parameters assigned by hand must keep them
        # (load_state_dict and update_lora check on their own)
        sdt = torch.float8_e4m3fn if fp4 else torch.bfloat16
        for name, shape, dtype in (("qweight", (N, K // 2), torch.int8), ("wscales", (K // mod.group_size, N), sdt),
                                   ("smooth_factor", (K,), torch.bfloat16), ("proj_down", (K, R), torch.bfloat16),
                                   ("proj_up", (N, R), torch.bfloat16), ("bias", (N,), torch.bfloat16), ("wcscales", (N,), torch.bfloat16)):
            p = mod._parameters.get(name)
            if p is None and name in ("bias", "wcscales"):
                continue
            if p is None or tuple(p.shape) != shape or p.dtype != dtype:
                raise ValueError(f"{name} must be {dtype} {shape} for in_features={K}, out_features={N}, rank={R}, got "
                                 f"{None if p is None else (p.dtype, tuple(p.shape))}")
        self.fp4 = fp4
        self.act_bytes = packing.act_nbytes_per_row(K, fp4)
        self.groups = K // mod.group_size
        self.scale_dtype = torch.float8_e4m3fn if fp4 else torch.bfloat16
        self.tensors = t  # keeps the converted tensors alive as long as their addresses are in the blocks
        self.q = nv.QuantizeArgs(
            lora_down=nv.ptr(t["proj_down"]) if R else None, smooth_rcp=nv.ptr(t["smooth_factor"]),
            K=K, R=R, fp4=int(fp4), fuse_glu=0,
        )
        self.device = t["qweight"].device
        self.sc = (ctypes.c_float * max(1, (R + 15) // 16))()
        self.scales_src = ()  # what self.sc was last written from (never a list or None: the first call writes)
        self.g = nv.GemmArgs(
            wgt=nv.ptr(t["qweight"]), wscales=nv.ptr(t["wscales"]), colnorm=nv.ptr(t["wscales"].colnorm), bias=nv.ptr(t["bias"]),
            wcscales=nv.ptr(t["wcscales"]), lora_up=nv.ptr(t["proj_up"]) if R else None, lora_scales=self.sc,
            N=N, K=K, N_out=N, R_up=R, R_down=0, alpha=float(mod.alpha), act_unsigned=int(mod.act_unsigned), fuse_silu=0, fp4=int(fp4),
            norm_eps=_gemm_op.NORM_EPS,
        )
        self.q_ref, self.g_ref = ctypes.byref(self.q), ctypes.byref(self.g)
        self.lock = threading.Lock()  # the blocks are shared by the threads that call the layer


class SVDQW4A4Linear(nn.Module):
    def __init__(
        self,
        in_features: int,
        out_features: int,
        rank: int = 32,
        bias: bool = True,
        precision: str = "int4",
        act_unsigned: bool = False,
        torch_dtype: torch.dtype = torch.bfloat16,
        device: str | torch.device | None = None,
    ):
        super().__init__()
        if device is None:
            device = torch.device("cpu")
        self.in_features = in_features
        self.out_features = out_features
        self.rank = rank
        self.precision = precision
        self.torch_dtype = torch_dtype
        if precision == "nvfp4":
            self.group_size = 16
        elif precision == "int4":
            self.group_size = 64
        else:
            raise ValueError(f"Invalid precision: {precision}")
        if torch_dtype != torch.bfloat16:
            raise NotImplementedError("only torch.bfloat16 layers are supported")

        self.qweight = nn.Parameter(torch.empty(out_features, in_features // 2, dtype=torch.int8, device=device), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(out_features, dtype=torch_dtype, device=device), requires_grad=True) if bias else None
        self.wscales = nn.Parameter(
            torch.empty(
                in_features // self.group_size, out_features,
                dtype=torch_dtype if precision == "int4" else torch.float8_e4m3fn, device=device,
            ),
            requires_grad=False,
        )
        self.smooth_factor = nn.Parameter(torch.empty(in_features, dtype=torch_dtype, device=device), requires_grad=False)
        self.smooth_factor_orig = nn.Parameter(torch.empty(in_features, dtype=torch_dtype, device=device), requires_grad=False)
        self.proj_down = nn.Parameter(torch.empty(in_features, rank, dtype=torch_dtype, device=device))
        self.proj_up = nn.Parameter(torch.empty(out_features, rank, dtype=torch_dtype, device=device))

        self.wtscale = None
        self.wcscales = None
        if precision == "nvfp4":
            self.wtscale = nn.Parameter(torch.ones(1, dtype=torch_dtype, device=device), requires_grad=False)
            self.wcscales = nn.Parameter(torch.ones(out_features, dtype=torch_dtype, device=device), requires_grad=False)

        self.act_unsigned = act_unsigned
        # one factor per 16 ranks of the low-rank branch (src/Linear.h:98); None: all ones
        self.lora_scales: list[float] | None = None
        self._native: dict[str, torch.Tensor | None] | None = None
        self._native_stamp: tuple | None = None
        self._alpha: float | None = None
        self._call: _LayerCall | None = None

    @classmethod
    def from_linear(cls, linear: nn.Linear, **kwargs):
        in_features = kwargs.pop("in_features", linear.in_features)
        return cls(
            in_features=in_features,
            out_features=linear.out_features,
            bias=linear.bias is not None,
            torch_dtype=linear.weight.dtype,
            device=linear.weight.device,
            **kwargs,
        )

    # ---- load-time repack -------------------------------------------------------------------
    def _load_from_state_dict(self, *args, **kwargs):
        self.invalidate_native()  # new checkpoint tensors: convert again on next use
        return super()._load_from_state_dict(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self.invalidate_native()
        return super()._apply(fn, *args, **kwargs)

    _NATIVE_SOURCES = ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias", "wcscales", "wtscale")

    def _stamp(self) -> tuple:
        """Identity and in-place modification counter of every parameter the native tensors come from."""
        params = self._parameters  # (nn.Module.__getattr__ is a slow way to the same dictionary)
        out = []
        for name in self._NATIVE_SOURCES:
            t = params.get(name)
            out.append(None if t is None else (t.data_ptr(), packing.tensor_version(t)))
        return tuple(out)

    def invalidate_native(self) -> None:
        """Forget the converted tensors (and the cached ``alpha``): the next use converts again.  Needed
        only after writes that leave no trace on the parameters (``param.data.copy_(...)``, or any write
        to inference-mode tensors); in-place operations on the parameters themselves, ``load_state_dict``
        and ``.to()`` are noticed without it."""
        self._native = None
        self._native_stamp = None
        self._alpha = None
        self._call = None

    def native_tensors(self) -> dict[str, torch.Tensor | None]:
        """The layer's tensors in the layouts the kernels read, converted on first use and again after
        a parameter has been replaced or modified in place (a low-rank swap, for example)."""
        stamp = self._stamp()
        if self._native is not None and stamp != self._native_stamp:
            self.invalidate_native()
        if self._native is None:
            self._native_stamp = stamp
            fp4 = self.precision == "nvfp4"
            self._native = {
                "qweight": packing.repack_qweight(self.qweight.data, fp4),
                "wscales": packing.repack_wscales(self.wscales.data, fp4),
                "smooth_factor": packing.repack_smooth(self.smooth_factor.data),
                "proj_down": packing.repack_lora_down(self.proj_down.data),
                "proj_up": packing.repack_lora_up(self.proj_up.data),
                "bias": None if self.bias is None else packing.repack_vector(self.bias.data),
                "wcscales": None if self.wcscales is None else packing.repack_vector(self.wcscales.data),
            }
            if fp4 and self.rank:
                packing.require_nonzero(self._native["wcscales"], "wcscales")
        return self._native

    # ---- low-rank hot swap ---------------------------------------------------------------------
    def update_lora(self, proj_down: torch.Tensor, proj_up: torch.Tensor) -> None:
        """Replace the low-rank branch by ``proj_down`` [K, R'] / ``proj_up`` [N, R'] (reference packed order,
        e.g. the layer's own branch with a user LoRA's ranks appended, ``checkpoint.concat_lowrank``).  The
        rank may change; the per-16-rank factors start again at one (GEMM_W4A4::loadParam,
        src/Linear.cpp:124-134)."""
        if proj_down.shape[0] != self.in_features or proj_up.shape[0] != self.out_features or proj_down.shape[1] != proj_up.shape[1]:
            raise ValueError(f"expected proj_down [{self.in_features}, R] and proj_up [{self.out_features}, R], got {tuple(proj_down.shape)} and {tuple(proj_up.shape)}")
        if proj_down.shape[1] % 16 != 0 or proj_down.shape[1] > 1024:
            raise ValueError("the rank must be a multiple of 16, at most 1024 (the reference's MAX_RANK, lora.cuh:22)")
        dev, dt = self.proj_down.device, self.proj_down.dtype
        self.proj_down = nn.Parameter(proj_down.detach().to(device=dev, dtype=dt).contiguous(), requires_grad=False)
        self.proj_up = nn.Parameter(proj_up.detach().to(device=dev, dtype=dt).contiguous(), requires_grad=False)
        self.rank = proj_down.shape[1]
        self.lora_scales = None
        self.invalidate_native()

    def set_lora_scale(self, skip_ranks: int, scale: float) -> None:
        """Factor ``scale`` on every rank behind the first ``skip_ranks`` (the layer's own branch keeps 1):
        QuantizedFluxModel::setLoraScale, nunchaku/csrc/flux.h:177-196."""
        if skip_ranks % 16 != 0:
            raise ValueError("skip_ranks must be a multiple of 16")
        groups = (self.rank + 15) // 16
        self.lora_scales = [1.0 if i < skip_ranks // 16 else float(scale) for i in range(groups)]
        self._call = None

    @property
    def alpha(self) -> float:
        """Per-tensor weight scale as a host float, read once (the reference hands the parameter to a
        ``float`` argument on every call, nunchaku/models/linear.py:128, which synchronises)."""
        self.native_tensors()  # (drops a stale value when wtscale was modified)
        if self._alpha is None:
            self._alpha = 1.0 if self.wtscale is None else float(self.wtscale.detach().float().cpu().item())
        return self._alpha

    # ---- forward path (nunchaku/models/linear.py:89-132) ----------------------------------------
    def forward(self, x: torch.Tensor, output: torch.Tensor | None = None) -> torch.Tensor:
        """``quantize`` then ``forward_quant`` (nunchaku/models/linear.py:89-110), through argument blocks prepared
        once per layer: a forward costs the host four allocations and two calls into the library."""
        batch_size, seq_len, channels = x.shape
        M = batch_size * seq_len
        x = x.view(M, channels)
        if M == 0:
            return self._forward_by_operators(x, output).view(batch_size, seq_len, -1)
        c = self._prepared(x)
        dev = c.device
        if output is None:
            output = torch.empty(M, self.out_features, dtype=x.dtype, device=dev)
        elif not (output.is_cuda and output.device == dev and output.dtype == torch.bfloat16 and output.is_contiguous()
                  and output.numel() == M * self.out_features and output.shape[-1] == self.out_features):
            raise ValueError(f"output must be a contiguous bf16 tensor of {M} x {self.out_features} elements on {dev}")
        M_pad = (M + 255) // 256 * 256
        qx, ascales, lora_act = self._quantize_prepared(c, x, M_pad)
        self._gemm_prepared(c, qx, ascales, lora_act, M_pad, out=output.data_ptr(), M_out=M)
        return output.view(batch_size, seq_len, -1)

    # The three steps of ``forward``, also used by ``ops.fused``: no argument is checked twice, none is looked up twice.
    def _prepared(self, x: torch.Tensor) -> _LayerCall:
        """Checks the activations ``x`` [M, K] against the layer and returns the layer's argument blocks."""
        if not x.is_cuda:
            raise RuntimeError(f"x must live on a GPU (got {x.device}); this path has no CPU implementation")
        if not x.is_contiguous():
            raise ValueError("x must be contiguous")
        if x.dtype != torch.bfloat16:
            raise NotImplementedError("only bf16 activations are supported")
        if x.shape[-1] != self.in_features:
            raise ValueError(f"x has {x.shape[-1]} channels, the layer takes {self.in_features}")
        return self._blocks(x.device)

    def _blocks(self, dev: torch.device) -> _LayerCall:
        t = self.native_tensors()
        c = self._call
        if c is None:
            c = self._call = _LayerCall(self, t)
        if c.device != dev:
            raise ValueError(f"the activations are on {dev}, the layer on {c.device}")
        return c

    def _quantize_prepared(self, c: _LayerCall, x: torch.Tensor, M_pad: int):
        dev = c.device
        qx = torch.empty(M_pad, c.act_bytes, dtype=torch.uint8, device=dev)
        ascales = torch.empty(c.groups, M_pad, dtype=c.scale_dtype, device=dev)
        lora_act = torch.empty(M_pad, self.rank, dtype=torch.float32, device=dev)
        with c.lock:
            q = c.q
            q.input, q.output, q.oscales = x.data_ptr(), qx.data_ptr(), ascales.data_ptr()
            q.lora_act_out = lora_act.data_ptr() if self.rank else None
            q.M, q.M_pad = x.shape[0], M_pad
            nv.launch(nv.lib().svdq_quantize_w4a4_act_fuse_lora, c.q_ref, dev)
        return qx, ascales, lora_act

    def _gemm_prepared(self, c: _LayerCall, qx: torch.Tensor, ascales: torch.Tensor, lora_act: torch.Tensor, M_pad: int,
                       out: int | None = None, M_out: int = 0, **epilogue) -> None:
        """The layer's GEMM on quantized activations made for it (``_quantize_prepared``, or another layer's
        next-layer epilogue).  ``out``: address of a bf16 [M_out, N] buffer.  ``epilogue``: further fields of the
        argument block (addresses and sizes), in force for this call only."""
        lib = nv.lib()
        with c.lock:
            g = c.g
            ls = self.lora_scales
            if ls is not None or c.scales_src is not None:  # one factor per 16 ranks; missing entries count as zero, None as all ones
                for i in range(len(c.sc)):
                    c.sc[i] = 1.0 if ls is None else (float(ls[i]) if i < len(ls) else 0.0)
                c.scales_src = ls
            g.act, g.ascales, g.out = qx.data_ptr(), ascales.data_ptr(), out
            g.lora_act_in = lora_act.data_ptr() if self.rank else None
            g.M_pad, g.M_out = M_pad, M_out
            g.k_split = int(_gemm_op.K_SPLIT or 0)
            for name, value in epilogue.items():
                setattr(g, name, value)
            try:
                nv.launch(lib.svdq_gemm_w4a4_noalloc if _gemm_op.NO_ALLOC else lib.svdq_gemm_w4a4, c.g_ref, c.device)
            finally:
                for name in epilogue:
                    setattr(g, name, 0 if name in ("R_down",) else None)

    def _forward_by_operators(self, x: torch.Tensor, output: torch.Tensor | None) -> torch.Tensor:
        """The same through the two operator wrappers (every argument checked on every call)."""
        quantized_x, ascales, lora_act_out = self.quantize(x)
        return self.forward_quant(quantized_x, ascales, lora_act_out, output)

    def quantize(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        t = self.native_tensors()
        return svdq_quantize_w4a4_act_fuse_lora(
            x, lora_down=t["proj_down"], smooth=t["smooth_factor"], fp4=self.precision == "nvfp4"
        )

    def forward_quant(
        self,
        quantized_x: torch.Tensor,
        ascales: torch.Tensor,
        lora_act: torch.Tensor,
        output: torch.Tensor | None = None,
    ) -> torch.Tensor:
        if output is None:
            output = torch.empty(quantized_x.shape[0], self.out_features, dtype=self.proj_up.dtype, device=quantized_x.device)
        t = self.native_tensors()
        svdq_gemm_w4a4(
            act=quantized_x, wgt=t["qweight"], out=output, ascales=ascales, wscales=t["wscales"],
            lora_act_in=lora_act, lora_up=t["proj_up"], bias=t["bias"], fp4=self.precision == "nvfp4",
            alpha=self.alpha, wcscales=t["wcscales"], act_unsigned=self.act_unsigned, lora_scales=self.lora_scales,
        )
        return output

    def __repr__(self):
        return (
            f"SVDQW4A4Linear(in_features={self.in_features}, out_features={self.out_features}, rank={self.rank}, "
            f"precision={self.precision}, act_unsigned={self.act_unsigned})"
        )


class AWQW4A16Linear(nn.Module):
    """AWQ W4A16 linear for a handful of rows (modulation layers, text encoder), parameters as in
    nunchaku/models/linear.py:138-208: qweight int32 [N/4, K/2], wscales / wzeros bf16 [K/G, N], bias
    bf16 [N]; the tensors are used in the reference's storage as they are."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, group_size: int = 64,
                 torch_dtype: torch.dtype = torch.bfloat16, device: str | torch.device | None = None):
        super().__init__()
        if device is None:
            device = torch.device("cpu")
        self.in_features, self.out_features, self.group_size = in_features, out_features, group_size
        self.qweight = nn.Parameter(torch.empty(out_features // 4, in_features // 2, dtype=torch.int32, device=device), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(out_features, dtype=torch_dtype, device=device), requires_grad=True) if bias else None
        self.wscales = nn.Parameter(torch.empty(in_features // group_size, out_features, dtype=torch_dtype, device=device), requires_grad=False)
        self.wzeros = nn.Parameter(torch.empty(in_features // group_size, out_features, dtype=torch_dtype, device=device), requires_grad=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        from ..ops.gemv import awq_gemv_w4a16

        x = x.contiguous()
        return awq_gemv_w4a16(
            in_feats=x, kernel=self.qweight, scaling_factors=self.wscales, zeros=self.wzeros,
            m=x.numel() // x.shape[-1], n=self.out_features, k=self.in_features, group_size=self.group_size,
            bias=None if self.bias is None else self.bias.detach(),
        )

    @classmethod
    def from_linear(cls, linear: nn.Linear, group_size: int = 64, torch_dtype: torch.dtype = torch.bfloat16, device: str = "cpu", **kwargs):
        return cls(linear.in_features, linear.out_features, bias=linear.bias is not None, group_size=group_size,
                   torch_dtype=torch_dtype, device=device)

    def __repr__(self):
        return f"AWQW4A16Linear(in_features={self.in_features}, out_features={self.out_features}, group_size={self.group_size})"
