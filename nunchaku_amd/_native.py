"""ctypes binding of ``libsvdq_amd.so`` (the C ABI declared in ``include/svdq_amd.h``) and the
tensor-level helpers built on it.

PyTorch is only used for device memory and streams: every call passes raw device pointers, sizes
and the current HIP stream.  There is no fallback path: if the library is missing, or a tensor is
not on a GPU, the call raises.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import torch

_PKG_DIR = Path(__file__).resolve().parent
_CSRC = _PKG_DIR / "csrc"
LIB_PATH = _PKG_DIR / "libsvdq_amd.so"
SOURCES = ["repack.hip", "quantize.hip", "gemm.hip", "awq_gemv.hip", "litela.hip"]
HIPCC_FLAGS = [
    "-shared", "-fPIC", "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

SVDQ_ABI_VERSION = 5
EXPORTED_SYMBOLS = [
    "svdq_abi_version", "svdq_last_error",
    "svdq_repack_qweight", "svdq_repack_wscales", "svdq_repack_wmscales", "svdq_repack_vector",
    "svdq_repack_smooth", "svdq_repack_lora_down", "svdq_repack_lora_up", "svdq_repack_rotemb",
    "svdq_quantize_w4a4_act_fuse_lora", "svdq_gemm_w4a4", "svdq_gemm_w4a4_noalloc", "svdq_awq_gemv_w4a16",
    "svdq_linearattn_vk_mul_q", "svdq_release_workspaces",
]


class QuantizeArgs(ctypes.Structure):
    """Mirror of ``svdq_quantize_args``."""

    _fields_ = [
        ("input", ctypes.c_void_p), ("output", ctypes.c_void_p), ("oscales", ctypes.c_void_p),
        ("lora_down", ctypes.c_void_p), ("lora_act_out", ctypes.c_void_p), ("smooth_rcp", ctypes.c_void_p),
        ("M", ctypes.c_int64), ("M_pad", ctypes.c_int64), ("K", ctypes.c_int64), ("R", ctypes.c_int64),
        ("fp4", ctypes.c_int32), ("fuse_glu", ctypes.c_int32),
    ]


class GemmArgs(ctypes.Structure):
    """Mirror of ``svdq_gemm_args``."""

    _fields_ = [
        ("act", ctypes.c_void_p), ("ascales", ctypes.c_void_p), ("wgt", ctypes.c_void_p),
        ("wscales", ctypes.c_void_p), ("colnorm", ctypes.c_void_p), ("bias", ctypes.c_void_p),
        ("wcscales", ctypes.c_void_p), ("lora_act_in", ctypes.c_void_p), ("lora_up", ctypes.c_void_p),
        ("lora_scales", ctypes.POINTER(ctypes.c_float)), ("out", ctypes.c_void_p),
        ("qout", ctypes.c_void_p), ("oscales", ctypes.c_void_p), ("next_smooth_rcp", ctypes.c_void_p),
        ("next_lora_down", ctypes.c_void_p), ("next_lora_act_out", ctypes.c_void_p),
        ("M_pad", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
        ("M_out", ctypes.c_int64), ("N_out", ctypes.c_int64),
        ("R_up", ctypes.c_int64), ("R_down", ctypes.c_int64),
        ("alpha", ctypes.c_float), ("act_unsigned", ctypes.c_int32), ("fuse_silu", ctypes.c_int32),
        ("fp4", ctypes.c_int32),
        ("norm_q", ctypes.c_void_p), ("norm_k", ctypes.c_void_p), ("rotary_emb", ctypes.c_void_p),
        ("rot_rows", ctypes.c_int64), ("norm_eps", ctypes.c_float), ("k_split", ctypes.c_int32),
        ("out_q", ctypes.c_void_p), ("out_k", ctypes.c_void_p), ("out_v", ctypes.c_void_p),
        ("qkv_head_stride", ctypes.c_int64 * 3), ("attn_tokens", ctypes.c_int64), ("qkv_rows", ctypes.c_int64),
        ("out_vk", ctypes.c_void_p), ("vk_rows", ctypes.c_int64),
    ]


class AwqGemvArgs(ctypes.Structure):
    """Mirror of ``svdq_awq_gemv_args``."""

    _fields_ = [
        ("x", ctypes.c_void_p), ("qweight", ctypes.c_void_p), ("scales", ctypes.c_void_p), ("zeros", ctypes.c_void_p),
        ("bias", ctypes.c_void_p), ("out", ctypes.c_void_p),
        ("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64), ("group_size", ctypes.c_int32),
    ]


# kernel variants, one translation unit each (-DSVDQ_VARIANT=n): the INT4 GEMM (gemm6_variant.hip: plain /
# next-layer epilogue) and the NVFP4 GEMM (gemm_variant.hip: the same two)
GEMM_VARIANT_UNITS = [("gemm6_variant.hip", 0), ("gemm6_variant.hip", 1), ("gemm_variant.hip", 4), ("gemm_variant.hip", 5)]


def build(verbose: bool = False, extra_flags: tuple[str, ...] = (), lib_path: Path | None = None) -> Path:
    """Compile the HIP sources for gfx950 into ``libsvdq_amd.so`` next to this file (hipcc
    cross-compiles; no GPU is needed).  Translation units are compiled in parallel, then linked."""
    import concurrent.futures
    import tempfile

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    flags = [f for f in HIPCC_FLAGS if f != "-shared"] + list(extra_flags)
    out = Path(lib_path) if lib_path else LIB_PATH
    with tempfile.TemporaryDirectory(prefix="svdq_build_") as tmp:
        jobs = [([str(_CSRC / src)], Path(tmp) / (src + ".o")) for src in SOURCES]
        jobs += [([str(_CSRC / src), f"-DSVDQ_VARIANT={v}"], Path(tmp) / f"{src}_{v}.o") for src, v in GEMM_VARIANT_UNITS]

        def compile_one(job):
            args, obj = job
            return subprocess.run([hipcc, *flags, "-c", *args, "-o", str(obj)], capture_output=True, text=True)

        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
            results = list(pool.map(compile_one, jobs))
        for (args, _), res in zip(jobs, results):
            if res.returncode != 0:
                raise RuntimeError(f"hipcc failed on {args}:\n" + res.stderr[-4000:])
        link = subprocess.run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *[str(o) for _, o in jobs], "-o", str(out)],
                              capture_output=True, text=True)
        if link.returncode != 0:
            raise RuntimeError("hipcc link failed:\n" + link.stderr[-4000:])
    if verbose:
        print(f"built {out}")
    return out


_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library.  Raises if it has not been built: there is no other implementation."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(the HIP extension is the only implementation of this path)"
            )
        L = ctypes.CDLL(str(LIB_PATH))
        L.svdq_abi_version.restype = ctypes.c_int
        L.svdq_last_error.restype = ctypes.c_char_p
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        L.svdq_repack_qweight.argtypes = [vp, vp, i64, i64, ci, vp]
        L.svdq_repack_wscales.argtypes = [vp, vp, i64, i64, vp]
        L.svdq_repack_wmscales.argtypes = [vp, vp, vp, i64, i64, vp]
        L.svdq_repack_vector.argtypes = [vp, vp, i64, vp]
        L.svdq_repack_smooth.argtypes = [vp, vp, i64, vp]
        L.svdq_repack_lora_down.argtypes = [vp, vp, i64, i64, vp]
        L.svdq_repack_lora_up.argtypes = [vp, vp, i64, i64, vp]
        L.svdq_repack_rotemb.argtypes = [vp, vp, i64, vp]
        L.svdq_quantize_w4a4_act_fuse_lora.argtypes = [ctypes.POINTER(QuantizeArgs), vp]
        L.svdq_gemm_w4a4.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.svdq_gemm_w4a4_noalloc.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.svdq_awq_gemv_w4a16.argtypes = [ctypes.POINTER(AwqGemvArgs), vp]
        L.svdq_linearattn_vk_mul_q.argtypes = [vp, vp, i64, i64, i64, i64, ctypes.c_float, vp]
        L.svdq_release_workspaces.argtypes = []
        for name in EXPORTED_SYMBOLS:
            getattr(L, name)
            if name not in ("svdq_last_error",):
                getattr(L, name).restype = ctypes.c_int if name != "svdq_last_error" else ctypes.c_char_p
        L.svdq_last_error.restype = ctypes.c_char_p
        if L.svdq_abi_version() != SVDQ_ABI_VERSION:
            raise RuntimeError("libsvdq_amd.so was built from a different header version; rebuild it")
        _lib = L
    return _lib


def check(rc: int) -> None:
    """Turn a C-ABI return code into the exception the reference's users expect."""
    if rc == 0:
        return
    msg = lib().svdq_last_error().decode()
    if rc == -1:
        raise ValueError(msg)
    if rc == -2:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def launch(entry, args_ref, device: torch.device) -> None:
    """Call ``entry(args, stream)`` of the C ABI on ``device``'s current stream.  The library launches on the
    current device: the switch (and torch's stream object) is only paid for when ``device`` is not current."""
    idx = device.index
    if idx is not None and idx == torch.cuda.current_device():
        rc = entry(args_ref, torch._C._cuda_getCurrentRawStream(idx))
    else:
        with torch.cuda.device(device):
            rc = entry(args_ref, torch.cuda.current_stream(device).cuda_stream)
    if rc:
        check(rc)


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on a GPU (got {t.device}); this path has no CPU implementation")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
