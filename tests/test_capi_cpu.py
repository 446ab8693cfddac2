"""Host-side checks that need no GPU: the shared library loads, exports every symbol the header
declares, and rejects bad arguments before launching anything."""

import ctypes
import re
from pathlib import Path

import pytest

from nunchaku_amd import _native as nv

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def lib():
    if not nv.LIB_PATH.exists():
        nv.build()
    return nv.lib()


def test_header_symbols_are_exported(lib):
    header = (ROOT / "include" / "svdq_amd.h").read_text()
    declared = set(re.findall(r"^(?:int|const char \*)\s*(svdq_\w+)\(", header, flags=re.M))
    assert declared == set(nv.EXPORTED_SYMBOLS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.svdq_abi_version() == nv.SVDQ_ABI_VERSION
    assert int(re.search(r"#define SVDQ_ABI_VERSION (\d+)", header).group(1)) == nv.SVDQ_ABI_VERSION


def test_struct_sizes_match_header_layout(tmp_path):
    """The ctypes mirrors against the header itself: a C program that includes it prints the size of every
    argument block and the offset of every field, compiled with the host compiler."""
    import re
    import shutil
    import subprocess
    from pathlib import Path

    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no host C compiler")
    header = Path(__file__).resolve().parent.parent / "include" / "svdq_amd.h"
    mirrors = {"svdq_quantize_args": nv.QuantizeArgs, "svdq_gemm_args": nv.GemmArgs, "svdq_awq_gemv_args": nv.AwqGemvArgs}
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{header}"', 'int main(void) {']
    for cname, mirror in mirrors.items():
        lines.append(f'printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, *_ in mirror._fields_:
            lines.append(f'printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    lines.append("return 0; }")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run([cc, str(src), "-o", str(exe)], check=True, capture_output=True)
    out = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, mirror in mirrors.items():
        assert int(out[cname]) == ctypes.sizeof(mirror), cname
        for fname, *_ in mirror._fields_:
            assert int(out[f"{cname}.{fname}"]) == getattr(mirror, fname).offset, f"{cname}.{fname}"
    # and no field of the header is missing from the mirror
    text = header.read_text()
    for cname, mirror in mirrors.items():
        body = text[text.index(f"typedef struct {cname}"):text.index(f"}} {cname};")]
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        names = re.findall(r"[\s\*]([A-Za-z_][A-Za-z0-9_]*)\s*(?:\[\d+\])?\s*[,;]", body)
        assert set(names) == {f[0] for f in mirror._fields_}, cname


def test_quantize_rejects_bad_arguments(lib):
    assert lib.svdq_quantize_w4a4_act_fuse_lora(None, None) == -1
    a = nv.QuantizeArgs()
    assert lib.svdq_quantize_w4a4_act_fuse_lora(ctypes.byref(a), None) == -1
    assert b"null" in lib.svdq_last_error()
    a = nv.QuantizeArgs(input=16, output=16, oscales=16, lora_down=16, lora_act_out=16, M=100, M_pad=200, K=256, R=32)
    assert lib.svdq_quantize_w4a4_act_fuse_lora(ctypes.byref(a), None) == -1
    assert b"M_pad" in lib.svdq_last_error()
    a.M_pad = 256
    a.K = 100
    assert lib.svdq_quantize_w4a4_act_fuse_lora(ctypes.byref(a), None) == -1
    assert b"K" in lib.svdq_last_error()
    a.K = 256
    a.R = 24
    assert lib.svdq_quantize_w4a4_act_fuse_lora(ctypes.byref(a), None) == -1
    a.R = 32
    a.input = 8  # misaligned
    assert lib.svdq_quantize_w4a4_act_fuse_lora(ctypes.byref(a), None) == -1
    assert b"aligned" in lib.svdq_last_error()
    a.input = 16
    a.R = 1040  # the reference's MAX_RANK is 1024 (lora.cuh:22)
    a.fuse_glu = 1
    assert lib.svdq_quantize_w4a4_act_fuse_lora(ctypes.byref(a), None) == -1
    assert b"rank" in lib.svdq_last_error()


def test_gemm_rejects_bad_arguments(lib):
    assert lib.svdq_gemm_w4a4(None, None) == -1
    a = nv.GemmArgs(act=16, ascales=16, wgt=16, wscales=16, colnorm=16, out=16, M_pad=256, N=128, K=128, M_out=256, N_out=128, alpha=1.0)
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.M_pad = 100
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.N = 100
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.out = None
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.lora_up = 16  # without lora_act_in
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.M_out = 300
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.fuse_silu = 1  # only with `out` alone
    bad.qout = 16
    bad.oscales = 16
    bad.next_smooth_rcp = 16
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -2
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.k_split = -1
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.fp4 = 1
    bad.colnorm = None  # NVFP4 needs the column factors of its repack
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.R_down = 32  # without next_lora_down / next_lora_act_out
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    # the norm + rotary epilogue: needs both norm weights, three equal parts of whole heads, enough table rows
    bad = nv.GemmArgs.from_buffer_copy(a)
    bad.norm_q = 16
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    bad.norm_k = 16
    bad.rotary_emb = 16
    bad.rot_rows = 256
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    assert b"three equal parts" in lib.svdq_last_error()
    bad.N = bad.N_out = 384
    bad.rot_rows = 128
    assert lib.svdq_gemm_w4a4(ctypes.byref(bad), None) == -1
    assert b"rows" in lib.svdq_last_error()


def test_awq_gemv_rejects_bad_arguments(lib):
    assert lib.svdq_awq_gemv_w4a16(None, None) == -1
    a = nv.AwqGemvArgs(x=16, qweight=16, scales=16, zeros=16, out=16, M=1, N=64, K=128, group_size=64)
    for field, value, code in (("M", 9, -1), ("M", 0, -1), ("N", 6, -1), ("K", 100, -1), ("group_size", 128, -2), ("x", 8, -1), ("out", None, -1)):
        bad = nv.AwqGemvArgs.from_buffer_copy(a)
        setattr(bad, field, value)
        assert lib.svdq_awq_gemv_w4a16(ctypes.byref(bad), None) == code, field


def test_repack_rejects_bad_arguments(lib):
    assert lib.svdq_repack_qweight(None, None, 128, 128, 0, None) == -1
    assert lib.svdq_repack_qweight(16, 32, 100, 128, 0, None) == -1
    assert lib.svdq_repack_qweight(16, 16, 128, 128, 0, None) == -1  # in place
    assert lib.svdq_repack_wscales(16, 32, 128, 100, None) == -1
    assert lib.svdq_repack_wscales(16, 40, 128, 128, None) == -1  # destination not 16-byte aligned
    assert lib.svdq_repack_vector(16, 32, 100, None) == -1
    assert lib.svdq_repack_smooth(16, 32, 64, None) == -1
    assert lib.svdq_repack_lora_down(16, 32, 128, 8, None) == -1
    assert lib.svdq_repack_lora_up(16, 32, 8, 16, None) == -1
    assert lib.svdq_repack_rotemb(16, 32, 48, None) == -1  # rows not a multiple of 32
    assert lib.svdq_repack_rotemb(16, 16, 64, None) == -1  # in place


def test_python_wrappers_refuse_cpu_tensors():
    import torch

    from nunchaku_amd.ops import svdq_gemm_w4a4, svdq_quantize_w4a4_act_fuse_lora

    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        svdq_quantize_w4a4_act_fuse_lora(x, lora_down=torch.zeros(128, 16, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        svdq_gemm_w4a4(act=x, wgt=x, poolout=x)
    with pytest.raises(RuntimeError, match="GPU"):
        svdq_gemm_w4a4(act=x.view(torch.uint8), wgt=x.view(torch.int8), ascales=x, wscales=x, out=x)


def test_module_mirrors_reference_parameters():
    import torch

    from nunchaku_amd.models.linear import SVDQW4A4Linear

    m = SVDQW4A4Linear(256, 384, rank=32)
    sd = m.state_dict()
    # names, shapes and dtypes of nunchaku/models/linear.py:38-72
    assert {k: (tuple(v.shape), v.dtype) for k, v in sd.items()} == {
        "qweight": ((384, 128), torch.int8),
        "bias": ((384,), torch.bfloat16),
        "wscales": ((4, 384), torch.bfloat16),
        "smooth_factor": ((256,), torch.bfloat16),
        "smooth_factor_orig": ((256,), torch.bfloat16),
        "proj_down": ((256, 32), torch.bfloat16),
        "proj_up": ((384, 32), torch.bfloat16),
    }
    m4 = SVDQW4A4Linear(256, 384, rank=16, precision="nvfp4", bias=False)
    sd4 = m4.state_dict()
    assert sd4["wscales"].dtype == torch.float8_e4m3fn and tuple(sd4["wscales"].shape) == (16, 384)
    assert "wtscale" in sd4 and "wcscales" in sd4 and "bias" not in sd4
    with pytest.raises(ValueError):
        SVDQW4A4Linear(256, 384, precision="int8")
    lin = torch.nn.Linear(256, 384, dtype=torch.bfloat16)
    assert SVDQW4A4Linear.from_linear(lin, rank=16).rank == 16


def test_gemm_wrapper_refuses_wrong_shapes(monkeypatch):
    """Every buffer the kernel walks over M_pad rows of is checked before anything is launched (an
    undersized one would be an out-of-bounds access on the device).  No GPU: the device check is
    switched off so that the shape checks are reached with CPU tensors."""
    import torch

    from nunchaku_amd import packing
    from nunchaku_amd.ops import gemm as gemm_mod

    monkeypatch.setattr(nv, "require_gpu", lambda t, name: None)

    def boom(*a, **k):
        raise AssertionError("reached the repack / launch")

    monkeypatch.setattr(packing, "native", boom)
    M_pad, K, N, R = 256, 128, 128, 16
    good = dict(
        act=torch.zeros(M_pad, K * 3 // 4, dtype=torch.uint8), wgt=torch.zeros(N, K // 2, dtype=torch.int8),
        ascales=torch.zeros(K // 64, M_pad, dtype=torch.bfloat16), wscales=torch.zeros(K // 64, N, dtype=torch.bfloat16),
        out=torch.zeros(M_pad, N, dtype=torch.bfloat16), lora_act_in=torch.zeros(M_pad, R), lora_up=torch.zeros(N, R, dtype=torch.bfloat16),
        bias=torch.zeros(N, dtype=torch.bfloat16),
    )
    with pytest.raises(AssertionError, match="reached"):
        gemm_mod.svdq_gemm_w4a4(**good)  # (the valid call gets as far as the repack)
    cases = {
        "act": torch.zeros(M_pad, K // 2, dtype=torch.uint8),           # the reference's 4-bit shape
        "ascales": torch.zeros(K // 64, 100, dtype=torch.bfloat16),     # unpadded
        "wscales": torch.zeros(K // 64, N + 1, dtype=torch.bfloat16),
        "lora_act_in": torch.zeros(100, R),                             # [M, R] instead of [M_pad, R]
        "lora_up": torch.zeros(N - 16, R, dtype=torch.bfloat16),
        "bias": torch.zeros(N, dtype=torch.float32),
    }
    for name, t in cases.items():
        with pytest.raises(ValueError, match=name):
            gemm_mod.svdq_gemm_w4a4(**{**good, name: t})
    nxt = dict(qout=torch.zeros(M_pad, N * 3 // 4, dtype=torch.uint8), oscales=torch.zeros(N // 64, M_pad, dtype=torch.bfloat16),
               smooth_factor=torch.ones(N, dtype=torch.bfloat16), lora_down=torch.zeros(N, R, dtype=torch.bfloat16), lora_act_out=torch.zeros(M_pad, R))
    for name, t in {"qout": torch.zeros(M_pad, N // 2, dtype=torch.uint8), "oscales": torch.zeros(N // 64, 128, dtype=torch.bfloat16),
                    "lora_act_out": torch.zeros(128, R), "smooth_factor": torch.ones(N - 1, dtype=torch.bfloat16)}.items():
        with pytest.raises(ValueError, match=name):
            gemm_mod.svdq_gemm_w4a4(**{**good, **nxt, name: t})


def test_quantize_wrapper_refuses_wrong_shapes(monkeypatch):
    import torch

    from nunchaku_amd.ops import svdq_quantize_w4a4_act_fuse_lora

    monkeypatch.setattr(nv, "require_gpu", lambda t, name: None)
    x = torch.zeros(100, 128, dtype=torch.bfloat16)
    down = torch.zeros(128, 16, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="output"):
        svdq_quantize_w4a4_act_fuse_lora(x, output=torch.zeros(256, 64, dtype=torch.uint8), lora_down=down)
    with pytest.raises(ValueError, match="oscales"):
        svdq_quantize_w4a4_act_fuse_lora(x, oscales=torch.zeros(2, 100, dtype=torch.bfloat16), lora_down=down)
    with pytest.raises(ValueError, match="lora_act_out"):
        svdq_quantize_w4a4_act_fuse_lora(x, lora_act_out=torch.zeros(100, 16), lora_down=down)
    with pytest.raises(ValueError, match="lora_down"):
        svdq_quantize_w4a4_act_fuse_lora(x, lora_down=torch.zeros(64, 16, dtype=torch.bfloat16))


def test_repack_cache_follows_modifications(monkeypatch):
    """The cache of repacked reference tensors: hit while the source is unchanged, redone after an
    in-place operation, and tensors without a version counter (inference mode) are never cached."""
    import torch

    from nunchaku_amd import packing

    calls = []

    def fake(t):
        calls.append(t)
        return t.clone()

    monkeypatch.setitem(packing._REPACKERS, "vector", fake)
    t = torch.ones(128, dtype=torch.bfloat16)
    a = packing.native(t, "vector")
    assert packing.native(t, "vector") is a and len(calls) == 1
    t.add_(1)
    assert packing.native(t, "vector") is not a and len(calls) == 2
    with torch.inference_mode():
        u = torch.ones(128, dtype=torch.bfloat16)
    assert packing.tensor_version(u) is None
    packing.native(u, "vector")
    packing.native(u, "vector")
    assert len(calls) == 4


def test_module_reconverts_after_a_parameter_changes(monkeypatch):
    """A low-rank swap or any other in-place update of a parameter is picked up by the next forward."""
    import torch

    from nunchaku_amd import packing
    from nunchaku_amd.models.linear import SVDQW4A4Linear

    count = {"n": 0}

    def fake(t, *a):
        count["n"] += 1
        return t.clone()

    for name in ("repack_qweight", "repack_wscales", "repack_smooth", "repack_lora_down", "repack_lora_up", "repack_vector"):
        monkeypatch.setattr(packing, name, fake)
    m = SVDQW4A4Linear(128, 128, rank=16)
    for p in m.parameters():
        p.data.zero_()
    m.native_tensors()
    n0 = count["n"]
    assert m.native_tensors() is m.native_tensors() and count["n"] == n0
    with torch.no_grad():
        m.proj_up.add_(1)  # in place: the version counter moves
    m.native_tensors()
    assert count["n"] == 2 * n0
    m.proj_up = torch.nn.Parameter(torch.zeros(128, 32, dtype=torch.bfloat16))  # replaced (rank growth)
    m.native_tensors()
    assert count["n"] == 3 * n0
    m.proj_up.data.copy_(torch.ones(128, 32))  # leaves no trace: needs the explicit call
    m.native_tensors()
    assert count["n"] == 3 * n0
    m.invalidate_native()
    m.native_tensors()
    assert count["n"] == 4 * n0
