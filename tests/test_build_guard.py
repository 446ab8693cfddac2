"""What the hot kernels' performance and correctness rest on in the compiler's output, checked on the CPU (hipcc
cross-compiles gfx950 without a GPU).

* Registers.  ``g6::gemm6_kernel`` holds 128 accumulators per lane and runs two workgroups per compute unit: it must
  fit 256 vector registers without scratch.  A compiler that spills there costs time silently (spills of 236 and 518
  registers were seen while the kernel was written).  The NVFP4 kernel's figures are recorded with a ceiling.
* Flags across inline assembly.  The asynchronous global -> LDS copies are inline assembly that writes ``m0`` and, where
  it adds, the scalar condition code (SCC).  A build whose asm statements did not declare that had the compiler keep the
  carry of a 64-bit pointer addition (``s_add_u32`` ... ``s_addc_u32``) and the result of ``ng < 2`` in SCC across such
  a statement: the carry was lost whenever an operand tensor straddled a 4 GiB address boundary, and the kernel then
  read 4 GiB below its operands (a GPU memory fault that depended on where the allocator had placed the tensors).  The
  generated code is scanned: after an asm statement that writes SCC, nothing may read SCC before something else has
  written it.
* The 32-input fp6 conversion.  ``v_cvt_scalef32_2xpk16_fp6_f32`` writes result words while it still has inputs to
  read: with a destination that overlapped its sources across the end of the first one, the last two result words came
  out wrong on the GPU (one instantiation of the quantize kernel, found by comparing configurations).  The compiler
  does not know; the source issues the instruction through inline assembly with an early-clobber destination, and the
  generated code of every kernel that converts is scanned for overlapping registers.
"""

import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

import pytest

from nunchaku_amd import _native as nv

CSRC = Path(nv.__file__).resolve().parent / "csrc"

SCC_READERS = re.compile(r"^\s*(s_cbranch_scc[01]|s_cselect_b(32|64)|s_addc_u32|s_subb_u32|s_cmov_b(32|64))\b")
SCC_WRITERS = re.compile(
    r"^\s*(s_cmp_|s_cmpk_|s_add_[ui]32|s_sub_[ui]32|s_addk_|s_mulk_|s_and_|s_or_|s_xor_|s_andn2_|s_orn2_|s_nand_|s_nor_|s_xnor_|"
    r"s_lshl_b|s_lshr_b|s_ashr_i|s_bfe_|s_min_|s_max_|s_abs_|s_absdiff_|s_bitcmp|s_not_|s_wqm_|s_quadmask_|s_lshl[1-4]_add_|s_bcnt|"
    r"s_ff[01]_|s_flbit_)")
CONTROL = re.compile(r"^\s*(s_branch|s_cbranch_|s_endpgm|s_setpc_|s_swappc_)")


def compile_variant(src: str, variant: int, tmp: str):
    out = Path(tmp) / f"{src}_{variant}.s"
    flags = [f for f in nv.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    res = subprocess.run(["/opt/rocm/bin/hipcc", *flags, f"-DSVDQ_VARIANT={variant}", "-S", "--cuda-device-only",
                          "-Rpass-analysis=kernel-resource-usage", str(CSRC / src), "-o", str(out)], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    usage = {}
    name = None
    for line in res.stderr.splitlines():
        m = re.search(r"remark: .*Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            usage[name] = {}
        m = re.search(r"remark: .*?\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+)", line)
        if m and name and "Function Name" not in line:
            usage[name][m.group(1).strip()] = int(m.group(2))
    return usage, out.read_text().splitlines()


def scc_live_across_asm(lines):
    """(line number, text) of every SCC reader that follows an SCC-writing inline-asm statement with no SCC writer
    between them, in straight-line order; control flow or a label right behind such a statement is reported too (the
    compiler treats a declared clobber as a definition, so neither occurs in a correct build)."""
    bad = []
    i = 0
    while i < len(lines):
        if "#ASMSTART" in lines[i]:
            j = i
            while "#ASMEND" not in lines[j]:
                j += 1
            if any(SCC_WRITERS.match(b) for b in lines[i + 1:j]):
                k = j + 1
                while k < len(lines):
                    s = lines[k]
                    if SCC_READERS.match(s):
                        bad.append((k + 1, s.strip()))
                        break
                    if SCC_WRITERS.match(s) or "#ASMSTART" in s or CONTROL.match(s) or re.match(r"^\.LBB\d+_\d+:", s.strip()):
                        break
                    k += 1
            i = j
        i += 1
    return bad


def fp6_conversions_with_overlap(lines):
    """Every ``v_cvt_scalef32_2xpk16_fp6_f32`` whose destination registers overlap one of its two 16-register sources."""
    total, bad = 0, []
    for n, l in enumerate(lines):
        if "v_cvt_scalef32_2xpk16_fp6_f32" in l:
            m = re.search(r"v\[(\d+):(\d+)\], v\[(\d+):(\d+)\], v\[(\d+):(\d+)\]", l)
            assert m, l
            d0, d1, a0, a1, b0, b1 = map(int, m.groups())
            total += 1
            if not (d1 < a0 or d0 > a1) or not (d1 < b0 or d0 > b1):
                bad.append((n + 1, l.strip()))
    return total, bad


def test_fp6_conversion_never_overwrites_its_own_inputs():
    assert fp6_conversions_with_overlap(["\tv_cvt_scalef32_2xpk16_fp6_f32 v[14:19], v[2:17], v[18:33], s52"])[1]  # the form that failed
    assert not fp6_conversions_with_overlap(["\tv_cvt_scalef32_2xpk16_fp6_f32 v[34:39], v[2:17], v[18:33], s52"])[1]
    flags = [f for f in nv.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    with tempfile.TemporaryDirectory(prefix="svdq_guard_") as tmp:
        for src, extra in (("quantize.hip", []), ("gemm6_variant.hip", ["-DSVDQ_VARIANT=1"])):
            out = Path(tmp) / (src + ".s")
            res = subprocess.run(["/opt/rocm/bin/hipcc", *flags, *extra, "-S", "--cuda-device-only", str(CSRC / src), "-o", str(out)],
                                 capture_output=True, text=True)
            assert res.returncode == 0, res.stderr[-3000:]
            total, bad = fp6_conversions_with_overlap(out.read_text().splitlines())
            assert total > 0 and not bad, (src, bad[:3])


def test_scanner_finds_a_carry_kept_across_an_asm_add():
    bad = """
	s_add_u32 s26, s8, 0x1800
	;;#ASMSTART
	s_add_u32 m0, s44, s11
	s_nop 0
	global_load_lds_dwordx4 v1, s[6:7] offset:1024
	;;#ASMEND
	s_addc_u32 s27, s9, 0
""".splitlines()
    assert scc_live_across_asm(bad) == [(8, "s_addc_u32 s27, s9, 0")]
    good = """
	;;#ASMSTART
	s_add_u32 m0, s44, s11
	;;#ASMEND
	s_add_u32 s26, s8, 0x1800
	s_addc_u32 s27, s9, 0
""".splitlines()
    assert scc_live_across_asm(good) == []


def test_the_build_before_the_clobbers_were_declared_kept_flags_across_the_copies():
    """The sources as they were before the commit that declared what the copy statements overwrite (``07f9e0a``),
    taken from the repository's history and compiled with today's flags: the scanner finds condition-code values kept
    alive across copy statements there (the carry of a 64-bit source pointer among them) and none in today's sources
    (``test_no_condition_code_kept_across_inline_asm``).  Skipped where the history is not at hand."""
    root = CSRC.parents[1]
    old = "07f9e0a^"
    probe = subprocess.run(["git", "-C", str(root), "cat-file", "-e", f"{old}:nunchaku_amd/csrc/gemm6_kernel.h"], capture_output=True)
    if probe.returncode != 0:
        pytest.skip("no git history with the earlier sources here")
    flags = [f for f in nv.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    with tempfile.TemporaryDirectory(prefix="svdq_guard_old_") as tmp:
        tar = subprocess.run(["git", "-C", str(root), "archive", old, "nunchaku_amd/csrc", "include"], capture_output=True)
        assert tar.returncode == 0, tar.stderr[-500:]
        subprocess.run(["tar", "-x", "-C", tmp], input=tar.stdout, check=True)
        out = Path(tmp) / "old.s"
        res = subprocess.run(["/opt/rocm/bin/hipcc", *flags, "-DSVDQ_VARIANT=0", "-S", "--cuda-device-only",
                              str(Path(tmp) / "nunchaku_amd/csrc/gemm6_variant.hip"), "-o", str(out)], capture_output=True, text=True)
        assert res.returncode == 0, res.stderr[-3000:]
        bad = scc_live_across_asm(out.read_text().splitlines())
    print(bad)
    assert bad, "the earlier build shows no condition code kept across an inline-asm statement"
    assert any(text.startswith("s_addc_u32") for _, text in bad), bad  # a lost carry: the source pointer of a copy, 4 GiB too low


@pytest.fixture(scope="module")
def compiled():
    units = [("gemm6_variant.hip", 0), ("gemm6_variant.hip", 1), ("gemm_variant.hip", 4), ("gemm_variant.hip", 5)]
    with tempfile.TemporaryDirectory(prefix="svdq_guard_") as tmp:
        with ThreadPoolExecutor(max_workers=4) as pool:
            results = list(pool.map(lambda u: compile_variant(u[0], u[1], tmp), units))
    return dict(zip(units, results))


def kernel_usage(usage, fragment):
    hits = [v for k, v in usage.items() if fragment in k]
    assert len(hits) == 1, list(usage)
    return hits[0]


@pytest.mark.parametrize("variant", [0, 1])
def test_int4_gemm_fits_its_registers(compiled, variant):
    usage, _ = compiled[("gemm6_variant.hip", variant)]
    u = kernel_usage(usage, "gemm6_kernel")
    print(u)
    assert u["VGPRs"] <= 256 and u["AGPRs"] == 0, u
    assert u["ScratchSize"] == 0, f"gemm6_kernel spills: {u}"
    assert u["Occupancy"] >= 2, u


@pytest.mark.parametrize("variant,max_scratch", [(4, 48), (5, 256)])
def test_nvfp4_gemm_register_figures(compiled, variant, max_scratch):
    usage, _ = compiled[("gemm_variant.hip", variant)]
    u = kernel_usage(usage, "gemm_w4a4_kernel")
    print(u)
    assert u["VGPRs"] + u["AGPRs"] <= 512, u
    # the epilogue keeps some values in scratch; the main loop must not (a much larger figure means it does)
    assert u["ScratchSize"] <= max_scratch, u


@pytest.mark.parametrize("unit", [("gemm6_variant.hip", 0), ("gemm6_variant.hip", 1), ("gemm_variant.hip", 4), ("gemm_variant.hip", 5)])
def test_no_condition_code_kept_across_inline_asm(compiled, unit):
    _, lines = compiled[unit]
    assert sum("#ASMSTART" in l for l in lines) > 0
    assert scc_live_across_asm(lines) == []
