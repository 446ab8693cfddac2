"""Small helpers shared by the operator wrappers (counterparts of nunchaku/utils.py:77-95,153-194)."""


def ceil_divide(x: int, divisor: int) -> int:
    """nunchaku/utils.py:77."""
    return (x + divisor - 1) // divisor


def get_precision(precision: str = "auto", device=None, pretrained_model_name_or_path=None) -> str:
    """Which 4-bit format to run (nunchaku/utils.py:153-194 picks it from the NVIDIA SM version).
    On gfx950 the INT4 path is the default; NVFP4 is available on request."""
    assert precision in ("auto", "int4", "fp4", "nvfp4")
    if precision == "auto":
        return "int4"
    return "nvfp4" if precision in ("fp4", "nvfp4") else "int4"
