"""MI355X (gfx950) implementation of Nunchaku's SVDQuant W4A4 + low-rank linear path.

Mirrors ``nunchaku.ops`` (``svdq_quantize_w4a4_act_fuse_lora``, ``svdq_gemm_w4a4``,
``fused_gelu_mlp``) and ``nunchaku.models.linear.SVDQW4A4Linear``; the math runs in hand-written
HIP kernels behind the C ABI of ``include/svdq_amd.h``.
"""

__version__ = "0.1.0"

from .utils import ceil_divide, get_precision  # noqa: F401
