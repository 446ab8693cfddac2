"""Operator wrappers with the signatures of ``nunchaku.ops`` (nunchaku/ops/{quantize,gemm,fused}.py)."""

from .fused import fused_gelu_mlp, fused_qkv_norm_rottary, linearattn_vk_mul_q
from .gemm import svdq_gemm_w4a4, svdq_gemm_w4a4_cuda
from .gemv import awq_gemv_w4a16, awq_gemv_w4a16_cuda
from .quantize import svdq_quantize_w4a4_act_fuse_lora, svdq_quantize_w4a4_act_fuse_lora_cuda

__all__ = [
    "svdq_quantize_w4a4_act_fuse_lora",
    "svdq_quantize_w4a4_act_fuse_lora_cuda",
    "svdq_gemm_w4a4",
    "svdq_gemm_w4a4_cuda",
    "awq_gemv_w4a16",
    "awq_gemv_w4a16_cuda",
    "fused_gelu_mlp",
    "fused_qkv_norm_rottary",
    "linearattn_vk_mul_q",
]
