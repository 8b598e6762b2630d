"""GPU input preparation for ``fused_moe_w8a8_up_down``: the HIP kernels behind
``torch.ops.alpha_moe.per_token_group_quant_fp8`` and ``torch.ops.alpha_moe.moe_align_block_size``.

Same names, arguments and results as the torch restatements in ``alpha_moe_python.prep`` (and as the SGLang functions
the reference's callers use, jit_moe.py:142,158), bit for bit; these run as one to three small kernels on the current
stream and need the built extension.
"""
from typing import Tuple

import torch

import alpha_moe  # noqa: F401  (registers the operators; fails if the libraries are not built)


def per_token_group_quant_fp8(x: torch.Tensor, group_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """``x [M, K]`` bf16 or fp32 on the GPU -> ``(q [M, K] float8_e4m3fn, scale [M, K/128] float32)``."""
    return torch.ops.alpha_moe.per_token_group_quant_fp8(x, group_size)


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """``topk_ids [M, top_k]`` int32 on the GPU -> ``(sorted_token_ids, expert_ids, num_tokens_post_padded)``."""
    if topk_ids.dtype != torch.int32:
        topk_ids = topk_ids.to(torch.int32)
    return torch.ops.alpha_moe.moe_align_block_size(topk_ids.contiguous(), block_size, num_experts)
