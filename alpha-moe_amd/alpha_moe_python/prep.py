"""Caller-side input preparation for ``fused_moe_w8a8_up_down``.

The reference takes these three steps from SGLang, which is not part of its
tree: ``sglang_per_token_group_quant_fp8`` (jit_moe.py:142),
``moe_align_block_size`` (jit_moe.py:158) and the checkpoint's 128x128
block-quantised weights.  They are restated here with plain torch tensor ops
so callers, the autotuner and the benchmarks need nothing outside this
package; they run on whatever device their inputs live on.

The contracts are the ones the fused kernel consumes
(fused_moe_w8a8_up_down_acc.cu:676-679, 756-758, 793, 800-807, 857).
"""
from typing import Tuple

import torch

FP8_MAX = 448.0
GROUP = 128
AMAX_FLOOR = 1e-10


def per_token_group_quant_fp8(x: torch.Tensor, group_size: int = GROUP) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantise ``x [M, K]`` to FP8 e4m3 with one fp32 scale per token per ``group_size`` columns.

    ``scale = max(amax, 1e-10) / 448``; ``q = fp8_rne(clamp(x / scale, -448, 448))``.
    Returns ``(q [M, K] float8_e4m3fn, scale [M, K/group_size] float32)``.
    """
    if x.dim() != 2 or x.shape[1] % group_size != 0:
        raise ValueError(f"x must be [M, K] with K % {group_size} == 0, got {tuple(x.shape)}")
    M, K = x.shape
    xf = x.float().reshape(M, K // group_size, group_size)
    amax = xf.abs().amax(dim=-1, keepdim=True).clamp_min(AMAX_FLOOR)
    scale = amax / FP8_MAX
    q = (xf / scale).clamp_(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.reshape(M, K), scale.reshape(M, K // group_size).contiguous()


def block_quant_fp8(w: torch.Tensor, block: int = GROUP) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantise ``w [..., R, C]`` to FP8 e4m3 with one fp32 scale per ``block x block`` tile.

    Returns ``(q [..., R, C] float8_e4m3fn, scale [..., R/block, C/block] float32)``.
    """
    R, C = w.shape[-2:]
    if R % block or C % block:
        raise ValueError(f"last two dims {R}x{C} must be multiples of {block}")
    lead = w.shape[:-2]
    t = w.float().reshape(*lead, R // block, block, C // block, block)
    amax = t.abs().amax(dim=(-3, -1), keepdim=True).clamp_min(AMAX_FLOOR)
    scale = amax / FP8_MAX
    q = (t / scale).clamp_(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.reshape(*lead, R, C), scale.reshape(*lead, R // block, C // block).contiguous()


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """Group routing slots by expert and pad every expert's segment to a multiple of ``block_size``.

    ``topk_ids [M, top_k]`` holds the expert of each (token, slot).  Returns

    * ``sorted_token_ids`` int32 ``[numel + num_experts*(block_size-1)]``: flat
      slot ids ``t*top_k + s`` in ascending expert order, ascending flat id
      within an expert (stable), padding entries equal to ``numel``;
    * ``expert_ids`` int32 ``[ceil(len(sorted_token_ids)/block_size)]``: expert of
      each block, ``-1`` for blocks past the padded total;
    * ``num_tokens_post_padded`` int32 ``[1]``: the padded total.

    Experts without tokens take no block.
    """
    if topk_ids.dim() != 2:
        raise ValueError("topk_ids must be [M, top_k]")
    if block_size <= 0 or num_experts <= 0:
        raise ValueError("block_size and num_experts must be positive")
    dev = topk_ids.device
    flat = topk_ids.reshape(-1).to(torch.int64)
    numel = flat.numel()
    # value check only where it costs no device synchronisation
    if numel and dev.type == "cpu" and (int(flat.min()) < 0 or int(flat.max()) >= num_experts):
        raise ValueError("topk_ids holds an expert outside [0, num_experts)")
    sorted_num = numel + num_experts * (block_size - 1)
    n_blocks = (sorted_num + block_size - 1) // block_size

    counts = torch.bincount(flat, minlength=num_experts)
    padded = (counts + block_size - 1) // block_size * block_size
    pad_end = torch.cumsum(padded, 0)
    pad_start = pad_end - padded
    start = torch.cumsum(counts, 0) - counts

    order = torch.argsort(flat, stable=True)
    experts_sorted = flat[order]
    rank_in_expert = torch.arange(numel, device=dev) - start[experts_sorted]
    sorted_token_ids = torch.full((sorted_num,), numel, dtype=torch.int32, device=dev)
    sorted_token_ids[pad_start[experts_sorted] + rank_in_expert] = order.to(torch.int32)

    block_start = torch.arange(n_blocks, device=dev) * block_size
    expert_ids = torch.searchsorted(pad_end, block_start, right=True)
    expert_ids = torch.where(block_start < pad_end[-1], expert_ids, torch.full_like(expert_ids, -1)).to(torch.int32)
    num_tokens_post_padded = pad_end[-1:].to(torch.int32)
    return sorted_token_ids, expert_ids, num_tokens_post_padded
