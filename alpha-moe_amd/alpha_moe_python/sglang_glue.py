"""What an SGLang-on-ROCm build calls to run its fused-MoE layers through this operator.

The reference wires itself into SGLang with a patch (extra/sglang.patch: the weight loader interleaves ``w13`` and
its block scales once both halves of an expert have arrived, lines 46-98; ``fused_experts_impl`` is short-circuited
into quantise -> align -> operator, lines 1-44).  ``extra/sglang_rocm.patch`` of this repository is the same wiring
for a ROCm build, and keeps the logic here so that it can be exercised without SGLang:

* :class:`W13Interleaver` - the weight-loader bookkeeping;
* :func:`fused_experts`   - the forward path, with this library's own HIP quantiser and aligner in place of SGLang's
  helpers and the storing variant of the operator in place of zero-fill + add.
"""
import os
from typing import Optional

import torch

from .utils import get_best_config, interleave_tensor


class W13Interleaver:
    """Counts the gate (``w1``) and up (``w3``) shards an expert's fused ``w13`` slot has received and, once both are
    there, rewrites the slot in the operator's interleaved row order - chunks of 8 rows for weights, of 1 row for
    128x128 block scales (reference extra/sglang.patch:71-78,87-94)."""

    def __init__(self, num_experts: int, rep: int):
        self.rep = rep
        self.halves_loaded = [0] * num_experts

    def shard_loaded(self, expert_data: torch.Tensor, expert_id: int, shard_id: str) -> bool:
        """Call after the loader has copied ``shard_id`` into ``expert_data`` (the expert's ``[N, K]`` slot of the
        parameter).  Returns True when this call interleaved the slot."""
        if shard_id not in ("w1", "w3", "w13"):
            return False
        self.halves_loaded[expert_id] += 2 if shard_id == "w13" else 1
        if self.halves_loaded[expert_id] != 2:
            return False
        expert_data.copy_(interleave_tensor(expert_data.unsqueeze(0), self.rep)[0])
        return True


def fused_experts(hidden_states: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, topk_weights: torch.Tensor,
                  topk_ids: torch.Tensor, w13_scale: torch.Tensor, w2_scale: torch.Tensor,
                  routed_scaling_factor: Optional[float] = None, config_path: Optional[str] = None,
                  group_size: int = 128) -> torch.Tensor:
    """The body ``fused_experts_impl`` is replaced with (reference extra/sglang.patch:18-41): tuning knobs from the
    table ``ALPHA_MOE_CONFIG`` names, per-token-group FP8 quantisation of ``hidden_states``, block alignment of the
    routing, the fused operator.  ``hidden_states`` ``[M, K]`` bf16 is overwritten with the result and returned, as in
    the reference (which zero-fills it and adds; the storing variant needs no zero-fill)."""
    import alpha_moe  # noqa: F401  registers the operators
    from .prep_hip import moe_align_block_size, per_token_group_quant_fp8

    config_path = config_path or os.environ["ALPHA_MOE_CONFIG"]
    M, top_k, E = hidden_states.shape[0], topk_ids.shape[1], w13.shape[0]
    cfg = get_best_config(config_path, M)
    a_q, a_scale = per_token_group_quant_fp8(hidden_states, group_size)
    sorted_token_ids, expert_ids, num_tokens_post_padded = moe_align_block_size(
        topk_ids.to(torch.int32), cfg["block_m"], E)
    torch.ops.alpha_moe.fused_moe_w8a8_up_down_store(
        a_q, a_scale, w13, w13_scale, w2, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
        topk_weights.to(torch.float32), hidden_states, top_k, cfg["block_m"], cfg["block_n"], cfg["warp_n"], cfg["stages"],
        routed_scaling_factor or 1.0)
    return hidden_states
