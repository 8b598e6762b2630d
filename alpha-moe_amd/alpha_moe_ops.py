"""Typed Python front of ``torch.ops.alpha_moe.fused_moe_w8a8_up_down`` plus its fake (meta) registration, so the
operator can be traced by ``torch.compile`` / ``torch.export``.  Same module name, function name and argument list
as the reference's alpha_moe_ops.py:5-25,28-88.
"""
import torch

import alpha_moe  # noqa: F401  (registers the operator)


@torch.library.register_fake("alpha_moe::fused_moe_w8a8_up_down")
def _fused_moe_w8a8_up_down_fake(x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids,
                                 num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n, stages,
                                 scaling_factor):
    # the operator returns nothing; it only mutates ``out``
    return None


@torch.library.register_fake("alpha_moe::fused_moe_w8a8_up_down_store")
def _fused_moe_w8a8_up_down_store_fake(x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids,
                                       num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n,
                                       stages, scaling_factor):
    return None


@torch.library.register_fake("alpha_moe::fused_moe_w8a8_up_down_prepacked")
def _fused_moe_w8a8_up_down_prepacked_fake(x, x_scale, w_packed, w_scale, w2_packed, w2_scale, sorted_token_ids,
                                           expert_ids, num_tokens_post_padded, topk_weights, out, top_k, block_m,
                                           block_n, warp_n, stages, scaling_factor, store):
    return None


@torch.library.register_fake("alpha_moe::per_token_group_quant_fp8")
def _per_token_group_quant_fp8_fake(x, group_size):
    return (torch.empty_like(x, dtype=torch.float8_e4m3fn),
            x.new_empty((x.shape[0], x.shape[1] // group_size), dtype=torch.float32))


@torch.library.register_fake("alpha_moe::moe_align_block_size")
def _moe_align_block_size_fake(topk_ids, block_size, num_experts):
    sorted_num = topk_ids.numel() + num_experts * (block_size - 1)
    return (topk_ids.new_empty((sorted_num,)), topk_ids.new_empty(((sorted_num + block_size - 1) // block_size,)),
            topk_ids.new_empty((1,)))


def fused_moe_w8a8_up_down(
    x: torch.Tensor,
    x_scale: torch.Tensor,
    w: torch.Tensor,
    w_scale: torch.Tensor,
    w2: torch.Tensor,
    w2_scale: torch.Tensor,
    sorted_token_ids: torch.Tensor,
    expert_ids: torch.Tensor,
    num_tokens_post_padded: torch.Tensor,
    topk_weights: torch.Tensor,
    out: torch.Tensor,
    top_k: int,
    block_m: int,
    block_n: int,
    warp_n: int,
    stages: int,
    scaling_factor: float,
) -> torch.Tensor:
    """Fused FP8 expert MLP: ``out += scaling_factor * sum_s topk_weights[t,s] * W2_e(requant(SwiGLU(W1_e x_t)))``.

    x ``[M, K]`` fp8 e4m3 with x_scale ``[M, K/128]``; w ``[E, N, K]`` fp8, gate/up rows interleaved in chunks of 8
    (``interleave_tensor(w, 8)``), w_scale ``[E, N/128, K/128]`` interleaved in chunks of 1; w2 ``[E, K, N/2]`` fp8 with
    w2_scale ``[E, K/128, N/256]``; sorted_token_ids / expert_ids / num_tokens_post_padded from
    ``moe_align_block_size(topk_ids, block_m, E)``; topk_weights ``[M, top_k]`` fp32; out ``[M, K]`` bf16, zero-filled by
    the caller and updated in place.  block_m (8..128 step 8), (block_n, warp_n) in {(64,4),(32,8)} and stages (1..5)
    are tuning knobs that do not change the result.  Returns ``out``.
    """
    torch.ops.alpha_moe.fused_moe_w8a8_up_down(
        x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, out,
        top_k, block_m, block_n, warp_n, stages, scaling_factor)
    return out


def fused_moe_w8a8_up_down_store(x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids,
                                 num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n, stages,
                                 scaling_factor) -> torch.Tensor:
    """``fused_moe_w8a8_up_down`` with store semantics: ``out`` is overwritten with the result, so it may come from
    ``torch.empty_like`` and the zero-fill before every call (one more kernel launch at decode sizes) goes away.  The
    reference has no such variant.  Returns ``out``."""
    torch.ops.alpha_moe.fused_moe_w8a8_up_down_store(
        x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, out,
        top_k, block_m, block_n, warp_n, stages, scaling_factor)
    return out


def fused_moe_w8a8_up_down_prepacked(x, x_scale, w_packed, w_scale, w2_packed, w2_scale, sorted_token_ids, expert_ids,
                                     num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n, stages,
                                     scaling_factor, store: bool = False) -> torch.Tensor:
    """The operator on weights re-laid-out once by ``alpha_moe_python.utils.prepack_weights`` (``w_packed``
    ``[E, K/128, N, 128]``, ``w2_packed`` ``[E, I/128, K, 128]``); every other argument as in
    ``fused_moe_w8a8_up_down``, ``store=True`` for the overwriting variant.  Bit for bit the result of the call on the
    unpacked weights.  The reference has no such variant.  Returns ``out``."""
    torch.ops.alpha_moe.fused_moe_w8a8_up_down_prepacked(
        x, x_scale, w_packed, w_scale, w2_packed, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
        topk_weights, out, top_k, block_m, block_n, warp_n, stages, scaling_factor, store)
    return out


__all__ = ["fused_moe_w8a8_up_down", "fused_moe_w8a8_up_down_store", "fused_moe_w8a8_up_down_prepacked"]
