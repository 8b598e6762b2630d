"""Layout and tuning-table helpers of the fused W8A8 MoE operator.

Same import path and signatures as the reference's
``alpha_moe_python/utils.py`` (``interleave_tensor`` at utils.py:5-17,
``get_best_config`` at utils.py:19-29); the implementations are independent
restatements of the closed forms.
"""
import functools
import json

import torch


def interleave_tensor(tensor: torch.Tensor, rep: int = 8) -> torch.Tensor:
    """Interleave the gate half and the up half of dim 1 in chunks of ``rep`` rows.

    Input ``[E, N, K]`` holds rows ``[gate_0..gate_{N/2-1}, up_0..up_{N/2-1}]``.
    Output row ``2*rep*c + h*rep + j`` is input row ``h*(N/2) + rep*c + j``
    (``h`` = 0 gate / 1 up, ``c`` = chunk, ``j`` < rep).  Weights use rep=8,
    128x128 block scales use rep=1 (reference utils.py:5-17).
    """
    if tensor.dim() != 3:
        raise ValueError(f"interleave_tensor expects [E, N, K], got {tuple(tensor.shape)}")
    E, N, K = tensor.shape
    if rep <= 0 or N % (2 * rep) != 0:
        raise ValueError(f"N={N} must be a multiple of 2*rep={2 * rep}")
    chunks = N // (2 * rep)
    # [E, half, chunk, j, K] -> [E, chunk, half, j, K]
    return tensor.reshape(E, 2, chunks, rep, K).permute(0, 2, 1, 3, 4).reshape(E, N, K).contiguous()


def deinterleave_tensor(tensor: torch.Tensor, rep: int = 8) -> torch.Tensor:
    """Inverse of :func:`interleave_tensor` (no counterpart in the reference; used by tests and tools)."""
    if tensor.dim() != 3:
        raise ValueError(f"deinterleave_tensor expects [E, N, K], got {tuple(tensor.shape)}")
    E, N, K = tensor.shape
    if rep <= 0 or N % (2 * rep) != 0:
        raise ValueError(f"N={N} must be a multiple of 2*rep={2 * rep}")
    chunks = N // (2 * rep)
    return tensor.reshape(E, chunks, 2, rep, K).permute(0, 2, 1, 3, 4).reshape(E, N, K).contiguous()


def prepack_weights(w: torch.Tensor, w2: torch.Tensor):
    """Optional offline re-layout of the expert weights for ``fused_moe_w8a8_up_down_prepacked``.

    ``w`` is the operator's ``[E, N, K]`` (already through ``interleave_tensor(w, 8)``), ``w2`` its ``[E, K, I]``.
    Returns ``(w_packed [E, K/128, N, 128], w2_packed [E, I/128, K, 128])``: the same bytes with every 128-byte K block
    of consecutive rows contiguous, so that the 256 rows a kernel step consumes are one 32 KiB burst instead of 256 row
    pieces K bytes apart.  Scales are unchanged.  The interleave-8 layout stays the operator's API (reference
    utils.py:5-17, README.md:94-102); this comes after it and has no counterpart in the reference.
    """
    if w.dim() != 3 or w2.dim() != 3 or w.shape[2] % 128 or w2.shape[2] % 128:
        raise ValueError(f"prepack_weights expects [E, N, K] and [E, K, I] with K and I multiples of 128, got "
                         f"{tuple(w.shape)} and {tuple(w2.shape)}")
    E, N, K = w.shape
    if tuple(w2.shape) != (E, K, N // 2):
        raise ValueError(f"w2 must be [E, K, N/2] = {(E, K, N // 2)}, got {tuple(w2.shape)}")
    wp = w.reshape(E, N, K // 128, 128).permute(0, 2, 1, 3).contiguous()
    w2p = w2.reshape(E, K, (N // 2) // 128, 128).permute(0, 2, 1, 3).contiguous()
    return wp, w2p


def unpack_weights(w_packed: torch.Tensor, w2_packed: torch.Tensor):
    """Inverse of :func:`prepack_weights`: back to ``[E, N, K]`` and ``[E, K, I]``."""
    E, nkb, N, _ = w_packed.shape
    _, nib, K, _ = w2_packed.shape
    w = w_packed.permute(0, 2, 1, 3).reshape(E, N, nkb * 128).contiguous()
    w2 = w2_packed.permute(0, 2, 1, 3).reshape(E, K, nib * 128).contiguous()
    return w, w2


@functools.lru_cache()
def get_best_config(path: str, n_tokens: int):
    """Entry of the JSON tuning table whose integer key is nearest to ``n_tokens``.

    The table maps ``str(M)`` to ``{"block_m", "block_n", "warp_n", "stages"}``.
    Ties go to the key that comes first in the file; results are memoised per
    ``(path, n_tokens)`` (reference utils.py:19-29).
    """
    with open(path, "r") as fh:
        table = json.load(fh)
    best = None
    best_dist = None
    for key, cfg in table.items():
        dist = abs(int(key) - n_tokens)
        if best_dist is None or dist < best_dist:
            best, best_dist = cfg, dist
    return best
