"""Synthetic problems for the fused W8A8 MoE operator: the shapes the benchmarks and parity tests run on.

Every problem is generated from one seeded ``torch.Generator`` on the
requested device, so the device kernel and a CPU checker can be handed the
very same quantised bits (copy the tensors, do not regenerate).

Input distributions follow the reference's callers where they exist
(test_moe_correctness.py:49-67, jit_moe.py:113-142) and realistic checkpoints
otherwise: weights ~N(0, std) block-quantised 128x128, activations ~N(0, 1)
bf16 quantised per token per 128 columns, router logits ~N(0, 1).
"""
from dataclasses import dataclass, field
from typing import Dict, Optional

import torch

from .prep import block_quant_fp8, moe_align_block_size, per_token_group_quant_fp8
from .utils import interleave_tensor


@dataclass(frozen=True)
class Shape:
    """One expert-shard shape.  ``E`` counts the fused shared expert when there is one."""
    name: str
    E: int
    top_k: int
    K: int
    I: int
    shared_expert: bool
    routing: str            # "softmax_renorm" | "softmax_shared" | "zipf"
    scaling_factor: float
    w_std: float = 0.02

    @property
    def N(self) -> int:
        return 2 * self.I


SHAPES: Dict[str, Shape] = {
    # CPU-runnable case: E=8, top-2 renormalised
    "c1": Shape("c1", E=8, top_k=2, K=512, I=128, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0),
    # DeepSeek-V3-like TP shard: 256 routed + 1 shared expert that every token selects
    "ds": Shape("ds", E=257, top_k=9, K=7168, I=256, shared_expert=True, routing="softmax_shared", scaling_factor=2.5),
    # Qwen3-Next-like: many small experts
    "qn": Shape("qn", E=512, top_k=10, K=2048, I=256, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0),
    # Qwen3-30B-A3B-like with Zipf(1.2) expert popularity (load imbalance)
    "q3": Shape("q3", E=128, top_k=8, K=2048, I=768, shared_expert=False, routing="zipf", scaling_factor=1.0),
}


@dataclass
class Weights:
    """Quantised expert weights in the operator's layout (w1 gate/up interleaved)."""
    shape: Shape
    w1: torch.Tensor          # fp8 [E, N, K], rows interleaved rep=8
    w1_scale: torch.Tensor    # f32 [E, N/128, K/128], rows interleaved rep=1
    w2: torch.Tensor          # fp8 [E, K, I]
    w2_scale: torch.Tensor    # f32 [E, K/128, I/128]


@dataclass
class Problem:
    """One call's worth of inputs."""
    weights: Weights
    M: int
    x: torch.Tensor           # fp8 [M, K]
    x_scale: torch.Tensor     # f32 [M, K/128]
    topk_ids: torch.Tensor    # int32 [M, top_k]
    topk_weights: torch.Tensor  # f32 [M, top_k]
    aligned: dict = field(default_factory=dict)

    @property
    def shape(self) -> Shape:
        return self.weights.shape

    def align(self, block_m: int):
        """Routing arrays for ``block_m`` (cached per block size)."""
        if block_m not in self.aligned:
            self.aligned[block_m] = moe_align_block_size(self.topk_ids, block_m, self.shape.E)
        return self.aligned[block_m]

    def active_experts(self) -> int:
        return int(torch.unique(self.topk_ids).numel())

    def algorithmic_bytes(self) -> int:
        """HBM bytes one call must move: active experts' weights and scales once, activations, routing, output once."""
        s, M = self.shape, self.M
        per_expert = s.N * s.K + s.K * s.I + 4 * ((s.N // 128) * (s.K // 128) + (s.K // 128) * (s.I // 128))
        n_blocks = 0
        if self.aligned:
            bm = sorted(self.aligned)[0]
            n_blocks = int(self.aligned[bm][2].item()) // bm
        return (self.active_experts() * per_expert + M * s.K + 4 * M * (s.K // 128) + 2 * M * s.K
                + 8 * M * s.top_k + 4 * n_blocks)

    def algorithmic_flops(self) -> int:
        s = self.shape
        return 3 * self.M * s.top_k * s.K * s.N


def make_weights(shape: Shape, device="cpu", seed: int = 0, experts_per_chunk: int = 16) -> Weights:
    """Random block-quantised expert weights, generated a few experts at a time to bound memory."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    s = shape
    w1 = torch.empty((s.E, s.N, s.K), dtype=torch.float8_e4m3fn, device=device)
    w2 = torch.empty((s.E, s.K, s.I), dtype=torch.float8_e4m3fn, device=device)
    w1_scale = torch.empty((s.E, s.N // 128, s.K // 128), dtype=torch.float32, device=device)
    w2_scale = torch.empty((s.E, s.K // 128, s.I // 128), dtype=torch.float32, device=device)
    for e0 in range(0, s.E, experts_per_chunk):
        e1 = min(s.E, e0 + experts_per_chunk)
        a = torch.randn((e1 - e0, s.N, s.K), generator=gen, device=device) * s.w_std
        q, sc = block_quant_fp8(a)
        w1[e0:e1] = interleave_tensor(q, 8)
        w1_scale[e0:e1] = interleave_tensor(sc, 1)
        b = torch.randn((e1 - e0, s.K, s.I), generator=gen, device=device) * s.w_std
        q, sc = block_quant_fp8(b)
        w2[e0:e1] = q
        w2_scale[e0:e1] = sc
    return Weights(s, w1, w1_scale, w2, w2_scale)


def make_routing(shape: Shape, M: int, gen: torch.Generator, device="cpu"):
    """``(topk_ids int32 [M, top_k], topk_weights f32 [M, top_k])`` for the shape's routing rule."""
    s = shape
    if s.routing == "softmax_renorm":
        logits = torch.randn((M, s.E), generator=gen, device=device)
        w, ids = torch.softmax(logits, dim=-1).topk(s.top_k, dim=-1)
        w = w / w.sum(dim=-1, keepdim=True)
    elif s.routing == "softmax_shared":
        routed = s.E - 1
        logits = torch.randn((M, routed), generator=gen, device=device)
        w, ids = torch.softmax(logits, dim=-1).topk(s.top_k - 1, dim=-1)
        ids = torch.cat([ids, torch.full((M, 1), routed, dtype=ids.dtype, device=device)], dim=1)
        w = torch.cat([w, torch.ones((M, 1), device=device)], dim=1)
    elif s.routing == "zipf":
        p = torch.arange(1, s.E + 1, dtype=torch.float32, device=device).pow(-1.2)
        ids = torch.multinomial((p / p.sum()).expand(M, s.E), s.top_k, replacement=False, generator=gen)
        w = torch.softmax(torch.randn((M, s.top_k), generator=gen, device=device), dim=-1)
    else:
        raise ValueError(f"unknown routing rule {s.routing!r}")
    return ids.to(torch.int32).contiguous(), w.float().contiguous()


def make_problem(weights: Weights, M: int, seed: int = 0, device: Optional[str] = None) -> Problem:
    """Activations and routing for ``M`` tokens on the device the weights live on."""
    device = device if device is not None else weights.w1.device
    gen = torch.Generator(device=device)
    gen.manual_seed(seed + 1000003 * M)
    s = weights.shape
    x = torch.randn((M, s.K), generator=gen, device=device).to(torch.bfloat16)
    xq, xs = per_token_group_quant_fp8(x)
    ids, w = make_routing(s, M, gen, device)
    return Problem(weights, M, xq.contiguous(), xs, ids, w)
