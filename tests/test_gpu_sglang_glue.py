"""The SGLang wiring of extra/sglang_rocm.patch, replayed without SGLang: the weight loader hands gate and up shards of
every expert to W13Interleaver the way FusedMoE.weight_loader does, fused_experts runs the forward path of
fused_experts_impl (tuning table from ALPHA_MOE_CONFIG, HIP quantiser, HIP aligner, storing operator), and the result is
checked against the CPU oracle fed with the ORIGINAL (not interleaved) checkpoint tensors."""
import json
import os

import pytest
import torch

from alpha_moe_python.prep import block_quant_fp8
from alpha_moe_python.sglang_glue import W13Interleaver, fused_experts
from alpha_moe_python.utils import get_best_config, interleave_tensor
from gpu_util import MAX_ABS_OVER_MAX_REF, MIN_COSINE
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("M", [3, 40, 300])
def test_fused_experts_matches_the_oracle_on_the_checkpoint_tensors(M, tmp_path):
    E, top_k, K, I = 10, 4, 512, 256
    g = torch.Generator().manual_seed(11 + M)
    # the checkpoint: per expert a gate matrix (w1), an up matrix (w3) and a down matrix (w2), block-quantised FP8
    w13_f = torch.randn((E, 2 * I, K), generator=g) * 0.05
    w2_f = torch.randn((E, K, I), generator=g) * 0.05
    w13_q, w13_s = block_quant_fp8(w13_f)            # [E, 2I, K] fp8 (gate rows first, up rows second), [E, 2I/128, K/128]
    w2_q, w2_s = block_quant_fp8(w2_f)
    # FusedMoE's parameters, filled shard by shard
    w13 = torch.zeros((E, 2 * I, K), dtype=torch.float8_e4m3fn, device=DEV)
    w13_scale = torch.zeros((E, 2 * I // 128, K // 128), dtype=torch.float32, device=DEV)
    il_w, il_s = W13Interleaver(E, 8), W13Interleaver(E, 1)
    for e in range(E):
        for shard in (("w3", "w1") if e % 2 else ("w1", "w3")):
            rows = slice(0, I) if shard == "w1" else slice(I, 2 * I)
            srows = slice(0, I // 128) if shard == "w1" else slice(I // 128, 2 * I // 128)
            w13[e, rows] = w13_q[e, rows].to(DEV)
            il_w.shard_loaded(w13[e], e, shard)
            w13_scale[e, srows] = w13_s[e, srows].to(DEV)
            il_s.shard_loaded(w13_scale[e], e, shard)
    assert torch.equal(w13.cpu().view(torch.uint8), interleave_tensor(w13_q, 8).view(torch.uint8))
    assert torch.equal(w13_scale.cpu(), interleave_tensor(w13_s, 1))
    # the forward call of one layer
    cfg_path = os.path.join(tmp_path, "table.json")
    with open(cfg_path, "w") as fh:
        json.dump({"1": {"block_m": 16, "block_n": 32, "warp_n": 8, "stages": 4},
                   "64": {"block_m": 16, "block_n": 64, "warp_n": 4, "stages": 3},
                   "512": {"block_m": 64, "block_n": 64, "warp_n": 4, "stages": 3}}, fh)
    hidden = (torch.randn((M, K), generator=g)).to(torch.bfloat16)
    probs = torch.softmax(torch.randn((M, E), generator=g), dim=-1)
    topk_weights, topk_ids = probs.topk(top_k, dim=-1)
    os.environ["ALPHA_MOE_CONFIG"] = cfg_path
    try:
        h = hidden.to(DEV).clone()
        print(f"case sglang glue M={M} knobs {get_best_config(cfg_path, M)}", flush=True)
        got = fused_experts(h, w13, w2_q.to(DEV), topk_weights.to(DEV), topk_ids.to(DEV), w13_scale, w2_s.to(DEV),
                            routed_scaling_factor=2.5)
        torch.cuda.synchronize()
    finally:
        del os.environ["ALPHA_MOE_CONFIG"]
    assert got.data_ptr() == h.data_ptr()   # hidden_states is reused as the output, as the reference's patch does
    # oracle: quantise the activations the same way, route, and run the maths on the interleaved tensors' originals
    xq, xs = O.quant_group_reference(hidden)
    ids = O.align_reference(topk_ids.to(torch.int32), 16, E)
    ref = O.fused_moe_oracle(xq.view(torch.float8_e4m3fn), xs, interleave_tensor(w13_q, 8), interleave_tensor(w13_s, 1), w2_q,
                             w2_s, *ids, topk_weights.float().contiguous(), torch.zeros((M, K), dtype=torch.bfloat16),
                             top_k, 16, 2.5)
    m = O.error_metrics(got, ref)
    assert m["max_abs_over_max_ref"] <= MAX_ABS_OVER_MAX_REF and m["cosine"] >= MIN_COSINE, m
