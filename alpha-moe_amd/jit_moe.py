"""Autotuner of the fused W8A8 MoE operator: for every batch size, time each (block_m, block_n, warp_n, stages)
the operator accepts and write the fastest to a JSON table that `alpha_moe_python.utils.get_best_config` reads.

Same command line and the same JSON as the reference's jit_moe.py (flags jit_moe.py:54-98, sweep jit_moe.py:151-157,
writer jit_moe.py:169-183):

    python alpha-moe_amd/jit_moe.py --E 256 --N 512 --K 7168 --out-config moe_jit_257_512_7168.json

Differences, all on purpose:
  * activations are quantised and routing arrays built by this package's own HIP kernels (alpha_moe_python.prep_hip), not SGLang;
  * `--balancedness` is honoured (the reference parses it and then samples uniformly, jit_moe.py:135);
  * a call is timed with HIP events on the launch stream after a 512 MiB write that evicts L2 and the 256 MiB
    Infinity Cache (the reference allocates 2 GiB of randn before every call, jit_moe.py:21-22);
  * `--block-ms`, `--stages` and `--num-tests` bound the sweep (the full space is 160 configurations) and `--update`
    merges the result into an existing table;
  * on MI355X the knobs select this: row blocks of at most 32 rows take the streaming kernel (`warp_n` = wavefronts per
    workgroup, `stages` = depth of each wavefront's LDS ring); above that `warp_n` 4 takes the tile kernel (one row
    block per item, four token tiles per wavefront), `warp_n` 8 the wide kernel (macro blocks of 256 rows, eight token
    tiles per wavefront), and `stages` sets the length of their down-projection items.
"""
import argparse
import json
import os
import sys
from statistics import mean

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

_FLUSH = None


def bench_events(fn, num_tests: int = 25, flush_bytes: int = 512 << 20):
    """Mean device time of `fn` in microseconds over `num_tests` calls, each on a cold cache."""
    global _FLUSH
    if _FLUSH is None or _FLUSH.numel() * 4 < flush_bytes:
        _FLUSH = torch.empty(flush_bytes // 4, dtype=torch.int32, device="cuda")
    times = []
    for i in range(num_tests):
        _FLUSH.fill_(i)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end) * 1e3)
    return sum(times) / len(times)


def generate_topk_ids(num_experts, num_tokens, top_k, balancedness=1.0):
    """Routing for the sweep: every slot independently goes to a uniformly drawn expert with probability
    `balancedness` and to expert 0 otherwise (the mixture the reference's generator draws from, jit_moe.py:34-51;
    a token may name an expert twice, as there)."""
    n_slots = num_tokens * top_k
    ids = torch.randint(0, num_experts, (n_slots,))
    ids[torch.rand(n_slots) >= balancedness] = 0
    return ids.view(num_tokens, top_k)


def candidate_list(block_ms, stages):
    """Every (block_m, block_n, warp_n, stages) of the sweep: the reference's space (jit_moe.py:151-157) restricted to
    the requested block sizes and stages.  Each combination selects a different kernel variant or item size."""
    return [(bm, bn, wn, st) for bm in block_ms for (bn, wn) in ((64, 4), (32, 8)) for st in stages]


def pick_best(times):
    """{batch size: {candidate: [mean us per routing sample]}} -> {batch size: table entry}, fastest mean first."""
    table = {}
    for nt, val in times.items():
        timed = [(k, mean(v)) for k, v in val.items() if len(v) > 0]
        (block_m, bn, wn, stages), best_us = sorted(timed, key=lambda kv: kv[1])[0]
        print(f"M={nt}: best {(block_m, bn, wn, stages)} {best_us:.1f} us", flush=True)
        table[nt] = {"block_m": block_m, "block_n": bn, "warp_n": wn, "stages": stages}
    return table


def write_table(path, table, update=False):
    """The reference's writer (jit_moe.py:181-183): json.dump of {batch size: entry}, so keys come out as strings.
    update=True keeps the entries `path` already holds for batch sizes not in `table`."""
    if update and os.path.exists(path):
        with open(path) as f:
            merged = {int(k): v for k, v in json.load(f).items()}
        merged.update(table)
        table = dict(sorted(merged.items()))
    with open(path, "w") as f:
        json.dump(table, f)
    return table


def parse_arguments(argv=None):
    parser = argparse.ArgumentParser(description="MoE autotuner (MI355X)")
    parser.add_argument("--batch-sizes", type=int, nargs="+", default=[8, 32, 128, 256, 512, 1024, 2048, 4096, 8192],
                        help="Batch sizes to benchmark")
    parser.add_argument("--balancedness", type=float, nargs="+", default=[0.8, 0.7, 0.6, 0.5],
                        help="Balancedness values to test")
    parser.add_argument("--N", type=int, default=256, help="N dimension for MoE")
    parser.add_argument("--K", type=int, default=7168, help="K dimension for MoE")
    parser.add_argument("--E", type=int, default=256, help="num_experts for MoE(not including shared expert)")
    parser.add_argument("--top-k", type=int, default=8, help="top-k experts picked")
    parser.add_argument("--shared-expert", default=True, action=argparse.BooleanOptionalAction,
                        help="If MoE is using a shared expert")
    parser.add_argument("--out-config", default=None, help="Where to store config, default: moe_jit_E_N_K.json")
    parser.add_argument("--block-ms", type=int, nargs="+", default=list(range(8, 129, 8)), help="block_m values to sweep")
    parser.add_argument("--stages", type=int, nargs="+", default=[1, 2, 3, 4, 5], help="stages values to sweep")
    parser.add_argument("--num-tests", type=int, default=25, help="timed calls per configuration and routing sample")
    parser.add_argument("--update", action="store_true",
                        help="keep the entries --out-config already holds for batch sizes not benchmarked in this run")
    return parser.parse_args(argv)


def main(argv=None):
    args = parse_arguments(argv)
    import alpha_moe  # noqa: F401  registers torch.ops.alpha_moe.fused_moe_w8a8_up_down
    from alpha_moe_python.prep_hip import moe_align_block_size, per_token_group_quant_fp8
    torch.manual_seed(42)
    dev = "cuda:0"
    top_k = args.top_k + args.shared_expert
    E = args.E + args.shared_expert
    N, K = args.N, args.K
    if N % 256 or K % 128:
        raise SystemExit("N must be a multiple of 256 and K a multiple of 128")
    w1 = torch.randn((E, N, K)).to(torch.float8_e4m3fn).to(dev)
    w2 = torch.randn((E, K, N // 2)).to(torch.float8_e4m3fn).to(dev)
    w1_scale = (torch.randn((E, N // 128, K // 128), dtype=torch.float32) * 0.01).to(dev)
    w2_scale = (torch.randn((E, K // 128, N // 256), dtype=torch.float32) * 0.01).to(dev)

    candidates = candidate_list(args.block_ms, args.stages)
    times = {}
    for num_tokens in args.batch_sizes:
        times[num_tokens] = {c: [] for c in candidates}
        print("Batch size", num_tokens, flush=True)
        topk_weights = torch.softmax(torch.randn((num_tokens, top_k), dtype=torch.float32), dim=-1).to(dev)
        for balancedness in args.balancedness:
            topk_ids = generate_topk_ids(E - args.shared_expert, num_tokens, top_k - args.shared_expert, balancedness)
            if args.shared_expert:
                topk_ids = torch.hstack((topk_ids, torch.full((num_tokens, 1), E - 1, dtype=topk_ids.dtype)))
            topk_ids = topk_ids.to(torch.int32).to(dev)
            x = torch.empty((num_tokens, K), dtype=torch.bfloat16).normal_(mean=0, std=0.05).to(dev)
            x_q, x_scale = per_token_group_quant_fp8(x, 128)
            out = torch.zeros_like(x)
            for block_m, bn, wn, stages in candidates:
                if num_tokens < block_m and block_m != 16:
                    continue
                # far from any plausible winner: whole-K streaming items with 8-row blocks at prefill sizes, and
                # 256-row macro blocks at decode sizes, cost minutes of sweep for nothing
                if (block_m <= 32 and num_tokens * top_k > 64 * E) or (block_m > 32 and num_tokens * top_k < E):
                    continue
                sorted_token_ids, expert_ids, num_tokens_post_padded = moe_align_block_size(topk_ids, block_m, E)

                def call():
                    torch.ops.alpha_moe.fused_moe_w8a8_up_down(
                        x_q, x_scale, w1, w1_scale, w2, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                        topk_weights, out, top_k, block_m, bn, wn, stages, 2.5)
                call()
                times[num_tokens][(block_m, bn, wn, stages)].append(bench_events(call, args.num_tests))

    out_config = args.out_config or f"moe_jit_{E}_{N}_{K}.json"
    write_table(out_config, pick_best(times), args.update)
    return 0


if __name__ == "__main__":
    sys.exit(main())
