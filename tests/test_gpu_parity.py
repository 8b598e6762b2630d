"""GPU parity: the HIP operator against the CPU oracle on the same seeded bits.

Bar (written out in gpu_util.py): max |err| / max |ref| <= 1e-2 and cosine >= 0.9999 on the bf16 output.
"""
import pytest
import torch

from alpha_moe_python.workloads import SHAPES, Shape, make_problem, make_weights
from gpu_util import (assert_parity, assert_parity_rows, oracle_out, oracle_variants, run_op, sampled_tokens_match_oracle,
                      tunables, worst_row_error)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

ALL_KNOBS = [(bm, bn, wn, st) for bm in range(8, 129, 8) for (bn, wn) in ((64, 4), (32, 8)) for st in range(1, 6)]


@pytest.fixture(scope="module")
def c1():
    W = make_weights(SHAPES["c1"], device=DEV, seed=0)
    P = make_problem(W, 16, seed=0)
    return P, oracle_out(P)


def test_c1_default_knobs_torch_op_and_c_abi(c1):
    P, ref = c1
    print("case c1 M=16 block_m=16 (64,4) stages=3", flush=True)
    assert_parity(run_op(P, 16, 64, 4, 3, via="torch"), ref, "torch op")
    assert_parity(run_op(P, 16, 64, 4, 3, via="c_abi"), ref, "c abi")


def test_c_abi_workspace_is_reusable_without_clearing(c1):
    """One zero-filled workspace, many calls with different knobs (and so different kernels and layouts inside it)."""
    import alpha_moe
    P, ref = c1
    sizes = [alpha_moe.c_abi.alpha_moe_workspace_bytes(P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, P.align(bm)[0].numel(), bm)
             for bm in (8, 16, 32, 64)]
    ws = torch.zeros(max(sizes), dtype=torch.uint8, device=DEV)
    for bm, bn, wn, st in [(16, 64, 4, 2), (16, 64, 4, 2), (8, 32, 8, 3), (64, 64, 4, 2), (32, 32, 8, 1), (16, 64, 4, 4)]:
        print(f"case c1 shared workspace knobs {(bm, bn, wn, st)}", flush=True)
        assert_parity(run_op(P, bm, bn, wn, st, via="c_abi", workspace=ws), ref, f"shared ws {(bm, bn, wn, st)}")
    # a second problem of another size on the same buffer, streaming and tile kernels taking turns
    P2 = make_problem(P.weights, 150, seed=9)
    need = max(alpha_moe.c_abi.alpha_moe_workspace_bytes(P2.shape.top_k, P2.M, P2.shape.K, P2.shape.N, P2.shape.E,
                                                         P2.align(bm)[0].numel(), bm) for bm in (16, 64, 128))
    ws2 = torch.zeros(max(need, ws.numel()), dtype=torch.uint8, device=DEV)
    cases = [(P2, (128, 64, 4, 3)), (P, (16, 32, 8, 5)), (P2, (64, 64, 4, 3)), (P2, (16, 64, 4, 3)), (P, (96, 64, 4, 3))]
    fresh = [run_op(prob, *knobs, via="c_abi") for prob, knobs in cases]   # each on a zero-filled buffer of its own
    for rep in range(3):
        for (prob, knobs), want in zip(cases, fresh):
            print(f"case shared workspace round {rep} M={prob.M} knobs {knobs}", flush=True)
            assert torch.equal(run_op(prob, *knobs, via="c_abi", workspace=ws2), want), (rep, prob.M, knobs)


def test_c1_result_independent_of_every_knob(c1):
    """The reference's correctness sweep runs every (block_m, block_n/warp_n, stages) it accepts
    (test_moe_correctness.py:172-190); the result may not depend on them."""
    P, ref = c1
    for bm, bn, wn, st in ALL_KNOBS:
        print(f"case c1 M=16 knobs {(bm, bn, wn, st)}", flush=True)
        assert_parity(run_op(P, bm, bn, wn, st), ref, f"knobs {(bm, bn, wn, st)}")


def test_add_semantics_scaling_and_zero_weights(c1):
    P, ref = c1
    pre = torch.full((P.M, P.shape.K), 0.25, dtype=torch.bfloat16, device=DEV)
    got = run_op(P, 16, 32, 8, 2, out=pre.clone())
    assert_parity(got, oracle_out(P, out=pre.cpu()), "out pre-filled")
    assert_parity(run_op(P, 16, 64, 4, 2, scaling=2.5), oracle_out(P, scaling=2.5), "scaling 2.5")
    saved = P.topk_weights
    P.topk_weights = torch.zeros_like(saved)
    assert float(run_op(P, 16, 64, 4, 2).float().abs().max()) == 0.0
    P.topk_weights = saved


@pytest.mark.parametrize("knobs", [(16, 32, 8, 2), (16, 64, 4, 5), (64, 64, 4, 3), (128, 64, 4, 3)])
def test_store_variant_overwrites_whatever_out_held(c1, knobs):
    """fused_moe_w8a8_up_down_store: out = bf16(sum) on every element, NaN-filled or not, and bit for bit what the
    adding call leaves in a zero-filled out - streaming and tile kernels, torch op and C ABI."""
    P, ref = c1
    zero = run_op(P, *knobs, via="c_abi")
    assert_parity(zero, ref, f"knobs {knobs}")
    for via in ("torch", "c_abi"):
        junk = torch.full((P.M, P.shape.K), float("nan"), dtype=torch.bfloat16, device=DEV)
        got = run_op(P, *knobs, out=junk, via=via, store=True)
        assert torch.equal(got, zero), (knobs, via)
    # a token none of whose slots contributes still gets its row written
    saved = P.topk_weights
    P.topk_weights = torch.zeros_like(saved)
    junk = torch.full((P.M, P.shape.K), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert float(run_op(P, *knobs, out=junk, store=True).float().abs().max()) == 0.0
    P.topk_weights = saved


def test_nine_slices_row_blocks_above_32():
    """Nine 128-column slices are more than the tile kernel takes: the wide kernel streams any number of them, whatever
    (block_n, warp_n) asks for."""
    shape = Shape("s9", E=6, top_k=2, K=256, I=1152, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0)
    W = make_weights(shape, device=DEV, seed=5)
    P = make_problem(W, 150, seed=5)
    ref = oracle_out(P)
    for knobs in ((128, 64, 4, 2), (64, 32, 8, 3)):
        print(f"case nine slices knobs {knobs}", flush=True)
        assert_parity(run_op(P, *knobs, via="c_abi"), ref, f"nine slices {knobs}")


def test_prefill_kernels_fetch_activation_scales_both_ways():
    """The tile and wide kernels take a token's activation scales four K blocks at a time where the row of scales allows
    16-byte loads (K / 128 a multiple of 4, x_scale 16-byte aligned) and one at a time otherwise: both ways against the
    oracle, and bit for bit against each other on the same problem."""
    for K in (384, 512, 640, 1024):
        shape = Shape("wx", E=6, top_k=4, K=K, I=256, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0)
        W = make_weights(shape, device=DEV, seed=K)
        P = make_problem(W, 300, seed=K)
        ref = oracle_out(P)
        for knobs in ((128, 32, 8, 2), (48, 32, 8, 1), (128, 64, 4, 3), (64, 64, 4, 4)):
            print(f"case scale fetch K={K} knobs {knobs}", flush=True)
            a = run_op(P, *knobs, via="c_abi")
            m = assert_parity(a, ref, f"K={K} {knobs}")
            print(f"   -> {m['max_abs_over_max_ref']:.2e}", flush=True)
            # the same scales four bytes off a 16-byte boundary: the kernel must fall back to single loads
            aligned = P.x_scale
            raw = torch.empty(aligned.numel() + 1, dtype=torch.float32, device=DEV)
            raw[1:].copy_(aligned.flatten())
            P.x_scale = raw[1:].view_as(aligned)
            assert P.x_scale.data_ptr() % 16 == 4
            b = run_op(P, *knobs, via="c_abi")
            P.x_scale = aligned
            assert torch.equal(a, b), (K, knobs)


def test_wide_kernel_up_loop_variants_give_the_same_bits():
    """The wide kernel has two forms of its up/gate loop: both wavefronts of a SIMD in step, or half a step apart (one
    multiplies a whole step alone, token tiles in blocks of four from the top down with a queue of pending products
    that lives across steps, while the other loads).  ALPHA_MOE_WIDE_PP picks one (unset: by rows per expert).  Both
    against the oracle and bit for bit against each other, over: one to sixteen live token tiles in a block and blocks
    whose second wavefront of a pair has none; one, two, three, four and eight K steps (the loop's prologue issues
    two steps of loads; activation scales are fetched four steps at a time from K = 512 on and singly otherwise, also
    from a row of scales that is not 16-byte aligned); experts with one block of rows and with several."""
    for K, M in ((128, 150), (256, 300), (384, 40), (512, 700), (1024, 300), (512, 9), (640, 150)):
        shape = Shape("pp", E=6, top_k=4, K=K, I=256, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0)
        W = make_weights(shape, device=DEV, seed=K + M)
        P = make_problem(W, M, seed=K + M)
        ref = oracle_out(P)
        for knobs in ((128, 32, 8, 2), (48, 32, 8, 1)):
            outs = []
            for pp in (0, 1):
                print(f"case up loop K={K} M={M} knobs {knobs} ALPHA_MOE_WIDE_PP={pp}", flush=True)
                with tunables(ALPHA_MOE_WIDE_PP=pp):
                    outs.append(run_op(P, *knobs, via="c_abi"))
                assert_parity(outs[-1], ref, f"K={K} M={M} {knobs} pp={pp}")
            assert torch.equal(outs[0], outs[1]), (K, M, knobs)
            if K == 512 and M == 700:
                aligned = P.x_scale
                raw = torch.empty(aligned.numel() + 1, dtype=torch.float32, device=DEV)
                raw[1:].copy_(aligned.flatten())
                P.x_scale = raw[1:].view_as(aligned)
                with tunables(ALPHA_MOE_WIDE_PP=1):
                    b = run_op(P, *knobs, via="c_abi")
                P.x_scale = aligned
                assert torch.equal(outs[0], b), (K, M, knobs, "unaligned scales")


def test_store_variant_fallback_kernel():
    """129 K blocks are more than the tile and wide kernels take: the fallback kernel serves the call, and its store
    variant overwrites too."""
    from alpha_moe_python.workloads import Shape
    shape = Shape("fb", E=6, top_k=2, K=16512, I=128, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0)
    W = make_weights(shape, device=DEV, seed=5)
    P = make_problem(W, 150, seed=5)
    ref = oracle_out(P)
    assert_parity(run_op(P, 128, 64, 4, 2, via="c_abi"), ref, "fallback kernel")
    junk = torch.full((P.M, P.shape.K), float("nan"), dtype=torch.bfloat16, device=DEV)
    # this kernel sums with fp32 atomics, so two runs agree to rounding, not bit for bit
    assert_parity(run_op(P, 128, 64, 4, 2, out=junk, via="c_abi", store=True), ref, "fallback kernel, store")


@pytest.mark.parametrize("M,E,top_k,K,I", [(1, 4, 2, 128, 128), (3, 5, 3, 384, 256), (37, 3, 2, 256, 384), (200, 2, 1, 128, 128)])
def test_ragged_small_shapes(M, E, top_k, K, I):
    """K a single block, K % 256 == 128 (the reference silently drops the last 128 columns there), more I blocks,
    more tokens than one block, experts without tokens."""
    shape = Shape("t", E=E, top_k=top_k, K=K, I=I, shared_expert=False, routing="softmax_renorm", scaling_factor=1.3,
                  w_std=0.05)
    W = make_weights(shape, device=DEV, seed=M)
    P = make_problem(W, M, seed=M)
    ref = oracle_out(P)
    for bm, bn, wn, st in [(8, 64, 4, 1), (16, 32, 8, 5), (48, 64, 4, 3), (128, 32, 8, 2)]:
        print(f"case ragged {(M, E, top_k, K, I)} knobs {(bm, bn, wn, st)}", flush=True)
        assert_parity(run_op(P, bm, bn, wn, st), ref, f"{(M, E, top_k, K, I)} knobs {(bm, bn, wn, st)}")


def test_duplicate_experts_and_negative_scales():
    """Duplicate expert ids inside one token's top-k and negative block scales are legal inputs
    (test_moe_correctness.py:42,59-60 of the reference generates both)."""
    shape = Shape("t", E=6, top_k=4, K=256, I=128, shared_expert=False, routing="softmax_renorm", scaling_factor=2.5,
                  w_std=0.05)
    W = make_weights(shape, device=DEV, seed=3)
    W.w1_scale.mul_(torch.where(torch.rand_like(W.w1_scale) < 0.5, -1.0, 1.0))
    W.w2_scale.mul_(torch.where(torch.rand_like(W.w2_scale) < 0.5, -1.0, 1.0))
    P = make_problem(W, 24, seed=3)
    g = torch.Generator(device=DEV).manual_seed(7)
    P.topk_ids = torch.randint(0, 6, (24, 4), generator=g, device=DEV, dtype=torch.int32)   # with replacement
    P.aligned.clear()
    ref = oracle_out(P)
    for bm, bn, wn, st in [(8, 32, 8, 3), (32, 64, 4, 2)]:
        print(f"case dup/neg knobs {(bm, bn, wn, st)}", flush=True)
        assert_parity(run_op(P, bm, bn, wn, st), ref, f"dup/neg knobs {(bm, bn, wn, st)}")


def test_bad_arguments_raise(c1):
    P, _ = c1
    with pytest.raises(RuntimeError):
        run_op(P, 12, 64, 4, 2)
    with pytest.raises(RuntimeError):
        run_op(P, 16, 64, 8, 2)
    with pytest.raises(RuntimeError):
        run_op(P, 16, 64, 4, 6)
    with pytest.raises(RuntimeError):
        run_op(P, 16, 64, 4, 2, out=torch.zeros((P.M, P.shape.K), dtype=torch.float16, device=DEV))


@pytest.fixture(scope="module")
def ds_weights():
    return make_weights(SHAPES["ds"], device=DEV, seed=0)


@pytest.mark.parametrize("M,knobs", [(1, (16, 32, 8, 5)), (4, (16, 64, 4, 4)), (16, (16, 64, 4, 3)), (64, (16, 32, 8, 3)),
                                     (64, (8, 64, 4, 2))])
def test_deepseek_shard_decode_full_size(ds_weights, M, knobs):
    """The headline decode configuration at its real size: E=257, top_k=9, K=7168, I=256."""
    P = make_problem(ds_weights, M, seed=0)
    print(f"case ds M={M} knobs {knobs}", flush=True)
    m = assert_parity(run_op(P, *knobs), oracle_out(P), f"ds M={M} knobs {knobs}")
    print("metrics", m, flush=True)


@pytest.mark.parametrize("knobs", [(48, 64, 4, 3), (64, 32, 8, 2), (128, 64, 4, 3)])
def test_deepseek_shard_prefill_tile_kernel(ds_weights, knobs):
    """Row blocks above 32 rows go to the tile kernel: M=256 of the DeepSeek-V3 shard against the oracle."""
    P = make_problem(ds_weights, 256, seed=1)
    print(f"case ds M=256 knobs {knobs}", flush=True)
    m = assert_parity(run_op(P, *knobs, via="c_abi"), oracle_out(P), f"ds M=256 knobs {knobs}")
    print("metrics", m, flush=True)


def test_deepseek_shard_prefill_full_size_properties(ds_weights):
    """M=8192 (73 728 routed rows) is beyond what the oracle finishes in seconds, but a token's result depends on
    nothing but its own row, routing and the weights: the oracle recomputes a random sample of tokens as a
    48-token problem and must agree with the corresponding rows.  Two launches agree bit for bit (no atomics), and
    so do two row-block sizes (the per-slot sums do not depend on which rows share a block)."""
    from alpha_moe_python.workloads import Problem
    M = 8192
    P = make_problem(ds_weights, M, seed=2)
    print("case ds M=8192 knobs (128, 64, 4, 3)", flush=True)
    out = run_op(P, 128, 64, 4, 3, via="c_abi")
    gen = torch.Generator().manual_seed(7)
    idx = torch.randperm(M, generator=gen)[:48].sort().values.to(DEV)
    sub = Problem(ds_weights, 48, P.x[idx].contiguous(), P.x_scale[idx].contiguous(), P.topk_ids[idx].contiguous(),
                  P.topk_weights[idx].contiguous())
    m = assert_parity(out[idx], oracle_out(sub), "ds M=8192 sampled tokens")
    print("metrics", m, flush=True)
    print("case ds M=8192 second launch", flush=True)
    assert torch.equal(out, run_op(P, 128, 64, 4, 3, via="c_abi"))
    print("case ds M=8192 knobs (64, 64, 4, 3)", flush=True)
    assert torch.equal(out, run_op(P, 64, 64, 4, 3, via="c_abi"))


@pytest.mark.parametrize("M,knobs", [(512, (64, 64, 4, 3)), (2048, (96, 64, 4, 3))])
def test_deepseek_shard_prefill_mid_sizes(ds_weights, M, knobs):
    """The two mid prefill sizes of the DeepSeek-V3 shard with the knobs of the shipped tuning table: sampled tokens
    against the oracle (a token's result depends only on its own row, routing and the weights), and a second launch
    bit for bit."""
    P = make_problem(ds_weights, M, seed=3)
    print(f"case ds M={M} knobs {knobs}", flush=True)
    out = run_op(P, *knobs, via="c_abi")
    print("metrics", sampled_tokens_match_oracle(P, out, f"ds M={M} sampled tokens"), flush=True)
    print(f"case ds M={M} second launch", flush=True)
    assert torch.equal(out, run_op(P, *knobs, via="c_abi"))


def _sampled_tokens_match_oracle(P, out, what, n=48, seed=11):
    """A token's result depends on nothing but its own row, routing and the weights: recompute a sample on the CPU."""
    from alpha_moe_python.workloads import Problem
    gen = torch.Generator().manual_seed(seed)
    idx = torch.randperm(P.M, generator=gen)[:n].sort().values.to(DEV)
    sub = Problem(P.weights, n, P.x[idx].contiguous(), P.x_scale[idx].contiguous(), P.topk_ids[idx].contiguous(),
                  P.topk_weights[idx].contiguous())
    return assert_parity(out[idx], oracle_out(sub), what)


@pytest.fixture(scope="module")
def qn_weights():
    return make_weights(SHAPES["qn"], device=DEV, seed=0)


@pytest.mark.parametrize("M,knobs", [(1, (16, 32, 8, 5)), (32, (16, 32, 8, 5)), (256, (16, 64, 4, 3)), (256, (64, 64, 4, 3))])
def test_qwen3_next_shard_against_oracle(qn_weights, M, knobs):
    """Many small experts: E=512, top_k=10, K=2048, I=256, no shared expert (most experts idle at small M)."""
    P = make_problem(qn_weights, M, seed=0)
    print(f"case qn M={M} knobs {knobs}", flush=True)
    m = assert_parity(run_op(P, *knobs, via="c_abi"), oracle_out(P), f"qn M={M} knobs {knobs}")
    print("metrics", m, flush=True)


def test_qwen3_next_shard_prefill_full_size(qn_weights):
    P = make_problem(qn_weights, 4096, seed=1)
    print("case qn M=4096 knobs (64, 32, 8, 2)", flush=True)
    out = run_op(P, 64, 32, 8, 2, via="c_abi")
    print("metrics", _sampled_tokens_match_oracle(P, out, "qn M=4096 sampled tokens"), flush=True)
    print("case qn M=4096 knobs (128, 64, 4, 3)", flush=True)
    assert torch.equal(out, run_op(P, 128, 64, 4, 3, via="c_abi"))


@pytest.fixture(scope="module")
def q3_weights():
    return make_weights(SHAPES["q3"], device=DEV, seed=0)


@pytest.mark.parametrize("M,knobs", [(64, (16, 32, 8, 5)), (64, (32, 64, 4, 3)), (200, (64, 64, 4, 3)), (200, (128, 64, 4, 2))])
def test_qwen3_30b_zipf_shard_against_oracle(q3_weights, M, knobs):
    """Load imbalance: E=128, top_k=8, K=2048, I=768 (six 128-column slices), Zipf(1.2) expert popularity.  With six
    slices a 128-row block's requantised tiles do not fit LDS at once: its DOWN items serve the tokens in two parts."""
    P = make_problem(q3_weights, M, seed=0)
    print(f"case q3 M={M} knobs {knobs}", flush=True)
    m = assert_parity(run_op(P, *knobs, via="c_abi"), oracle_out(P), f"q3 M={M} knobs {knobs}")
    print("metrics", m, flush=True)


def test_qwen3_30b_zipf_shard_prefill_M1024(q3_weights):
    """M=1024 of the Zipf shard with the shipped table's knobs: the hot experts have many row blocks, most have one."""
    P = make_problem(q3_weights, 1024, seed=2)
    knobs = (64, 64, 4, 3)
    print(f"case q3 M=1024 knobs {knobs}", flush=True)
    out = run_op(P, *knobs, via="c_abi")
    print("metrics", sampled_tokens_match_oracle(P, out, "q3 M=1024 sampled tokens"), flush=True)
    print("case q3 M=1024 second launch", flush=True)
    assert torch.equal(out, run_op(P, *knobs, via="c_abi"))


def test_qwen3_30b_zipf_shard_prefill_full_size(q3_weights):
    P = make_problem(q3_weights, 8192, seed=1)
    print("case q3 M=8192 knobs (64, 32, 8, 3)", flush=True)
    out = run_op(P, 64, 32, 8, 3, via="c_abi")
    print("metrics", _sampled_tokens_match_oracle(P, out, "q3 M=8192 sampled tokens"), flush=True)
    print("case q3 M=8192 second launch", flush=True)
    assert torch.equal(out, run_op(P, 64, 32, 8, 3, via="c_abi"))


def test_short_up_items_repeat_launches():
    """Many row blocks, short K: the UP items are a few K blocks long, so item starts, ends (loads pointed past the end
    of an item) and LDS-ring reuse dominate.  Ten launches must all agree with the oracle and with each other."""
    from alpha_moe_python.workloads import Shape
    shape = Shape("short", E=512, top_k=10, K=1024, I=256, shared_expert=False, routing="softmax_renorm",
                  scaling_factor=1.0)
    W = make_weights(shape, device=DEV, seed=0)
    P = make_problem(W, 32, seed=0)
    ref = oracle_out(P)
    for knobs in ((16, 32, 8, 5), (16, 32, 8, 2), (16, 64, 4, 1), (16, 64, 4, 2),
                  (32, 32, 8, 5), (32, 64, 4, 2), (24, 32, 8, 3)):   # the last three: two token tiles per row block
        print(f"case short M=32 knobs {knobs}", flush=True)
        first = run_op(P, *knobs, via="c_abi")
        assert_parity(first, ref, f"short M=32 knobs {knobs}")
        for rep in range(9):
            assert torch.equal(first, run_op(P, *knobs, via="c_abi")), (knobs, rep)


@pytest.mark.parametrize("knobs", [(8, 64, 4, 2), (16, 64, 4, 5), (16, 32, 8, 4), (32, 64, 4, 3), (32, 32, 8, 5)])
def test_grid_fits_the_device(ds_weights, knobs):
    """The workgroups of a launch wait for each other, so the grid must not exceed what the device holds at once -
    also for ring sizes where the LDS allocation granule decides how many workgroups fit a CU.  A grid that is too
    large shows as a launch that takes seconds (bounded waits running out) and as wrong results."""
    import time
    P = make_problem(ds_weights, 64, seed=0)
    print(f"case ds M=64 knobs {knobs}", flush=True)
    run_op(P, *knobs, via="c_abi")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = run_op(P, *knobs, via="c_abi")
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert dt < 0.5, f"launch took {dt:.2f} s"
    assert_parity(out, oracle_out(P), f"ds M=64 knobs {knobs}")


def test_tile_kernel_result_independent_of_item_schedule():
    """The tile kernel's work items (up/gate slices, slabs of output columns) may run on any workgroup in any order
    that respects their flags: few workgroups (every one serves all eight queues), down items right behind their
    up/gate items, the smallest and the largest column slabs, cached or non-temporal weight loads - the output is
    the same bit for bit, and agrees with the oracle.  K=640 gives 10 column groups: the last slab is ragged and
    some wavefront pairs have no group in it."""
    from alpha_moe_python.workloads import Shape
    shape = Shape("sched", E=12, top_k=3, K=640, I=256, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0)
    W = make_weights(shape, device=DEV, seed=3)
    P = make_problem(W, 300, seed=3)
    ref = oracle_out(P)
    for block_m in (48, 128):
        print(f"case sched M=300 block_m {block_m} default schedule", flush=True)
        base = run_op(P, block_m, 64, 4, 3, via="c_abi")
        assert_parity(base, ref, f"sched block_m {block_m}")
        for env in ({"ALPHA_MOE_TILE_GRID": 8}, {"ALPHA_MOE_TILE_LAG": 1}, {"ALPHA_MOE_TILE_GPS": 4},
                    {"ALPHA_MOE_TILE_GPS": 1000}, {"ALPHA_MOE_TILE_NT": 1}, {"ALPHA_MOE_TILE_NT": 0},
                    {"ALPHA_MOE_TILE_GRID": 16, "ALPHA_MOE_TILE_LAG": 2, "ALPHA_MOE_TILE_GPS": 8}):
            print(f"case sched M=300 block_m {block_m} {env}", flush=True)
            with tunables(**env):
                got = run_op(P, block_m, 64, 4, 3, via="c_abi")
            assert torch.equal(got, base), (block_m, env)


@pytest.mark.parametrize("knobs", [(16, 32, 8, 5), (64, 64, 4, 3)])
def test_workspace_needs_only_its_prefix_zeroed(c1, knobs):
    """Everything behind alpha_moe_workspace_zero_bytes() may hold anything: fill it with 0xff."""
    import alpha_moe
    P, ref = c1
    s_ids, _, _ = P.align(knobs[0])
    need = alpha_moe.c_abi.alpha_moe_workspace_bytes(P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, s_ids.numel(),
                                                     knobs[0])
    ws = torch.full((need,), 255, dtype=torch.uint8, device=DEV)
    ws[: alpha_moe.c_abi.alpha_moe_workspace_zero_bytes()] = 0
    first = run_op(P, *knobs, via="c_abi", workspace=ws)
    assert_parity(first, ref, f"knobs {knobs}")
    assert torch.equal(first, run_op(P, *knobs, via="c_abi", workspace=ws))


@pytest.mark.parametrize("knobs,store", [((16, 32, 8, 5), False), ((16, 64, 4, 2), True), ((64, 64, 4, 3), False)])
def test_hip_graph_capture_and_replay(c1, knobs, store):
    """The operator allocates and synchronises nothing once it has run on a stream, so it can be captured into a HIP
    graph there.  Replays with new activations in the captured buffers agree bit for bit with eager calls, with eager
    work and synchronisations between the replays."""
    from alpha_moe_python.workloads import Problem
    P, _ = c1
    W = P.weights
    block_m = knobs[0]
    s_ids, e_ids, total = P.align(block_m)
    op = torch.ops.alpha_moe.fused_moe_w8a8_up_down_store if store else torch.ops.alpha_moe.fused_moe_w8a8_up_down
    x, xs, tw = P.x.clone(), P.x_scale.clone(), P.topk_weights.clone()
    out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16, device=DEV)

    def step():
        if not store:
            out.zero_()
        op(x, xs, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total, tw, out, P.shape.top_k, *knobs,
           P.shape.scaling_factor)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()   # first call on this stream: scratch is allocated and its prefix zeroed here, outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for rep in range(4):
        P2 = make_problem(W, P.M, seed=100 + rep)
        # new activations and routing weights, same routing (the captured sorted ids): copy into the captured buffers
        x.copy_(P2.x)
        xs.copy_(P2.x_scale)
        tw.copy_(P2.topk_weights)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager_problem = Problem(W, P.M, P2.x, P2.x_scale, P.topk_ids, P2.topk_weights)
        want = run_op(eager_problem, *knobs, via="c_abi")   # eager work between replays
        assert torch.equal(got, want), (knobs, store, rep)


def test_random_small_shapes_and_knobs():
    """Forty seeded random problems - token counts, expert counts, top_k, K (any multiple of 128, so also a single
    64-column group pair and ragged column slabs), one to five 128-column slices, every row-block size of both kernels -
    against the oracle."""
    import random
    from alpha_moe_python.workloads import Shape
    rng = random.Random(20240607)
    for case in range(40):
        E = rng.choice([1, 2, 3, 5, 8, 17])
        top_k = rng.randint(1, min(E, 4))
        K = 128 * rng.choice([1, 2, 3, 5, 8, 9])
        I = 128 * rng.choice([1, 1, 2, 3, 5])
        M = rng.choice([1, 2, 7, 16, 33, 100, 257])
        block_m = rng.choice([8, 16, 24, 32, 40, 64, 96, 128])
        bn, wn = rng.choice([(64, 4), (32, 8)])
        stages = rng.randint(1, 5)
        shape = Shape(f"rnd{case}", E=E, top_k=top_k, K=K, I=I, shared_expert=False, routing="softmax_renorm",
                      scaling_factor=rng.choice([1.0, 2.5]))
        W = make_weights(shape, device=DEV, seed=case)
        P = make_problem(W, M, seed=case)
        print(f"case rnd{case} E={E} top_k={top_k} K={K} I={I} M={M} knobs {(block_m, bn, wn, stages)}", flush=True)
        got = run_op(P, block_m, bn, wn, stages, via="c_abi")
        # The 1e-2 bar per token row, against the oracle or one of its neighbours within rounding-order noise of the
        # up/gate sums: a sum on a bf16 rounding boundary that decides a group's FP8 scale may fall on either side.
        assert_parity_rows(got, oracle_variants(P), f"rnd{case}")


@pytest.mark.parametrize("knobs", [(16, 32, 8, 5), (64, 64, 4, 3)])
def test_nothing_routed(c1, knobs):
    """No live row block at all (num_tokens_post_padded = 0), and row blocks whose expert id is out of range: the adding
    call leaves `out` as it was, the storing call writes zeros - both kernels."""
    import alpha_moe
    P, _ = c1
    W = P.weights
    block_m = knobs[0]
    s_ids, e_ids, total = P.align(block_m)
    for what in ("no blocks", "invalid experts"):
        tot = torch.zeros_like(total) if what == "no blocks" else total
        eid = e_ids if what == "no blocks" else torch.full_like(e_ids, -1)
        for store in (False, True):
            out = torch.full((P.M, P.shape.K), 0.5, dtype=torch.bfloat16, device=DEV)
            op = torch.ops.alpha_moe.fused_moe_w8a8_up_down_store if store else torch.ops.alpha_moe.fused_moe_w8a8_up_down
            print(f"case c1 {what} store={store} knobs {knobs}", flush=True)
            op(P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, eid, tot, P.topk_weights, out, P.shape.top_k,
               *knobs, P.shape.scaling_factor)
            torch.cuda.synchronize()
            assert torch.all(out == (0.0 if store else 0.5)), (what, store)


def test_workspace_check_reports_an_expired_wait(c1):
    """alpha_moe_workspace_check: 0 after ordinary launches of both kernels; 8 once the sticky word that a workgroup
    writes when its bounded wait runs out is set (set here from the host: no kernel is made to wait)."""
    import alpha_moe
    P, ref = c1
    need = max(alpha_moe.c_abi.alpha_moe_workspace_bytes(P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E,
                                                         P.align(bm)[0].numel(), bm) for bm in (16, 64))
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    for knobs in ((16, 32, 8, 5), (64, 64, 4, 3)):
        assert_parity(run_op(P, *knobs, via="c_abi", workspace=ws), ref, f"knobs {knobs}")
        assert alpha_moe.c_abi.alpha_moe_workspace_check(ws.data_ptr(), stream) == 0
    error_word = 33   # the control block's sticky error word (kErrorWord in csrc/moe_common.hpp)
    ws.view(torch.int32)[error_word] = 1
    rc = alpha_moe.c_abi.alpha_moe_workspace_check(ws.data_ptr(), stream)
    assert rc == 8 and b"wait" in alpha_moe.c_abi.alpha_moe_status_string(rc)
    # while the word is set, every call on the workspace says so in its output: NaN everywhere, adding or storing,
    # from the streaming kernel and from the tile kernel
    for knobs in ((16, 32, 8, 5), (64, 64, 4, 3)):
        for store in (False, True):
            got = run_op(P, *knobs, via="c_abi", workspace=ws, store=store)
            assert torch.isnan(got.float()).all(), (knobs, store)
    ws.view(torch.int32)[error_word] = 0
    assert_parity(run_op(P, 16, 32, 8, 5, via="c_abi", workspace=ws), ref, "after clearing the error word")
    # An expiry DURING a launch of the streaming kernel reaches the closing items through the counter they poll: the
    # waiter sets a high bit in it (an OR, so the value below is what the kernel produces).  Set from the host here, the bit makes that one launch answer NaN (its closing items
    # do not wait and do not trust what they read); the launch resets the counter, and the next one is clean again.
    down_counter, expired_bit = 32, 1 << 30   # StreamCtl::down_done and kExpiredBit in csrc/moe_common.hpp
    ws.view(torch.int32)[down_counter] = expired_bit
    got = run_op(P, 16, 32, 8, 5, via="c_abi", workspace=ws)
    assert torch.isnan(got.float()).all()
    assert_parity(run_op(P, 16, 32, 8, 5, via="c_abi", workspace=ws), ref, "the launch after a marked counter")
    assert alpha_moe.c_abi.alpha_moe_workspace_check(ws.data_ptr(), stream) == 0


def test_queue_survives_a_grid_the_device_cannot_hold(ds_weights):
    """No workgroup owns an item before it runs, so even a grid of four times what the device holds at once
    (workgroups that start only when others have left) finishes at once and correctly - the property callers need who
    overlap launches on several streams.  Handing the first items out by workgroup index (ALPHA_MOE_STRICT_QUEUE=0, an
    experiment switch) gives the same result on a grid the device holds."""
    import time
    P = make_problem(ds_weights, 16, seed=4)
    base = run_op(P, 16, 32, 8, 5, via="c_abi")
    assert_parity(base, oracle_out(P), "ds M=16")
    with tunables(ALPHA_MOE_STRICT_QUEUE=0):
        assert torch.equal(run_op(P, 16, 32, 8, 5, via="c_abi"), base)
    with tunables(ALPHA_MOE_GRID=1024):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        got = run_op(P, 16, 32, 8, 5, via="c_abi")
        dt = time.perf_counter() - t0
    assert dt < 0.5, f"launch took {dt:.2f} s"
    assert torch.equal(got, base)
    P = make_problem(ds_weights, 48, seed=4)   # whole-K UP items
    base = run_op(P, 16, 32, 8, 5, via="c_abi")
    with tunables(ALPHA_MOE_GRID=1024):
        assert torch.equal(run_op(P, 16, 32, 8, 5, via="c_abi"), base)


def test_two_streams_at_once(ds_weights):
    """Two launches in flight at the same time on two streams, each with a workspace of its own: both finish at once
    and agree bit for bit with launches that ran alone."""
    import time
    import alpha_moe
    P1 = make_problem(ds_weights, 32, seed=5)
    P2 = make_problem(ds_weights, 24, seed=6)
    knobs = (16, 32, 8, 5)
    alone = [run_op(P, *knobs, via="c_abi") for P in (P1, P2)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs, keep = [], []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for rep in range(5):
        for P, st in zip((P1, P2), streams):
            with torch.cuda.stream(st):
                s_ids, e_ids, total = P.align(knobs[0])
                need = alpha_moe.c_abi.alpha_moe_workspace_bytes(P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E,
                                                                 s_ids.numel(), knobs[0])
                ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
                out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16, device=DEV)
                W = P.weights
                rc = alpha_moe.c_abi.alpha_moe_fused_moe_w8a8_up_down(
                    P.x.data_ptr(), P.x_scale.data_ptr(), W.w1.data_ptr(), W.w1_scale.data_ptr(), W.w2.data_ptr(),
                    W.w2_scale.data_ptr(), out.data_ptr(), s_ids.data_ptr(), e_ids.data_ptr(), total.data_ptr(),
                    P.topk_weights.data_ptr(), P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, s_ids.numel(),
                    *knobs, float(P.shape.scaling_factor), ws.data_ptr(), ws.numel(), st.cuda_stream)
                assert rc == 0
                outs.append(out)
                keep.append((ws, s_ids, e_ids, total))
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert dt < 1.0, f"ten overlapping launches took {dt:.2f} s"
    for i, out in enumerate(outs):
        assert torch.equal(out, alone[i % 2]), i


@pytest.mark.parametrize("name", ["ds", "qn"])
def test_tiny_batches(name, ds_weights, qn_weights):
    """M in {1, 2, 4, 8, 16}: K-split UP items whose partial sums the last arrival adds up (in batches of eight
    splits), on both shards, several knobs, adding and storing, two launches bit for bit; against the oracle.  The 1e-2
    bar holds on every size: on the benchmark sizes against the oracle as it is, on the sizes in between per token row
    against the oracle or its neighbours within rounding-order noise of the up/gate sums (at M=2 of the DeepSeek-V3
    shard one up-projection sum of the shared expert, the largest activation of its group, sits 6e-6 of its size from a
    bf16 rounding boundary; the device's K-split sum falls on the other side, the group's FP8 scale moves by 0.6 %, 12
    of its 128 codes re-round and that token moves by 1.2e-2 of the output range - see test_an_up_sum_on_a_bf16_boundary)."""
    W = ds_weights if name == "ds" else qn_weights
    benchmark_sizes = (1, 4, 16) if name == "ds" else (1,)
    for M in (1, 2, 4, 8, 16):
        P = make_problem(W, M, seed=20 + M)
        ref = oracle_out(P)
        variants = None if M in benchmark_sizes else oracle_variants(P)
        for knobs in ((16, 32, 8, 5), (16, 64, 4, 3), (8, 32, 8, 2), (32, 64, 4, 4)):
            print(f"case {name} M={M} knobs {knobs}", flush=True)
            got = run_op(P, *knobs, via="c_abi")
            if M in benchmark_sizes:
                assert_parity(got, ref, f"{name} M={M} knobs {knobs}")
            else:
                assert_parity_rows(got, variants, f"{name} M={M} knobs {knobs}")
            assert torch.equal(got, run_op(P, *knobs, via="c_abi")), (name, M, knobs)
            junk = torch.full((P.M, P.shape.K), float("nan"), dtype=torch.bfloat16, device=DEV)
            assert torch.equal(run_op(P, *knobs, out=junk, via="c_abi", store=True), got), (name, M, knobs, "store")
        pre = torch.full((P.M, P.shape.K), 0.25, dtype=torch.bfloat16, device=DEV)
        assert_parity_rows(run_op(P, 16, 32, 8, 5, out=pre.clone(), via="c_abi"), oracle_variants(P, out=pre.cpu()),
                           f"{name} M={M} out pre-filled")


def test_an_up_sum_on_a_bf16_boundary(ds_weights):
    """The one problem on which the device and the oracle disagree by more than the bar (DeepSeek-V3 shard, M=2): the
    disagreement is the oracle's own discontinuity.  Seventeen of the eighteen (token, slot) rows agree; in the shared
    expert's row of token 0 the up-projection sum of the group's largest activation is -3.429666, at 0.4986 of the way
    between two bf16 values, and moving the oracle's sums by 1e-5 of their size moves its answer for that token by 1.2e-2
    of the output range - onto the device's."""
    from oracle import moe_oracle as O
    P = make_problem(ds_weights, 2, seed=22)
    got = run_op(P, 16, 32, 8, 5, via="c_abi")
    plain, up, down = oracle_variants(P)
    scale = float(plain.float().abs().max())
    row = lambda a, b, t: float((a[t].float().cpu() - b[t].float().cpu()).abs().max()) / scale
    # the oracle against itself, sums moved by 1e-5: token 0 jumps, token 1 does not
    assert max(row(plain, up, 0), row(plain, down, 0)) > 1e-2
    assert max(row(plain, up, 1), row(plain, down, 1)) <= 5e-3
    # the device is within the bar of the neighbour and, on token 1, of the oracle as it is
    assert min(row(got, up, 0), row(got, down, 0)) <= 5e-3
    assert row(got, plain, 1) <= 5e-3
    assert O.error_metrics(got, plain)["cosine"] >= 0.9999


def test_tiny_batch_duplicates_padding_and_missing_experts():
    """A tiny batch with what makes the bookkeeping interesting: a token that picks one expert twice (two rows of one
    block), row blocks whose expert id is out of range (skipped), K % 256 == 128, three 128-column slices."""
    shape = Shape("t", E=6, top_k=4, K=384, I=384, shared_expert=False, routing="softmax_renorm", scaling_factor=2.5,
                  w_std=0.05)
    W = make_weights(shape, device=DEV, seed=3)
    P = make_problem(W, 12, seed=3)
    g = torch.Generator(device=DEV).manual_seed(7)
    P.topk_ids = torch.randint(0, 6, (12, 4), generator=g, device=DEV, dtype=torch.int32)   # with replacement
    P.aligned.clear()
    ref = oracle_out(P)
    for knobs in ((8, 32, 8, 3), (16, 64, 4, 2), (32, 32, 8, 5)):
        print(f"case tiny dup knobs {knobs}", flush=True)
        got = run_op(P, *knobs, via="c_abi")
        assert_parity(got, ref, f"tiny dup knobs {knobs}")
        assert torch.equal(got, run_op(P, *knobs, via="c_abi"))
    # experts 4 and 5 declared missing: their blocks are skipped, the others' results stay
    s_ids, e_ids, total = P.align(16)
    e_bad = torch.where(e_ids >= 4, torch.full_like(e_ids, -1), e_ids)
    P.aligned[16] = (s_ids, e_bad, total)
    keep = (P.topk_ids < 4)
    saved = P.topk_weights
    try:
        print("case tiny missing experts", flush=True)
        got = run_op(P, 16, 32, 8, 4, via="c_abi")
        P.aligned.clear()
        P.topk_weights = saved * keep   # the same thing said through the routing weights
        want = oracle_out(P)
    finally:
        P.topk_weights = saved
        P.aligned.clear()
    assert_parity(got, want, "tiny missing experts")


def test_ring_depth_is_clamped_to_what_lds_holds():
    """block_m = 32 with stages = 5 and twelve 128-column slices asks for more LDS than a compute unit has next to the
    item tables: the ring is made shallower instead of the launch failing."""
    shape = Shape("wide", E=4, top_k=2, K=256, I=1536, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0,
                  w_std=0.05)
    W = make_weights(shape, device=DEV, seed=1)
    P = make_problem(W, 40, seed=1)
    ref = oracle_out(P)
    for knobs in ((32, 64, 4, 5), (32, 32, 8, 5), (16, 64, 4, 5)):
        print(f"case wide I=1536 knobs {knobs}", flush=True)
        assert_parity(run_op(P, *knobs, via="c_abi"), ref, f"wide knobs {knobs}")


def test_eager_calls_of_growing_size_keep_one_scratch_buffer(c1):
    """The binding's scratch buffer of a stream that only ever runs eager calls: twenty calls of growing size leave ONE
    buffer alive (replaced buffers go back to the allocator; growth is geometric, so few of the calls reallocate), and
    the results stay right across the replacements."""
    P0, _ = c1
    W = P0.weights
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    sizes, allocations, last = [], 0, 0
    with torch.cuda.stream(side):
        for i in range(20):
            M = 16 + 40 * i
            Q = make_problem(W, M, seed=100 + i)
            knobs = (64, 32, 8, 2) if i % 2 else (16, 64, 4, 3)
            got = run_op(Q, *knobs, via="torch")
            n_alive, current, retired = torch.ops.alpha_moe.scratch_buffers(Q.x)
            assert n_alive == 1 and retired == 0, (i, n_alive, retired)
            allocations += current != last
            last = current
            sizes.append(current)
            if i in (0, 7, 19):
                assert_parity(got, oracle_out(Q), f"growing sizes, call {i}")
    assert sizes == sorted(sizes) and allocations <= 10, (sizes, allocations)


def test_scratch_regrowth_after_graph_capture(c1):
    """A graph captured on a stream keeps replaying into the scratch buffer the stream had then, also after a larger
    eager call on the same stream made the binding take a bigger buffer; growth DURING capture is refused with an
    error that names the remedy, and reserve_workspace makes the capture of the larger call possible."""
    P, _ = c1
    W = P.weights
    knobs = (16, 32, 8, 3)
    s_ids, e_ids, total = P.align(16)
    out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16, device=DEV)

    def step(Q, ids, o, kn):
        o.zero_()
        torch.ops.alpha_moe.fused_moe_w8a8_up_down(Q.x, Q.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, *ids,
                                                   Q.topk_weights, o, Q.shape.top_k, *kn, Q.shape.scaling_factor)

    big = make_problem(W, 600, seed=8)
    big_knobs = (128, 64, 4, 3)
    big_ids = big.align(128)
    big_out = torch.zeros((big.M, big.shape.K), dtype=torch.bfloat16, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(P, (s_ids, e_ids, total), out, knobs)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(P, (s_ids, e_ids, total), out, knobs)
        # a larger call during another capture on this stream: refused, nothing recorded
        g2 = torch.cuda.CUDAGraph()
        with pytest.raises(RuntimeError, match="reserve_workspace"):
            with torch.cuda.graph(g2, stream=side):
                step(big, big_ids, big_out, big_knobs)
        side.synchronize()
        want = run_op(P, *knobs, via="c_abi")
        graph.replay()
        side.synchronize()
        assert torch.equal(out, want)
        # the larger call, eagerly, on the capture stream: the binding takes a bigger buffer ...
        step(big, big_ids, big_out, big_knobs)
        side.synchronize()
        assert torch.equal(big_out, run_op(big, *big_knobs, via="c_abi"))
        n_alive, _, retired = torch.ops.alpha_moe.scratch_buffers(P.x)
        assert n_alive == 2 and retired > 0   # the buffer the graph was captured with is kept beside the new one
        # ... and the graph still replays into the one it was captured with
        for _ in range(3):
            out.fill_(7.0)
            graph.replay()
            side.synchronize()
            assert torch.equal(out, want)
            step(big, big_ids, big_out, big_knobs)
        side.synchronize()
    # reserve first, then even the first call of a size may be captured
    side2 = torch.cuda.Stream()
    side2.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side2):
        need = torch.ops.alpha_moe.workspace_bytes(big.shape.top_k, big.M, big.shape.K, big.shape.N, big.shape.E,
                                                   big_ids[0].numel(), 128)
        torch.ops.alpha_moe.reserve_workspace(big.x, need)
        side2.synchronize()
        g3 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g3, stream=side2):
            step(big, big_ids, big_out, big_knobs)
        big_out.fill_(3.0)
        g3.replay()
        side2.synchronize()
        assert torch.equal(big_out, run_op(big, *big_knobs, via="c_abi"))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.current_stream().wait_stream(side2)
    torch.cuda.synchronize()


def _run_prepacked(P, packed, knobs, store=False, via="c_abi", out=None):
    import alpha_moe
    wp, w2p = packed
    W = P.weights
    s_ids, e_ids, total = P.align(knobs[0])
    if out is None:
        out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16, device=DEV)
    if via == "torch":
        torch.ops.alpha_moe.fused_moe_w8a8_up_down_prepacked(P.x, P.x_scale, wp, W.w1_scale, w2p, W.w2_scale, s_ids, e_ids,
                                                             total, P.topk_weights, out, P.shape.top_k, *knobs,
                                                             P.shape.scaling_factor, store)
    else:
        need = alpha_moe.c_abi.alpha_moe_workspace_bytes(P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, s_ids.numel(), knobs[0])
        ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
        rc = alpha_moe.c_abi.alpha_moe_fused_moe_w8a8_up_down_prepacked(
            P.x.data_ptr(), P.x_scale.data_ptr(), wp.data_ptr(), W.w1_scale.data_ptr(), w2p.data_ptr(),
            W.w2_scale.data_ptr(), out.data_ptr(), s_ids.data_ptr(), e_ids.data_ptr(), total.data_ptr(),
            P.topk_weights.data_ptr(), P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, s_ids.numel(), *knobs,
            float(P.shape.scaling_factor), 1 if store else 0, ws.data_ptr(), ws.numel(),
            torch.cuda.current_stream().cuda_stream)
        assert rc == 0, alpha_moe.c_abi.alpha_moe_status_string(rc)
    torch.cuda.synchronize()
    return out


def test_prepacked_weights_give_the_same_bits(c1, ds_weights, q3_weights):
    """fused_moe_w8a8_up_down_prepacked on prepack_weights(w, w2) against the operator on w, w2: bit for bit, streaming
    and tile kernels, adding and storing, torch op and C ABI - on the CPU-sized case, the DeepSeek-V3 shard at M=256 and
    the Zipf shard at M=200 (six slices)."""
    from alpha_moe_python.utils import prepack_weights
    P, ref = c1
    packed = prepack_weights(P.weights.w1, P.weights.w2)
    for knobs in ((16, 32, 8, 5), (16, 64, 4, 2), (32, 64, 4, 3), (64, 64, 4, 3), (128, 64, 4, 3)):
        print(f"case prepacked c1 knobs {knobs}", flush=True)
        want = run_op(P, *knobs, via="c_abi")
        for via in ("c_abi", "torch"):
            assert torch.equal(_run_prepacked(P, packed, knobs, via=via), want), (knobs, via)
        junk = torch.full((P.M, P.shape.K), float("nan"), dtype=torch.bfloat16, device=DEV)
        assert torch.equal(_run_prepacked(P, packed, knobs, store=True, out=junk), want), (knobs, "store")
    assert_parity(_run_prepacked(P, packed, (16, 32, 8, 5)), ref, "prepacked c1")
    for W, M, knob_list in ((ds_weights, 256, ((16, 64, 4, 3), (64, 64, 4, 3), (128, 64, 4, 3))),
                            (q3_weights, 200, ((16, 32, 8, 5), (64, 64, 4, 3), (128, 64, 4, 2)))):
        Q = make_problem(W, M, seed=1)
        packed = prepack_weights(W.w1, W.w2)
        for knobs in knob_list:
            print(f"case prepacked {W.shape.name} M={M} knobs {knobs}", flush=True)
            assert torch.equal(_run_prepacked(Q, packed, knobs), run_op(Q, *knobs, via="c_abi")), (W.shape.name, knobs)
        del packed
    # shapes only the fallback kernel takes are refused for pre-packed weights
    import alpha_moe
    shape = Shape("fb", E=2, top_k=1, K=16512, I=128, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0)
    Wf = make_weights(shape, device=DEV, seed=5)
    Pf = make_problem(Wf, 8, seed=5)
    with pytest.raises(AssertionError):
        _run_prepacked(Pf, prepack_weights(Wf.w1, Wf.w2), (128, 64, 4, 2))


# ---- the reference's correctness sweep on real-K problems, and the shipped tuning tables on several seeds ----------
def test_every_knob_on_the_deepseek_shard_M32(ds_weights):
    """test_moe_correctness.py:172-190 of the reference runs every (block_m, block_n/warp_n, stages) it accepts on
    K = 7168: 56 K blocks, so K-split counts, ring wrap-around, LDS clamps and item sizes differ per knob set.  All 160
    against one oracle result (the routing arrays depend on block_m, the result does not)."""
    P = make_problem(ds_weights, 32, seed=41)
    ref = oracle_out(P)
    worst = 0.0
    for knobs in ALL_KNOBS:
        print(f"case ds M=32 knobs {knobs}", flush=True)
        worst = max(worst, assert_parity(run_op(P, *knobs, via="c_abi"), ref, f"ds M=32 knobs {knobs}")["max_abs_over_max_ref"])
    print(f"worst of {len(ALL_KNOBS)} knob sets: {worst:.2e}", flush=True)


def test_every_knob_on_a_37_expert_shape_M128():
    """The reference's sweep shape E = 37, N = 256, K = 4096, shared expert last (test_moe_correctness.py:133,172-190),
    M = 128: every accepted knob set against one oracle result."""
    shape = Shape("e37", E=37, top_k=9, K=4096, I=128, shared_expert=True, routing="softmax_shared", scaling_factor=2.5)
    W = make_weights(shape, device=DEV, seed=37)
    P = make_problem(W, 128, seed=37)
    ref = oracle_out(P)
    worst = 0.0
    for knobs in ALL_KNOBS:
        print(f"case e37 M=128 knobs {knobs}", flush=True)
        worst = max(worst, assert_parity(run_op(P, *knobs, via="c_abi"), ref, f"e37 M=128 knobs {knobs}")["max_abs_over_max_ref"])
    print(f"worst of {len(ALL_KNOBS)} knob sets: {worst:.2e}", flush=True)


SHIPPED = {"ds": ("moe_jit_257_512_7168.json", (1, 4, 16, 64, 512, 2048, 8192)),
           "qn": ("moe_jit_512_512_2048.json", (1, 32, 256, 4096)),
           "q3": ("moe_jit_128_1536_2048.json", (64, 1024, 8192))}


@pytest.mark.parametrize("name", ["ds", "qn", "q3"])
def test_shipped_tables_on_four_seeds(name, ds_weights, qn_weights, q3_weights):
    """Every benchmark size with the knobs the shipped tuning table gives for it (what bench.py and callers run), on
    four seeds each: the worst token row stays within the bar.  Sizes up to 64 tokens are checked whole, larger ones on
    a sample of 32 tokens recomputed by the oracle as a problem of their own."""
    import os
    from alpha_moe_python.utils import get_best_config
    table, sizes = SHIPPED[name]
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "alpha-moe_amd", "configs", table)
    W = {"ds": ds_weights, "qn": qn_weights, "q3": q3_weights}[name]
    for M in sizes:
        cfg = get_best_config(path, M)
        knobs = (cfg["block_m"], cfg["block_n"], cfg["warp_n"], cfg["stages"])
        worst = 0.0
        for seed in (101, 102, 103, 104):
            P = make_problem(W, M, seed=seed)
            got = run_op(P, *knobs, via="c_abi")
            worst = max(worst, worst_row_error(P, got, n=32 if M > 64 else None, seed=seed))
        print(f"{name} M={M} knobs {knobs}: worst row of four seeds {worst:.2e}", flush=True)
