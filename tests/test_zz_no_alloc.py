"""The entry point that allocates nothing (alpha_moe_fused_moe_w8a8_up_down_static): scratch memory is a buffer built
into the library.  Collected last on purpose: it must pass alone in a fresh process and after every other test."""
import pytest
import torch

from alpha_moe_python.workloads import SHAPES, make_problem, make_weights
from gpu_util import assert_parity, oracle_out, run_op

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run_static(P, block_m, block_n, warp_n, stages, out=None, sync=True):
    import alpha_moe
    W = P.weights
    s_ids, e_ids, total = P.align(block_m)
    if out is None:
        out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16, device=P.x.device)
    rc = alpha_moe.c_abi.alpha_moe_fused_moe_w8a8_up_down_static(
        P.x.data_ptr(), P.x_scale.data_ptr(), W.w1.data_ptr(), W.w1_scale.data_ptr(), W.w2.data_ptr(),
        W.w2_scale.data_ptr(), out.data_ptr(), s_ids.data_ptr(), e_ids.data_ptr(), total.data_ptr(),
        P.topk_weights.data_ptr(), P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, s_ids.numel(), block_m,
            block_n, warp_n, stages, float(P.shape.scaling_factor), torch.cuda.current_stream().cuda_stream)
    if sync:
        torch.cuda.synchronize()
    return rc, out


def test_static_scratch_entry_point_matches_the_workspace_entry_point():
    """Two calls in a row, the second with a smaller input, each bit for bit what the entry point with a caller's
    workspace returns (and within the parity bar of the oracle); then a tile-kernel call, a call that adds into a
    pre-filled `out`, and a call too large for the built-in buffer, which is refused without launching anything."""
    W = make_weights(SHAPES["ds"], device=DEV, seed=0)
    big = make_problem(W, 48, seed=31)
    small = make_problem(W, 3, seed=32)
    for P, knobs in ((big, (16, 32, 8, 4)), (small, (16, 32, 8, 5)), (big, (16, 64, 4, 3)), (small, (8, 64, 4, 2))):
        print(f"case static ds M={P.M} knobs {knobs}", flush=True)
        want = run_op(P, *knobs, via="c_abi")
        rc, got = run_static(P, *knobs)
        assert rc == 0
        assert torch.equal(got, want), (P.M, knobs)
        assert_parity(got, oracle_out(P, knobs[0]), f"static ds M={P.M}")
    Wc = make_weights(SHAPES["c1"], device=DEV, seed=0)
    mid = make_problem(Wc, 200, seed=33)
    print("case static c1 M=200 tile kernel", flush=True)
    rc, got = run_static(mid, 64, 64, 4, 3)
    assert rc == 0 and torch.equal(got, run_op(mid, 64, 64, 4, 3, via="c_abi"))
    pre = torch.full((small.M, small.shape.K), 0.5, dtype=torch.bfloat16, device=DEV)
    rc, got = run_static(small, 16, 32, 8, 5, out=pre.clone())
    assert rc == 0 and torch.equal(got, run_op(small, 16, 32, 8, 5, out=pre.clone(), via="c_abi"))
    print("case static ds M=2048: refused", flush=True)
    huge = make_problem(W, 2048, seed=34)
    keep = torch.full((huge.M, huge.shape.K), 0.5, dtype=torch.bfloat16, device=DEV)
    rc, got = run_static(huge, 128, 64, 4, 3, out=keep)
    import alpha_moe
    assert rc == 9 and b"scratch" in alpha_moe.c_abi.alpha_moe_status_string(rc)
    assert torch.all(got == 0.5)


def test_static_entry_point_allocates_nothing_and_replays_from_a_graph():
    """What the entry point exists for: after the first call on the device (which looks the buffer's address up), calls
    leave the device's free memory and torch's allocation count where they were - streaming, tile, wide and fallback
    kernels - and a call captured into a HIP graph replays bit for bit.  The health check and the reset of the built-in
    buffer run in between and change no result."""
    import alpha_moe
    from alpha_moe_python.workloads import Shape
    stream = torch.cuda.current_stream().cuda_stream
    Wc = make_weights(SHAPES["c1"], device=DEV, seed=0)
    P = make_problem(Wc, 40, seed=41)
    fb_shape = Shape("fb", E=4, top_k=2, K=16512, I=128, shared_expert=False, routing="softmax_renorm", scaling_factor=1.0)
    Pf = make_problem(make_weights(fb_shape, device=DEV, seed=6), 20, seed=42)   # 129 K blocks: the fallback kernel
    cases = [(P, (16, 32, 8, 3)), (P, (64, 64, 4, 3)), (P, (128, 32, 8, 2)), (Pf, (64, 64, 4, 2))]
    want, outs = [], []
    for Q, knobs in cases:   # warm-up: symbol lookup, function attributes, aligned routing arrays, reference results
        want.append(run_op(Q, *knobs, via="c_abi"))
        outs.append(torch.zeros_like(want[-1]))
        rc, _ = run_static(Q, *knobs)
        assert rc == 0
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    n_alloc0 = torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(2):
        for (Q, knobs), o in zip(cases, outs):
            o.zero_()
            rc, _ = run_static(Q, *knobs, out=o)
            assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == n_alloc0
    for o, w, (Q, knobs) in zip(outs, want, cases):
        if Q is Pf:
            assert_parity(o, w, "fallback kernel sums with atomics")   # agrees to rounding, not bit for bit
        else:
            assert torch.equal(o, w), knobs
    assert alpha_moe.c_abi.alpha_moe_static_scratch_check(stream) == 0
    # captured into a graph on a side stream: replays give the eager result
    Q, knobs = cases[0]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        o = outs[0]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            o.zero_()
            rc, _ = run_static(Q, *knobs, out=o, sync=False)
        assert rc == 0
        for _ in range(3):
            o.fill_(3.0)
            graph.replay()
            side.synchronize()
            assert torch.equal(o, want[0])
        side.synchronize()
    # the reset clears the buffer's control prefix; the next call starts from a clean state and gives the same bits
    assert alpha_moe.c_abi.alpha_moe_static_scratch_reset(stream) == 0
    torch.cuda.synchronize()
    rc, got = run_static(Q, *knobs)
    assert rc == 0 and torch.equal(got, want[0])
    assert alpha_moe.c_abi.alpha_moe_static_scratch_check(stream) == 0
