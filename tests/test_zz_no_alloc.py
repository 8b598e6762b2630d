"""The entry point that allocates nothing (alpha_moe_fused_moe_w8a8_up_down_static): scratch memory is a buffer built
into the library.  Collected last on purpose: it must pass alone in a fresh process and after every other test."""
import pytest
import torch

from alpha_moe_python.workloads import SHAPES, make_problem, make_weights
from gpu_util import assert_parity, oracle_out, run_op

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run_static(P, block_m, block_n, warp_n, stages, out=None):
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
