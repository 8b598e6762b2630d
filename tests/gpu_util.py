"""Shared helpers of the GPU parity tests: run the operator (through torch.ops or straight through the C ABI)
and the CPU oracle on the same bits."""
import contextlib

import torch

from oracle import moe_oracle as O

# north-star bar for the bf16 output: max |err| <= 1e-2 * max |ref| and cosine >= 0.9999
# (accumulation order of the bf16 atomics differs from run to run); routing/indexing is bit-exact.
MAX_ABS_OVER_MAX_REF = 1e-2
MIN_COSINE = 0.9999


def run_op(P, block_m, block_n, warp_n, stages, out=None, scaling=None, via="torch", workspace=None, store=False):
    import alpha_moe
    W = P.weights
    s_ids, e_ids, total = P.align(block_m)
    if out is None:
        out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16, device=P.x.device)
    scaling = P.shape.scaling_factor if scaling is None else scaling
    if via == "torch":
        op = torch.ops.alpha_moe.fused_moe_w8a8_up_down_store if store else torch.ops.alpha_moe.fused_moe_w8a8_up_down
        op(P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids,
                                                   total, P.topk_weights, out, P.shape.top_k, block_m, block_n, warp_n,
                                                   stages, scaling)
    else:
        stream = torch.cuda.current_stream().cuda_stream
        ws_bytes = alpha_moe.c_abi.alpha_moe_workspace_bytes(P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, s_ids.numel(), block_m)
        ws = workspace if workspace is not None else torch.zeros(ws_bytes, dtype=torch.uint8, device=P.x.device)
        assert ws.numel() >= ws_bytes
        entry = (alpha_moe.c_abi.alpha_moe_fused_moe_w8a8_up_down_store if store
                 else alpha_moe.c_abi.alpha_moe_fused_moe_w8a8_up_down)
        rc = entry(
            P.x.data_ptr(), P.x_scale.data_ptr(), W.w1.data_ptr(), W.w1_scale.data_ptr(), W.w2.data_ptr(),
            W.w2_scale.data_ptr(), out.data_ptr(), s_ids.data_ptr(), e_ids.data_ptr(), total.data_ptr(),
            P.topk_weights.data_ptr(), P.shape.top_k, P.M, P.shape.K, P.shape.N, P.shape.E, s_ids.numel(), block_m,
            block_n, warp_n, stages, float(scaling), ws.data_ptr(), ws.numel(), stream)
        assert rc == 0, alpha_moe.c_abi.alpha_moe_status_string(rc)


    torch.cuda.synchronize()
    return out


def oracle_out(P, block_m=16, out=None, scaling=None, accumulate="dense", up_nudge=0.0):
    W = P.weights
    s_ids, e_ids, total = P.align(block_m)
    if out is None:
        out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16)
    scaling = P.shape.scaling_factor if scaling is None else scaling
    return O.fused_moe_oracle(P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total,
                              P.topk_weights, out, P.shape.top_k, block_m, scaling, accumulate=accumulate,
                              up_nudge=up_nudge)


def assert_parity(out, ref, what=""):
    m = O.error_metrics(out, ref)
    assert torch.isfinite(out.float()).all(), what
    assert m["max_abs_over_max_ref"] <= MAX_ABS_OVER_MAX_REF and m["cosine"] >= MIN_COSINE, (what, m)
    return m


# The operator is discontinuous in its fp32 up/gate sums (bf16 rounding, then an FP8 scale per 128 columns taken from
# the largest activation): a sum within rounding-order noise of a bf16 boundary may legitimately fall on either side.
# The oracle recomputed with its sums moved by this relative amount, either way, brackets that noise.
UP_SUM_NOISE = 1e-5


def oracle_variants(P, block_m=16, out=None, scaling=None):
    """The oracle and its two neighbours within rounding-order noise of the up/gate sums."""
    return [oracle_out(P, block_m, out, scaling, up_nudge=d) for d in (0.0, UP_SUM_NOISE, -UP_SUM_NOISE)]


def assert_parity_rows(out, refs, what=""):
    """The parity bar per token row against the nearest of `refs` (oracle_variants): every row within 1e-2 of the
    output range of one of them, and the whole output at cosine >= 0.9999 with the first.  Returns the worst row."""
    o = out.detach().float().cpu()
    assert torch.isfinite(o).all(), what
    scale = refs[0].float().abs().max().clamp_min(1e-30)
    per_row = torch.stack([(o - r.float()).abs().amax(dim=1) for r in refs]).amin(dim=0) / scale
    m = O.error_metrics(out, refs[0])
    assert float(per_row.max()) <= MAX_ABS_OVER_MAX_REF and m["cosine"] >= MIN_COSINE, (what, float(per_row.max()), m)
    return float(per_row.max())


@contextlib.contextmanager
def tunables(**values):
    """Tuning overrides of the library for the duration of a with-block: tunables(ALPHA_MOE_TILE_GRID=8)."""
    import alpha_moe
    for name, value in values.items():
        alpha_moe.set_tunable(name, value)
    try:
        yield
    finally:
        for name in values:
            alpha_moe.set_tunable(name, None)


def sampled_tokens_match_oracle(P, out, what, n=48, seed=11):
    """A token's result depends on nothing but its own row, routing and the weights: the oracle recomputes a random
    sample of the tokens as an n-token problem of its own."""
    sub, idx = sample_problem(P, n, seed)
    return assert_parity(out[idx], oracle_out(sub), what)


def sample_problem(P, n, seed):
    from alpha_moe_python.workloads import Problem
    gen = torch.Generator().manual_seed(seed)
    idx = torch.randperm(P.M, generator=gen)[:n].sort().values.to(P.x.device)
    sub = Problem(P.weights, idx.numel(), P.x[idx].contiguous(), P.x_scale[idx].contiguous(), P.topk_ids[idx].contiguous(),
                  P.topk_weights[idx].contiguous())
    return sub, idx


def worst_row_error(P, out, n=None, seed=11):
    """max |err| / max |ref| of the worst token row (of a sample of n tokens when n is given), against the oracle as it
    is; where that exceeds the bar, against the nearest of the oracle's neighbours within rounding-order noise of the
    up/gate sums (assert_parity_rows), which then also checks the bar."""
    sub, idx = (P, None) if n is None or n >= P.M else sample_problem(P, n, seed)
    got = out if idx is None else out[idx]
    ref = oracle_out(sub)
    m = O.error_metrics(got, ref)
    assert torch.isfinite(got.float()).all() and m["cosine"] >= MIN_COSINE, m
    if m["max_abs_over_max_ref"] <= MAX_ABS_OVER_MAX_REF:
        return m["max_abs_over_max_ref"]
    return assert_parity_rows(got, oracle_variants(sub), f"M={P.M} sample seed {seed}")
