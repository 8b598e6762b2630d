"""Pins the CPU oracle: fp8 codec vs the library dtype, two independent restatements against each other,
a routing-free per-token loop, and special cases that collapse to plain matmuls."""
import numpy as np
import pytest
import torch

from alpha_moe_python.prep import block_quant_fp8, moe_align_block_size, per_token_group_quant_fp8
from alpha_moe_python.utils import deinterleave_tensor, interleave_tensor
from alpha_moe_python.workloads import SHAPES, Shape, make_problem, make_weights
from oracle import c_oracle
from oracle import moe_oracle as O


# ---------------------------------------------------------------- fp8 codec
def test_fp8_decode_table_vs_torch():
    table = O.fp8_e4m3fn_decode_table()
    lib = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(table), np.isnan(lib))
    ok = ~np.isnan(table)
    assert np.array_equal(table[ok], lib[ok])
    assert table[0x7E] == 448.0 and table[0x01] == 2.0 ** -9 and table[0x08] == 2.0 ** -6
    L = c_oracle.lib()
    for code in range(256):
        v = L.moe_oracle_fp8_decode(code)
        assert (np.isnan(v) and np.isnan(table[code])) or v == table[code]


def test_fp8_encode_exhaustive_midpoints_vs_torch():
    table = O.fp8_e4m3fn_decode_table()
    pos = table[:0x7F].astype(np.float64)
    mids = (pos[1:] + pos[:-1]) / 2                       # exact in float32 (one extra mantissa bit)
    below = np.nextafter(mids.astype(np.float32), np.float32(0))
    above = np.nextafter(mids.astype(np.float32), np.float32(1e9))
    vals = np.concatenate([pos, mids, below, above, [448.0, 2.0 ** -10, 1.0625, 1.1875, 0.0]]).astype(np.float32)
    vals = np.concatenate([vals, -vals])
    vals = vals[np.abs(vals) <= 448.0]                    # torch's cast does not saturate; callers clamp first
    lib = torch.from_numpy(vals).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    own = O.fp8_e4m3fn_encode(vals)
    assert np.array_equal(own, lib)
    L = c_oracle.lib()
    c_codes = np.array([L.moe_oracle_fp8_encode(float(v)) for v in vals], dtype=np.uint8)
    assert np.array_equal(c_codes, lib)
    # ties to even, underflow, saturation
    enc = lambda v: float(table[O.fp8_e4m3fn_encode(np.float32(v))])
    assert enc(1.0625) == 1.0 and enc(1.1875) == 1.25 and enc(2.0 ** -10) == 0.0
    assert enc(1000.0) == 448.0 and enc(-1000.0) == -448.0
    assert L.moe_oracle_fp8_encode(1000.0) == 0x7E and L.moe_oracle_fp8_encode(-460.0) == 0xFE


def test_bf16_rounding_of_c_oracle_vs_torch():
    g = torch.Generator().manual_seed(0)
    v = torch.randn(4096, generator=g) * 10
    v[:4] = torch.tensor([1.00390625, 1.01171875, 0.0, -3.0])      # ties
    lib = v.bfloat16().view(torch.int16).numpy().astype(np.uint16)
    L = c_oracle.lib()
    own = np.array([L.moe_oracle_float_to_bf16(float(x)) for x in v], dtype=np.uint16)
    assert np.array_equal(own, lib)


# ---------------------------------------------------------------- fused path
def _small_problem(E=4, top_k=2, K=256, I=128, M=5, seed=0, scaling=1.7):
    shape = Shape("t", E=E, top_k=top_k, K=K, I=I, shared_expert=False, routing="softmax_renorm",
                  scaling_factor=scaling, w_std=0.05)
    W = make_weights(shape, seed=seed)
    return make_problem(W, M, seed=seed)


def _oracle_out(P, block_m, out=None, scaling=None):
    s_ids, e_ids, total = P.align(block_m)
    W = P.weights
    out = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16) if out is None else out
    scaling = P.shape.scaling_factor if scaling is None else scaling
    return O.fused_moe_oracle(P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total,
                              P.topk_weights, out, P.shape.top_k, block_m, scaling)


@pytest.mark.parametrize("I,block_m", [(128, 8), (256, 16)])
def test_python_and_c_restatements_agree(I, block_m):
    """moe_oracle.py de-interleaves then block-scales by position; moe_oracle.c indexes the interleaved
    tensors the way the reference kernel does.  A layout mistake in either breaks this."""
    P = _small_problem(E=3, K=256, I=I, M=6, seed=I)
    s_ids, e_ids, total = P.align(block_m)
    W = P.weights
    out0 = torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16)
    py = _oracle_out(P, block_m)
    c = c_oracle.fused_moe_c(P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total,
                             P.topk_weights, out0, P.shape.top_k, block_m, P.shape.scaling_factor)
    m = O.error_metrics(c, py)
    assert m["max_abs_over_max_ref"] <= 2 ** -7 and m["cosine"] >= 0.99999, m   # one bf16 ulp of the largest value
    assert float(py.float().abs().max()) > 1e-3


def test_routing_free_per_token_loop_agrees():
    P = _small_problem(E=5, top_k=3, K=256, I=256, M=7, seed=11)
    W = P.weights
    w1o = deinterleave_tensor(W.w1.view(torch.uint8), 8).view(torch.float8_e4m3fn)
    w1so = deinterleave_tensor(W.w1_scale, 1)
    dense = O.fused_moe_dense(P.x, P.x_scale, w1o, w1so, W.w2, W.w2_scale, P.topk_ids, P.topk_weights,
                              P.shape.scaling_factor)
    for block_m in (8, 16, 32):
        m = O.error_metrics(_oracle_out(P, block_m), dense)
        assert m["max_abs_over_max_ref"] <= 2 ** -7 and m["cosine"] >= 0.99999, (block_m, m)


def test_collapses_to_dense_swiglu_mlp():
    """E=1, top_k=1, unit scales, small-integer values: every product and sum is exact, so the result is
    torch.matmul -> SwiGLU -> requant -> torch.matmul with nothing left to interpretation."""
    g = torch.Generator().manual_seed(5)
    K, I, M = 128, 128, 4
    x = torch.randint(-2, 3, (M, K), generator=g).float()
    w1o = torch.randint(-1, 2, (1, 2 * I, K), generator=g).float()
    w2 = torch.randint(-2, 3, (1, K, I), generator=g).float()
    ones = lambda *s: torch.ones(s, dtype=torch.float32)
    ids = torch.zeros((M, 1), dtype=torch.int32)
    tw = ones(M, 1)
    s_ids, e_ids, total = moe_align_block_size(ids, 8, 1)
    got = O.fused_moe_oracle(x.to(torch.float8_e4m3fn), ones(M, 1), interleave_tensor(w1o.to(torch.float8_e4m3fn), 8),
                             interleave_tensor(ones(1, 2, 1), 1), w2.to(torch.float8_e4m3fn), ones(1, 1, 1),
                             s_ids, e_ids, total, tw, torch.zeros((M, K), dtype=torch.bfloat16), 1, 8, 1.0)
    h = (x @ w1o[0].t()).bfloat16().float()
    a = (torch.nn.functional.silu(h[:, :I]) * h[:, I:]).bfloat16().float()
    s = a.abs().amax(-1, keepdim=True).clamp_min(1e-10) / 448.0
    q = torch.from_numpy(O.fp8_e4m3fn_decode_table()[O.fp8_e4m3fn_encode((a / s).clamp(-448, 448).numpy())])
    want = ((q * s) @ w2[0].t()).bfloat16()
    m = O.error_metrics(got, want)
    assert m["max_abs_over_max_ref"] <= 2 ** -7, m


def test_linearity_zero_weights_and_add_semantics():
    P = _small_problem(E=4, K=256, I=128, M=6, seed=2)
    base = _oracle_out(P, 8, scaling=1.0).float()
    twice = _oracle_out(P, 8, scaling=2.0).float()
    assert torch.allclose(twice, 2 * base, atol=2 ** -6 * float(base.abs().max()))
    pre = torch.full((P.M, P.shape.K), 0.5, dtype=torch.bfloat16)
    shifted = _oracle_out(P, 8, out=pre, scaling=1.0).float()
    assert torch.allclose(shifted, base + 0.5, atol=2 ** -6 * float((base.abs() + 0.5).max()))
    saved = P.topk_weights
    P.topk_weights = torch.zeros_like(saved)
    assert float(_oracle_out(P, 8).float().abs().max()) == 0.0
    P.topk_weights = saved


def test_duplicate_expert_counts_twice_and_padding_is_inert():
    P = _small_problem(E=4, top_k=2, K=256, I=128, M=3, seed=9)
    P.topk_ids = torch.tensor([[1, 1], [2, 0], [3, 3]], dtype=torch.int32)
    P.topk_weights = torch.tensor([[0.25, 0.25], [0.5, 0.5], [0.3, 0.7]])
    P.aligned.clear()
    dup = _oracle_out(P, 8).float()
    P.topk_ids = torch.tensor([[1, 0], [2, 0], [3, 0]], dtype=torch.int32)
    P.topk_weights = torch.tensor([[0.5, 0.0], [0.5, 0.5], [1.0, 0.0]])
    P.aligned.clear()
    single = _oracle_out(P, 8).float()
    assert torch.allclose(dup[0], single[0], atol=2 ** -7 * float(single.abs().max()))
    assert torch.allclose(dup[2], single[2], atol=2 ** -7 * float(single.abs().max()))
    # a larger block only adds padding rows
    assert torch.equal(_oracle_out(P, 8), _oracle_out(P, 64))


def test_c1_config_runs_and_is_finite():
    W = make_weights(SHAPES["c1"], seed=0)
    P = make_problem(W, 16, seed=0)
    out = _oracle_out(P, 16)
    assert out.shape == (16, 512) and torch.isfinite(out.float()).all()
    assert 0.01 < float(out.float().abs().max()) < 100
    assert P.algorithmic_flops() == 3 * 16 * 2 * 512 * 256


def test_block_scales_land_on_the_right_blocks_exactly():
    """Power-of-two block scales, every 128x128 weight block and every token group its own, small-integer values: all
    products and sums stay exact, so the scale of block (row block, K block) is pinned against torch.matmul on weights
    dequantised explicitly in their ORIGINAL (not interleaved) layout.  A scale row read from the wrong place - gate
    instead of up, slice b instead of b+1, K block k instead of k+1 - changes the result by a power of two."""
    g = torch.Generator().manual_seed(7)
    E, K, I, M, top_k = 2, 384, 256, 5, 2
    N = 2 * I
    x = torch.randint(-2, 3, (M, K), generator=g).float()
    w1o = torch.randint(-1, 2, (E, N, K), generator=g).float()
    w2 = torch.randint(-2, 3, (E, K, I), generator=g).float()
    pow2 = lambda *shape: torch.pow(2.0, torch.randint(-3, 4, shape, generator=g).float())
    xs = pow2(M, K // 128)
    w1so = pow2(E, N // 128, K // 128)          # original layout: gate row blocks, then up row blocks
    w2s = pow2(E, K // 128, I // 128)
    assert len(set(w1so.flatten().tolist())) > 3 and len(set(w2s.flatten().tolist())) > 3
    ids = torch.stack([torch.randperm(E, generator=g)[:top_k] for _ in range(M)]).to(torch.int32)
    tw = pow2(M, top_k)
    block_m = 8
    s_ids, e_ids, total = moe_align_block_size(ids, block_m, E)
    got = O.fused_moe_oracle(x.to(torch.float8_e4m3fn), xs, interleave_tensor(w1o.to(torch.float8_e4m3fn), 8),
                             interleave_tensor(w1so, 1), w2.to(torch.float8_e4m3fn), w2s, s_ids, e_ids, total, tw,
                             torch.zeros((M, K), dtype=torch.bfloat16), top_k, block_m, 2.0)
    for accumulate in ("dense", "kblock"):
        alt = O.fused_moe_oracle(x.to(torch.float8_e4m3fn), xs, interleave_tensor(w1o.to(torch.float8_e4m3fn), 8),
                                 interleave_tensor(w1so, 1), w2.to(torch.float8_e4m3fn), w2s, s_ids, e_ids, total, tw,
                                 torch.zeros((M, K), dtype=torch.bfloat16), top_k, block_m, 2.0, accumulate=accumulate)
        assert torch.equal(alt, got), accumulate        # nothing rounds before the bf16 casts: any order, same bits
    # the textbook computation on explicitly dequantised weights, no routing arrays
    xd = x * xs.repeat_interleave(128, dim=1)
    want = torch.zeros((M, K))
    for t in range(M):
        for s in range(top_k):
            e = int(ids[t, s])
            w1d = w1o[e] * w1so[e].repeat_interleave(128, 0).repeat_interleave(128, 1)
            w2d = w2[e] * w2s[e].repeat_interleave(128, 0).repeat_interleave(128, 1)
            h = (xd[t] @ w1d.t()).bfloat16().float()
            a = (torch.nn.functional.silu(h[:I]) * h[I:]).bfloat16().float().reshape(I // 128, 128)
            sa = a.abs().amax(-1, keepdim=True).clamp_min(1e-10) / 448.0
            q = (a / sa).clamp(-448, 448).to(torch.float8_e4m3fn).float()
            want[t] += ((q * sa).reshape(I) @ w2d.t()) * float(tw[t, s]) * 2.0
    m = O.error_metrics(got, want.bfloat16())
    assert m["max_abs_over_max_ref"] <= 2 ** -8 and float(want.abs().max()) > 1.0, m
    # the C restatement, which reads the interleaved scale rows 2b / 2b+1 the way the reference kernel does
    c = c_oracle.fused_moe_c(x.to(torch.float8_e4m3fn), xs, interleave_tensor(w1o.to(torch.float8_e4m3fn), 8),
                             interleave_tensor(w1so, 1), w2.to(torch.float8_e4m3fn), w2s, s_ids, e_ids, total, tw,
                             torch.zeros((M, K), dtype=torch.bfloat16), top_k, block_m, 2.0)
    assert O.error_metrics(c, want.bfloat16())["max_abs_over_max_ref"] <= 2 ** -7


def test_accumulation_orders_and_nudged_sums_stay_close():
    """On ordinary data the K-block-wise accumulation order and sums moved by 1e-5 give the dense oracle's answer to
    within a bf16 ulp or two of the largest output: they are the same mathematics."""
    P = _small_problem(E=4, K=512, I=128, M=9, seed=21)
    s_ids, e_ids, total = P.align(8)
    W = P.weights
    run = lambda **kw: O.fused_moe_oracle(P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total,
                                          P.topk_weights, torch.zeros((P.M, P.shape.K), dtype=torch.bfloat16),
                                          P.shape.top_k, 8, P.shape.scaling_factor, **kw)
    base = run()
    for kw in ({"accumulate": "kblock"}, {"up_nudge": 1e-5}, {"up_nudge": -1e-5}):
        m = O.error_metrics(run(**kw), base)
        assert m["max_abs_over_max_ref"] <= 1e-2 and m["cosine"] >= 0.9999, (kw, m)
    assert torch.equal(run(up_nudge=0.0), base)
