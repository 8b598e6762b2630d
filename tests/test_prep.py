"""Input preparation (quantisers, moe_align_block_size) against brute force and invariants."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from alpha_moe_python.prep import block_quant_fp8, moe_align_block_size, per_token_group_quant_fp8
from oracle import moe_oracle as O


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 40), st.integers(1, 6), st.integers(1, 12), st.sampled_from([1, 4, 8, 16, 24]), st.integers(0, 10 ** 6))
def test_align_matches_brute_force(M, top_k, E, block, seed):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, E, (M, top_k), generator=g, dtype=torch.int32)   # duplicates within a token allowed
    got = moe_align_block_size(ids, block, E)
    ref = O.align_reference(ids, block, E)
    for a, b in zip(got, ref):
        assert a.dtype == torch.int32
        assert torch.equal(a, b)


def test_align_invariants():
    g = torch.Generator().manual_seed(3)
    M, top_k, E, block = 64, 9, 257, 16
    ids = torch.randint(0, E, (M, top_k), generator=g, dtype=torch.int32)
    sorted_ids, expert_ids, total = moe_align_block_size(ids, block, E)
    numel = M * top_k
    assert sorted_ids.numel() == numel + E * (block - 1)
    assert expert_ids.numel() == -(-sorted_ids.numel() // block)
    counts = torch.bincount(ids.flatten().long(), minlength=E)
    assert int(total) == int(((counts + block - 1) // block * block).sum())
    live = sorted_ids[sorted_ids < numel]
    assert sorted(live.tolist()) == list(range(numel))            # every slot exactly once
    assert (sorted_ids[int(total):] == numel).all()
    flat = ids.flatten()
    prev_e = -1
    for b in range(int(total) // block):
        e = int(expert_ids[b])
        assert e >= prev_e                                        # ascending experts
        prev_e = e
        seg = sorted_ids[b * block:(b + 1) * block]
        real = seg[seg < numel]
        assert (flat[real.long()] == e).all()
        assert (real[1:] > real[:-1]).all()                       # stable inside a block
    assert (expert_ids[int(total) // block:] == -1).all()


def test_align_empty_experts_and_single_token():
    ids = torch.tensor([[5, 5]], dtype=torch.int32)               # duplicate expert in one token
    s, e, t = moe_align_block_size(ids, 8, 7)
    assert int(t) == 8 and e[0] == 5 and (e[1:] == -1).all()
    assert s[:2].tolist() == [0, 1] and (s[2:] == 2).all()


def test_group_quant_matches_own_encoder_and_bound():
    g = torch.Generator().manual_seed(0)
    x = (torch.randn((17, 384), generator=g) * 3).to(torch.bfloat16)
    q, s = per_token_group_quant_fp8(x)
    codes, s_ref = O.quant_group_reference(x)
    assert torch.equal(s, s_ref)
    assert torch.equal(q.view(torch.uint8), codes)
    assert torch.equal(s, x.float().reshape(17, 3, 128).abs().amax(-1) / 448.0)
    deq = O.fp8_to_float(q).reshape(17, 3, 128) * s.unsqueeze(-1)
    err = (deq - x.float().reshape(17, 3, 128)).abs()
    # half an ulp of a 3-bit mantissa relative to the value, plus half a subnormal step (2^-10) in scaled units
    assert (err <= deq.abs() * 2.0 ** -4 + s.unsqueeze(-1) * 2.0 ** -10 + 1e-12).all()


def test_group_quant_exact_and_zero_rows():
    x = torch.zeros((2, 128))
    x[0, :5] = torch.tensor([448.0, -224.0, 1.0, 0.5, -0.015625])
    q, s = per_token_group_quant_fp8(x)
    assert float(s[0, 0]) == 1.0
    assert torch.equal(O.fp8_to_float(q)[0, :5], x[0, :5])      # exactly representable values survive
    assert float(s[1, 0]) == pytest.approx(1e-10 / 448.0)
    assert (q.view(torch.uint8)[1] == 0).all()


def test_block_quant():
    g = torch.Generator().manual_seed(1)
    w = torch.randn((3, 256, 384), generator=g) * 0.02
    q, s = block_quant_fp8(w)
    assert q.shape == w.shape and s.shape == (3, 2, 3)
    for e in range(3):
        for i in range(2):
            for j in range(3):
                blk = w[e, 128 * i:128 * i + 128, 128 * j:128 * j + 128]
                assert float(s[e, i, j]) == pytest.approx(float(blk.abs().max()) / 448.0, rel=1e-6)
                ref = torch.from_numpy(O.fp8_e4m3fn_encode((blk / s[e, i, j]).clamp(-448, 448).numpy()))
                assert torch.equal(q[e, 128 * i:128 * i + 128, 128 * j:128 * j + 128].view(torch.uint8), ref)
    assert int((O.fp8_to_float(q).abs() == 448.0).sum()) >= 3 * 2 * 3   # each block's amax maps to +-448
