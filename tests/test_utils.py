"""interleave_tensor / get_best_config against closed forms, brute force and the reference's shipped tables."""
import json
import os

import pytest
import torch

from alpha_moe_python.utils import deinterleave_tensor, get_best_config, interleave_tensor
from oracle import moe_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "ref_config_entries.json")


@pytest.mark.parametrize("rep", [1, 2, 8])
@pytest.mark.parametrize("shape", [(2, 32, 3), (1, 16, 5), (3, 256, 4)])
def test_interleave_matches_index_loop(shape, rep):
    t = torch.arange(shape[0] * shape[1] * shape[2], dtype=torch.float32).reshape(shape)
    got = interleave_tensor(t, rep)
    assert got.is_contiguous()
    assert torch.equal(got, O.interleave_reference(t, rep))
    assert torch.equal(deinterleave_tensor(got, rep), t)
    assert torch.equal(O.deinterleave_reference(got, rep), t)


def test_interleave_row_pattern_of_readme():
    # README.md:96-102 of the reference: g0..g7,u0..u7,g8..g15,u8..u15,...
    N = 32
    t = torch.arange(N).reshape(1, N, 1)
    got = interleave_tensor(t, 8).flatten().tolist()
    g, u = list(range(0, 16)), list(range(16, 32))
    assert got == g[0:8] + u[0:8] + g[8:16] + u[8:16]
    # scales, rep=1: gs0,us0,gs1,us1
    s = torch.arange(4).reshape(1, 4, 1)
    assert interleave_tensor(s, 1).flatten().tolist() == [0, 2, 1, 3]


def test_interleave_dtypes_and_errors():
    w = torch.randn(2, 32, 128).to(torch.float8_e4m3fn)
    got = interleave_tensor(w, 8)
    assert got.dtype == torch.float8_e4m3fn
    assert torch.equal(got.view(torch.uint8), O.interleave_reference(w.view(torch.uint8), 8))
    with pytest.raises(ValueError):
        interleave_tensor(torch.zeros(1, 24, 4), 8)
    with pytest.raises(ValueError):
        interleave_tensor(torch.zeros(24, 4), 8)


def test_get_best_config_nearest_and_ties(tmp_path):
    table = {"1": {"block_m": 16, "block_n": 32, "warp_n": 8, "stages": 5},
             "8": {"block_m": 8, "block_n": 32, "warp_n": 8, "stages": 4},
             "64": {"block_m": 8, "block_n": 64, "warp_n": 4, "stages": 2}}
    p = tmp_path / "t.json"
    p.write_text(json.dumps(table))
    path = str(p)
    assert get_best_config(path, 1) == table["1"]
    assert get_best_config(path, 4) == table["1"]       # |1-4|=3 < |8-4|=4
    assert get_best_config(path, 5) == table["8"]
    assert get_best_config(path, 36) == table["8"]      # tie 28/28: first key in file order wins
    assert get_best_config(path, 37) == table["64"]
    assert get_best_config(path, 10 ** 6) == table["64"]
    # memoised per (path, n_tokens): a rewritten file is not re-read for a cached query
    p.write_text(json.dumps({"1": {"block_m": 128, "block_n": 64, "warp_n": 4, "stages": 1}}))
    assert get_best_config(path, 1) == table["1"]
    assert get_best_config(path, 2)["block_m"] == 128


def test_get_best_config_on_reference_tables(tmp_path):
    golden = json.load(open(GOLDEN))
    ds = golden["moe_jit_257_256_7168.json"]
    assert ds["n_keys"] == 48
    p = tmp_path / "ds.json"
    p.write_text(json.dumps(ds["entries"]))
    assert get_best_config(str(p), 1) == {"block_m": 16, "block_n": 32, "warp_n": 8, "stages": 5}
    assert get_best_config(str(p), 8192) == {"block_m": 72, "block_n": 32, "warp_n": 8, "stages": 5}
    assert get_best_config(str(p), 60) == ds["entries"]["64"]
    assert get_best_config(str(p), 3000) == ds["entries"]["2048"]
    for cfg in ds["entries"].values():
        assert set(cfg) == {"block_m", "block_n", "warp_n", "stages"}
        assert cfg["block_n"] * cfg["warp_n"] == 256


def test_prepack_weights_is_the_stated_permutation_and_round_trips():
    """w_packed[e, kb, n, :] = w[e, n, 128 kb : 128 kb + 128] and w2_packed[e, ib, c, :] = w2[e, c, 128 ib : 128 ib + 128]
    (brute force over every index of a small case), any dtype, and unpack_weights is the inverse."""
    import torch
    from alpha_moe_python.utils import prepack_weights, unpack_weights
    E, N, K = 3, 512, 384
    w = torch.arange(E * N * K, dtype=torch.int32).reshape(E, N, K)
    w2 = torch.arange(E * K * (N // 2), dtype=torch.int32).reshape(E, K, N // 2) + 7
    wp, w2p = prepack_weights(w, w2)
    assert tuple(wp.shape) == (E, K // 128, N, 128) and tuple(w2p.shape) == (E, N // 256, K, 128)
    assert wp.is_contiguous() and w2p.is_contiguous()
    for e in range(E):
        for kb in range(K // 128):
            for n in (0, 1, 7, 8, 255, 256, N - 1):
                assert torch.equal(wp[e, kb, n], w[e, n, 128 * kb:128 * kb + 128])
        for ib in range(N // 256):
            for c in (0, 5, 127, 128, K - 1):
                assert torch.equal(w2p[e, ib, c], w2[e, c, 128 * ib:128 * ib + 128])
    back = unpack_weights(wp, w2p)
    assert torch.equal(back[0], w) and torch.equal(back[1], w2)
    q = torch.randn(2, 256, 128).to(torch.float8_e4m3fn)
    q2 = torch.randn(2, 128, 128).to(torch.float8_e4m3fn)
    a, b = prepack_weights(q, q2)
    assert a.dtype == torch.float8_e4m3fn and torch.equal(unpack_weights(a, b)[0].view(torch.uint8), q.view(torch.uint8))
    import pytest
    with pytest.raises(ValueError):
        prepack_weights(torch.zeros(2, 256, 100), torch.zeros(2, 100, 128))


def test_sglang_weight_loader_bookkeeping():
    import torch
    from alpha_moe_python.sglang_glue import W13Interleaver
    from alpha_moe_python.utils import interleave_tensor
    """Shards may arrive in any order, as w1 + w3 or as one fused w13; the slot is interleaved exactly once, when
    complete, and other shard ids are ignored."""
    E, I, K = 3, 16, 8
    ckpt = torch.arange(E * 2 * I * K, dtype=torch.float32).reshape(E, 2 * I, K)
    param = torch.zeros_like(ckpt)
    il = W13Interleaver(E, rep=8)
    order = [(0, "w3"), (1, "w1"), (0, "w2"), (0, "w1"), (2, "w13"), (1, "w3")]
    done = []
    for e, shard in order:
        if shard == "w1":
            param[e, :I] = ckpt[e, :I]
        elif shard == "w3":
            param[e, I:] = ckpt[e, I:]
        elif shard == "w13":
            param[e] = ckpt[e]
        done.append(il.shard_loaded(param[e], e, shard))
    assert done == [False, False, False, True, True, True]
    assert torch.equal(param, interleave_tensor(ckpt, 8))
