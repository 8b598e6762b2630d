"""The autotuner (alpha-moe_amd/jit_moe.py; the reference's jit_moe.py:104-183): sweep space, table writer and `--update`
merge on the CPU, and a two-candidate sweep on the GPU whose table `get_best_config` reads back."""
import json
import os

import pytest

import jit_moe
from alpha_moe_python.utils import get_best_config

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "ref_config_entries.json")


def test_candidate_list_is_the_reference_sweep_space():
    # jit_moe.py:151-157 of the reference: block_m 8..128 step 8 x {(64,4), (32,8)} x stages 1..5 = 160 combinations
    full = jit_moe.candidate_list(list(range(8, 129, 8)), [1, 2, 3, 4, 5])
    assert len(full) == 160 and len(set(full)) == 160
    assert {bm for bm, _, _, _ in full} == set(range(8, 129, 8))
    assert {(bn, wn) for _, bn, wn, _ in full} == {(64, 4), (32, 8)}
    assert {st for _, _, _, st in full} == {1, 2, 3, 4, 5}
    # every candidate is one the operator accepts
    import ctypes
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ctypes.CDLL(os.path.join(root, "alpha-moe_amd", "alpha_moe", "libalpha_moe_hip.so"))
    lib.alpha_moe_validate.argtypes = [ctypes.c_int] * 10
    for bm, bn, wn, st in full:
        assert lib.alpha_moe_validate(9, 64, 7168, 512, 257, 4431, bm, bn, wn, st) == 0
    # bounded sweeps keep the order block_m-major
    assert jit_moe.candidate_list([16, 128], [2]) == [(16, 64, 4, 2), (16, 32, 8, 2), (128, 64, 4, 2), (128, 32, 8, 2)]


def test_argument_defaults_follow_the_reference():
    # jit_moe.py:54-98 of the reference
    a = jit_moe.parse_arguments([])
    assert a.batch_sizes == [8, 32, 128, 256, 512, 1024, 2048, 4096, 8192]
    assert a.balancedness == [0.8, 0.7, 0.6, 0.5]
    assert (a.N, a.K, a.E, a.top_k, a.shared_expert, a.out_config) == (256, 7168, 256, 8, True, None)
    assert jit_moe.parse_arguments(["--no-shared-expert"]).shared_expert is False


def test_pick_best_and_table_format_match_the_shipped_tables(tmp_path):
    times = {8: {(16, 64, 4, 2): [10.0, 12.0], (8, 32, 8, 5): [9.0, 9.5], (64, 64, 4, 3): []},
             4096: {(128, 32, 8, 2): [700.0], (128, 64, 4, 3): [710.0]}}
    table = jit_moe.pick_best(times)
    assert table == {8: {"block_m": 8, "block_n": 32, "warp_n": 8, "stages": 5},
                     4096: {"block_m": 128, "block_n": 32, "warp_n": 8, "stages": 2}}
    path = str(tmp_path / "moe_jit_test.json")
    jit_moe.write_table(path, table)
    on_disk = json.load(open(path))
    golden = json.load(open(GOLDEN))["moe_jit_257_256_7168.json"]["entries"]
    # same form as the tables the reference ships: decimal string keys, exactly these four integer fields
    assert list(on_disk) == ["8", "4096"]
    for entry in on_disk.values():
        assert set(entry) == set(next(iter(golden.values()))) == {"block_m", "block_n", "warp_n", "stages"}
        assert all(isinstance(v, int) for v in entry.values())
    assert get_best_config(path, 8) == table[8] and get_best_config(path, 3000) == table[4096]


def test_update_merges_into_an_existing_table(tmp_path):
    path = str(tmp_path / "t.json")
    old = {1: {"block_m": 16, "block_n": 32, "warp_n": 8, "stages": 5}, 64: {"block_m": 16, "block_n": 64, "warp_n": 4, "stages": 4}}
    jit_moe.write_table(path, old)
    new = {64: {"block_m": 8, "block_n": 32, "warp_n": 8, "stages": 3}, 16: {"block_m": 8, "block_n": 64, "warp_n": 4, "stages": 4}}
    merged = jit_moe.write_table(path, new, update=True)
    assert list(merged) == [1, 16, 64] and merged[1] == old[1] and merged[64] == new[64]
    assert list(json.load(open(path))) == ["1", "16", "64"]
    # without --update the file is replaced
    jit_moe.write_table(path, new)
    assert list(json.load(open(path))) == ["64", "16"]


def test_routing_generator_honours_balancedness():
    import torch
    torch.manual_seed(0)
    ids = jit_moe.generate_topk_ids(64, 4000, 8, balancedness=0.5)
    assert ids.shape == (4000, 8) and int(ids.min()) >= 0 and int(ids.max()) < 64
    share0 = float((ids == 0).float().mean())
    assert 0.45 < share0 < 0.56          # half of the slots forced to expert 0 plus its uniform share
    uniform = jit_moe.generate_topk_ids(64, 4000, 8, balancedness=1.0)
    assert float((uniform == 0).float().mean()) < 0.03


@pytest.mark.gpu
def test_two_candidate_sweep_writes_a_table_the_lookup_reads(tmp_path):
    path = str(tmp_path / "moe_jit_smoke.json")
    rc = jit_moe.main(["--E", "8", "--N", "256", "--K", "512", "--top-k", "2", "--no-shared-expert",
                       "--batch-sizes", "16", "200", "--balancedness", "0.8", "--block-ms", "16", "64",
                       "--stages", "2", "3", "--num-tests", "2", "--out-config", path])
    assert rc == 0
    table = json.load(open(path))
    assert list(table) == ["16", "200"]
    for key, entry in table.items():
        assert set(entry) == {"block_m", "block_n", "warp_n", "stages"}
        assert entry["block_m"] in (16, 64) and entry["stages"] in (2, 3)
        assert (entry["block_n"], entry["warp_n"]) in ((64, 4), (32, 8))
        assert get_best_config(path, int(key)) == entry
    # --update keeps what the file holds for sizes this run does not time
    rc = jit_moe.main(["--E", "8", "--N", "256", "--K", "512", "--top-k", "2", "--no-shared-expert",
                       "--batch-sizes", "64", "--balancedness", "0.8", "--block-ms", "16", "--stages", "2",
                       "--num-tests", "2", "--out-config", path, "--update"])
    assert rc == 0 and list(json.load(open(path))) == ["16", "64", "200"]
