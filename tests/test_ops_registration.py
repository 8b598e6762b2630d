"""`import alpha_moe` registers the operator with the reference's schema; the fake implementation lets it trace."""
import torch

import alpha_moe  # noqa: F401
import alpha_moe_ops


def test_schema_matches_the_reference():
    # csrc/torch_interface.cpp:105-125 of the reference
    schema = str(torch.ops.alpha_moe.fused_moe_w8a8_up_down.default._schema)
    want = ("alpha_moe::fused_moe_w8a8_up_down(Tensor x, Tensor x_scale, Tensor w, Tensor w_scale, Tensor w2, "
            "Tensor w2_scale, Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, "
            "Tensor topk_weights, Tensor(a!) out, int top_k, int block_m, int block_n, int warp_n, int stages, "
            "float scaling_factor) -> ()")
    assert schema == want


def test_fake_impl_runs_on_meta_tensors():
    M, K, N, E, top_k = 4, 256, 256, 3, 2
    meta = lambda shape, dt: torch.empty(shape, dtype=dt, device="meta")
    out = meta((M, K), torch.bfloat16)
    res = alpha_moe_ops.fused_moe_w8a8_up_down(
        meta((M, K), torch.float8_e4m3fn), meta((M, K // 128), torch.float32), meta((E, N, K), torch.float8_e4m3fn),
        meta((E, N // 128, K // 128), torch.float32), meta((E, K, N // 2), torch.float8_e4m3fn),
        meta((E, K // 128, N // 256), torch.float32), meta((M * top_k + E * 15,), torch.int32), meta((10,), torch.int32),
        meta((1,), torch.int32), meta((M, top_k), torch.float32), out, top_k, 16, 64, 4, 3, 1.0)
    assert res is out


def test_cpu_tensors_are_refused():
    import pytest
    M, K, N, E, top_k = 4, 256, 256, 3, 2
    with pytest.raises((RuntimeError, NotImplementedError)):
        torch.ops.alpha_moe.fused_moe_w8a8_up_down(
            torch.zeros((M, K)).to(torch.float8_e4m3fn), torch.ones((M, K // 128)), torch.zeros((E, N, K)).to(torch.float8_e4m3fn),
            torch.ones((E, N // 128, K // 128)), torch.zeros((E, K, N // 2)).to(torch.float8_e4m3fn),
            torch.ones((E, K // 128, N // 256)), torch.zeros(M * top_k + E * 15, dtype=torch.int32),
            torch.zeros(10, dtype=torch.int32), torch.zeros(1, dtype=torch.int32), torch.ones((M, top_k)),
            torch.zeros((M, K), dtype=torch.bfloat16), top_k, 16, 64, 4, 3, 1.0)


def test_store_variant_has_the_same_schema_and_a_fake_impl():
    a = str(torch.ops.alpha_moe.fused_moe_w8a8_up_down.default._schema)
    b = str(torch.ops.alpha_moe.fused_moe_w8a8_up_down_store.default._schema)
    assert b == a.replace("fused_moe_w8a8_up_down(", "fused_moe_w8a8_up_down_store(")
    M, K, N, E, top_k = 4, 256, 256, 3, 2
    meta = lambda shape, dt: torch.empty(shape, dtype=dt, device="meta")
    out = meta((M, K), torch.bfloat16)
    res = alpha_moe_ops.fused_moe_w8a8_up_down_store(
        meta((M, K), torch.float8_e4m3fn), meta((M, K // 128), torch.float32), meta((E, N, K), torch.float8_e4m3fn),
        meta((E, N // 128, K // 128), torch.float32), meta((E, K, N // 2), torch.float8_e4m3fn),
        meta((E, K // 128, N // 256), torch.float32), meta((M * top_k + E * 15,), torch.int32), meta((10,), torch.int32),
        meta((1,), torch.int32), meta((M, top_k), torch.float32), out, top_k, 16, 64, 4, 3, 1.0)
    assert res is out
