"""GPU input preparation (per-token-group FP8 quantisation, expert alignment) against the CPU oracle: bit-exact."""
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("M,K,dtype", [(1, 128, torch.bfloat16), (7, 512, torch.bfloat16), (64, 7168, torch.bfloat16),
                                       (33, 2048, torch.float32), (4096, 2048, torch.bfloat16)])
def test_quant_matches_oracle_bit_for_bit(M, K, dtype):
    from alpha_moe_python import prep, prep_hip
    g = torch.Generator().manual_seed(M * 31 + K)
    x = (torch.randn((M, K), generator=g) * torch.rand((M, 1), generator=g) * 4).to(dtype)
    x[0, :128] = 0                      # an all-zero group: scale = 1e-10 / 448, q = 0
    if M > 1:
        x[1, 5] = 3.0e4                 # a large outlier
    print(f"case quant M={M} K={K} {dtype}", flush=True)
    q, s = prep_hip.per_token_group_quant_fp8(x.to(DEV))
    torch.cuda.synchronize()
    q_ref, s_ref = O.quant_group_reference(x)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))
    # and the torch restatement the package ships agrees as well
    q_t, s_t = prep.per_token_group_quant_fp8(x)
    assert torch.equal(q_t.view(torch.uint8), q_ref.view(torch.uint8)) and torch.equal(s_t, s_ref)


@pytest.mark.parametrize("M,top_k,E,block", [(1, 9, 257, 16), (4, 2, 8, 8), (64, 9, 257, 16), (300, 8, 128, 64),
                                              (455, 9, 257, 128), (456, 9, 257, 16), (8192, 9, 257, 128),
                                              (4096, 10, 512, 24)])
def test_align_matches_oracle_bit_for_bit(M, top_k, E, block):
    from alpha_moe_python import prep_hip
    g = torch.Generator().manual_seed(M + 7 * E)
    # skewed routing: some experts empty, some hot
    probs = torch.rand(E, generator=g) ** 4
    ids = torch.multinomial(probs.expand(M, E), top_k, replacement=False, generator=g).to(torch.int32)
    print(f"case align M={M} top_k={top_k} E={E} block={block}", flush=True)
    s_ids, e_ids, total = prep_hip.moe_align_block_size(ids.to(DEV), block, E)
    torch.cuda.synchronize()
    r_ids, r_e, r_total = O.align_reference(ids, block, E)
    assert torch.equal(total.cpu(), r_total)
    assert torch.equal(e_ids.cpu(), r_e)
    assert torch.equal(s_ids.cpu(), r_ids)


def test_align_drops_slots_with_an_expert_out_of_range():
    from alpha_moe_python import prep_hip
    ids = torch.tensor([[0, 3], [7, -1], [9, 3]], dtype=torch.int32)
    s_ids, e_ids, total = prep_hip.moe_align_block_size(ids.to(DEV), 4, 8)
    torch.cuda.synchronize()
    assert total.item() == 12
    assert s_ids.cpu()[:12].tolist() == [0, 6, 6, 6, 1, 5, 6, 6, 2, 6, 6, 6]
    assert e_ids.cpu()[:3].tolist() == [0, 3, 7] and (e_ids.cpu()[3:] == -1).all()


def test_prepared_inputs_drive_the_fused_operator():
    """quantise + align on the GPU, then the fused call: same result as with the torch-prepared inputs."""
    from alpha_moe_python import prep, prep_hip
    from alpha_moe_python.workloads import SHAPES, make_weights
    import alpha_moe  # noqa: F401
    shape = SHAPES["c1"]
    W = make_weights(shape, device=DEV, seed=0)
    g = torch.Generator().manual_seed(5)
    M = 40
    x = torch.randn((M, shape.K), generator=g).to(torch.bfloat16).to(DEV)
    ids = torch.multinomial(torch.ones(M, shape.E), shape.top_k, generator=g).to(torch.int32).to(DEV)
    tw = torch.rand((M, shape.top_k), generator=g).to(DEV)
    outs = []
    for mod in (prep_hip, prep):
        if mod is prep_hip:
            xq, xs = mod.per_token_group_quant_fp8(x)
            s_ids, e_ids, total = mod.moe_align_block_size(ids, 16, shape.E)
        else:   # the torch restatement on the CPU (IEEE division), then copied over
            xq, xs = (t.to(DEV) for t in mod.per_token_group_quant_fp8(x.cpu()))
            s_ids, e_ids, total = (t.to(DEV) for t in mod.moe_align_block_size(ids.cpu(), 16, shape.E))
        out = torch.zeros((M, shape.K), dtype=torch.bfloat16, device=DEV)
        torch.ops.alpha_moe.fused_moe_w8a8_up_down(xq, xs, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total, tw,
                                                   out, shape.top_k, 16, 64, 4, 3, 1.0)
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
