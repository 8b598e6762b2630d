"""CPU oracle for the fused W8A8 MoE path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; nothing under the shipped package does.  It restates, in fp32
torch/numpy on the CPU, what the reference's single GPU kernel computes
(csrc/kernels/fused_moe_w8a8/fused_moe_w8a8_up_down_acc.cu, below "K.cu").
The reference holds no torch-only implementation and no golden vectors for this
path; its own test oracle is SGLang's Triton pipeline
(test/test_moe_correctness.py:82-89), which is absent here.

How each function is pinned (tests/test_oracle.py, tests/test_prep.py):

* fp8 e4m3fn decode/encode  - own bit-field arithmetic vs torch.float8_e4m3fn
  exhaustively (256 codes, all midpoints: ties to even, saturation at 448).
* deinterleave / interleave - closed form of alpha_moe_python/utils.py:5-17,
  brute-force index loop, round trip, and the README.md:96-102 row pattern.
* align_reference           - python loop; invariants the kernel relies on
  (K.cu:676-679,756-758,857).  SGLang's moe_align_block_size itself: parity
  unpinned (third-party, absent; order inside an expert segment is defined
  here as ascending flat id).
* quant_group_reference     - closed form restated by K.cu:939-991; exactly
  representable inputs; round-trip error bound.  SGLang's
  sglang_per_token_group_quant_fp8 itself: parity unpinned (absent).
* fused_moe_oracle          - (1) moe_oracle.c, an independent scalar C
  restatement that walks the INTERLEAVED layout with K.cu's own indexing
  (scale rows 2bx / 2bx+1, K.cu:800-807,921-929) whereas this file
  de-interleaves first; (2) fused_moe_dense, a per-token loop over topk_ids
  that never looks at the routing arrays; (3) special cases that collapse to
  torch.matmul (unit scales, exactly representable values), zero routing
  weights, linearity in topk_weights / scaling_factor, add-into-out semantics
  (K.cu:1085-1091), invariance to block_m and to order inside a segment.

Deliberate departures from the reference kernel, all stricter:
the K-block partial sums are added in fp32, not bf16 (K.cu:740,919-931);
every token row's amax is floored at 1e-10, not only row 0 (K.cu:940).
"""
import numpy as np
import torch

FP8_MAX = 448.0
AMAX_FLOOR = 1e-10


# --------------------------------------------------------------------------
# FP8 e4m3fn (OCP): 1 sign, 4 exponent (bias 7), 3 mantissa; no inf; 0x7f/0xff = NaN
# --------------------------------------------------------------------------
def fp8_e4m3fn_decode_table() -> np.ndarray:
    """float32 value of each of the 256 codes, from the bit fields."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            val = float("nan")
        elif exp == 0:
            val = man * 2.0 ** -9          # subnormal: man/8 * 2^-6
        else:
            val = (1.0 + man / 8.0) * 2.0 ** (exp - 7)
        out[code] = sign * val
    return out


def fp8_e4m3fn_encode(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even, saturating to +-448, float32 -> code (uint8).  Inputs must be finite."""
    x = np.asarray(x, dtype=np.float32)
    table = fp8_e4m3fn_decode_table()
    pos = table[:0x7F].astype(np.float64)                # 0 .. 448, ascending
    mag = np.minimum(np.abs(x).astype(np.float64), FP8_MAX)
    hi = np.searchsorted(pos, mag, side="left").clip(0, len(pos) - 1)
    lo = np.maximum(hi - 1, 0)
    d_hi = pos[hi] - mag
    d_lo = mag - pos[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    return np.where(np.signbit(x), code | 0x80, code).astype(np.uint8)


def fp8_to_float(t: torch.Tensor) -> torch.Tensor:
    """fp8 (or its uint8 codes) -> float32 through the decode table above."""
    codes = t.view(torch.uint8).cpu().numpy()
    return torch.from_numpy(fp8_e4m3fn_decode_table()[codes])


# --------------------------------------------------------------------------
# layout (alpha_moe_python/utils.py:5-17)
# --------------------------------------------------------------------------
def interleave_reference(t: torch.Tensor, rep: int) -> torch.Tensor:
    """out[e, 2*rep*c + h*rep + j] = in[e, h*(N/2) + rep*c + j], by explicit row indices."""
    E, N, K = t.shape
    src = torch.empty(N, dtype=torch.long)
    for c in range(N // (2 * rep)):
        for h in range(2):
            for j in range(rep):
                src[2 * rep * c + h * rep + j] = h * (N // 2) + rep * c + j
    return t[:, src, :].contiguous()


def deinterleave_reference(t: torch.Tensor, rep: int) -> torch.Tensor:
    E, N, K = t.shape
    dst = torch.empty(N, dtype=torch.long)
    for c in range(N // (2 * rep)):
        for h in range(2):
            for j in range(rep):
                dst[h * (N // 2) + rep * c + j] = 2 * rep * c + h * rep + j
    return t[:, dst, :].contiguous()


# --------------------------------------------------------------------------
# routing arrays (contract consumed at K.cu:676-679,756-758,857)
# --------------------------------------------------------------------------
def align_reference(topk_ids, block_size: int, num_experts: int):
    """Brute-force moe_align_block_size: stable by flat id, pad value = numel, unused blocks = -1."""
    ids = [int(v) for v in torch.as_tensor(topk_ids).reshape(-1).tolist()]
    numel = len(ids)
    sorted_num = numel + num_experts * (block_size - 1)
    n_blocks = -(-sorted_num // block_size)
    sorted_ids = [numel] * sorted_num
    expert_ids = [-1] * n_blocks
    pos = 0
    for e in range(num_experts):
        members = [i for i, v in enumerate(ids) if v == e]
        if not members:
            continue
        for b in range(-(-len(members) // block_size)):
            expert_ids[pos // block_size + b] = e
        for k, i in enumerate(members):
            sorted_ids[pos + k] = i
        pos += -(-len(members) // block_size) * block_size
    return (torch.tensor(sorted_ids, dtype=torch.int32), torch.tensor(expert_ids, dtype=torch.int32),
            torch.tensor([pos], dtype=torch.int32))


# --------------------------------------------------------------------------
# quantisers (K.cu:939-991 restates the per-token-group rule)
# --------------------------------------------------------------------------
def quant_group_reference(x: torch.Tensor, group: int = 128):
    """Per-token-group FP8 quantisation with own encoder: returns (codes uint8 [M,K], scale f32 [M,K/group])."""
    M, K = x.shape
    xf = x.float().reshape(M, K // group, group)
    amax = xf.abs().amax(-1, keepdim=True).clamp_min(AMAX_FLOOR)
    scale = amax / FP8_MAX
    q = (xf / scale).clamp(-FP8_MAX, FP8_MAX)
    codes = torch.from_numpy(fp8_e4m3fn_encode(q.numpy())).reshape(M, K)
    return codes, scale.reshape(M, K // group)


def _expand_block_scale(scale: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    return scale.repeat_interleave(128, dim=-2).repeat_interleave(128, dim=-1)[..., :rows, :cols]


def _silu_mul(g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    return g / (1.0 + torch.exp(-g)) * u           # K.cu:76-79


def _up_sums_kblock(xq, xs, w1_e, w1s_e):
    """The up/gate sums accumulated the way a block-scaled kernel does (K.cu:900-933): per 128-wide K block the
    exact sum of the FP8 products, rounded to fp32; then h = fma(partial, x_scale * w_scale, h) in fp32, blocks in
    ascending order.  Same mathematics as one dense fp32 product of the dequantised operands, another rounding order:
    the two differ in the last bits of h, which matters wherever a value sits on a bf16 rounding boundary."""
    n, K = xq.shape
    N = w1_e.shape[0]
    w = w1_e.float().double()
    xq = xq.double()
    h = torch.zeros((n, N), dtype=torch.float32)
    row_block = torch.arange(N) // 128
    for kb in range(K // 128):
        part = (xq[:, kb * 128:(kb + 1) * 128] @ w[:, kb * 128:(kb + 1) * 128].t()).float()     # exact, then one rounding
        scale = xs[:, kb:kb + 1] * w1s_e[row_block, kb].unsqueeze(0)                             # fp32 product
        h = (part.double() * scale.double() + h.double()).float()                                # fused multiply-add
    return h


def _expert_forward(xd, w1_e, w1s_e, w2_e, w2s_e, up_sums=None, up_nudge=0.0):
    """fp32 maths of one expert on dequantised activations xd [n, K]; returns y [n, K] before routing weights.

    w1_e / w1s_e are in the ORIGINAL (de-interleaved) row order: gate rows then up rows.  up_sums: the up/gate sums
    [n, N] where the caller has accumulated them in another order (_up_sums_kblock).  up_nudge: relative perturbation
    of those sums before they are rounded to bf16 (see fused_moe_oracle).
    """
    N, K = w1_e.shape
    I = N // 2
    if up_sums is None:
        w1d = w1_e.float() * _expand_block_scale(w1s_e, N, K)
        up_sums = xd @ w1d.t()
    if up_nudge:
        up_sums = up_sums * (1.0 + up_nudge)
    h = up_sums.bfloat16().float()                               # K.cu:919-931 keeps h in bf16
    a = _silu_mul(h[:, :I], h[:, I:]).bfloat16().float()         # K.cu:945-946
    n = a.shape[0]
    ag = a.reshape(n, I // 128, 128)
    s_a = ag.abs().amax(-1, keepdim=True).clamp_min(AMAX_FLOOR) / FP8_MAX   # K.cu:963,978-979
    q = (ag / s_a).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn).float()  # K.cu:985-991
    ad = (q * s_a).reshape(n, I)
    w2d = w2_e.float() * _expand_block_scale(w2s_e, K, I)
    return ad @ w2d.t()                                          # K.cu:1036-1061


def fused_moe_oracle(x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids,
                     num_tokens_post_padded, topk_weights, out, top_k, block_m, scaling_factor, accumulate="dense",
                     up_nudge=0.0):
    """What torch.ops.alpha_moe.fused_moe_w8a8_up_down leaves in ``out``, computed in fp32 on the CPU.

    accumulate: "dense" sums the up/gate products as one fp32 matrix product of the dequantised operands (the
    definition every pin of this oracle uses); "kblock" sums them per 128-wide K block and folds the block scales in
    with fp32 multiply-adds, the order of a block-scaled kernel (_up_sums_kblock) - the same mathematics, used by the
    tests to tell a legitimate rounding-order difference from an error.

    up_nudge: multiplies every up/gate sum by (1 + up_nudge) before it is rounded to bf16.  The operator is
    discontinuous in those sums: a sum on a bf16 rounding boundary that is also the largest activation of its
    128-column group decides the group's FP8 scale, and with it the rounding of all 128 codes.  Sums of thousands of
    fp32 products accumulated in another order differ by ~1e-5 of their size where terms cancel; a result that agrees
    with the oracle for some |up_nudge| <= 1e-5 is a result of the same mathematics.

    Takes the operator's own arguments (interleaved w / w_scale, routing arrays) and returns a new
    bf16 tensor = out + contribution; ``out`` is not modified.  Walks the routing arrays exactly as the
    kernel does: block b belongs to expert_ids[b], rows are sorted_token_ids[b*block_m : (b+1)*block_m],
    token = id // top_k, rows with token >= M are padding (K.cu:676-679,756-758,857).
    """
    from_dev = lambda t: t.detach().cpu()
    x, x_scale, w, w_scale, w2, w2_scale = map(from_dev, (x, x_scale, w, w_scale, w2, w2_scale))
    sorted_token_ids, expert_ids, topk_weights = map(from_dev, (sorted_token_ids, expert_ids, topk_weights))
    M, K = x.shape
    total = int(from_dev(num_tokens_post_padded)[0])
    n_live_blocks = -(-total // block_m)
    acc = torch.zeros((M, K), dtype=torch.float32)
    xd_all = x.float() * x_scale.repeat_interleave(128, dim=1)
    tw_flat = topk_weights.reshape(-1)

    blocks_of = {}
    for b in range(n_live_blocks):
        blocks_of.setdefault(int(expert_ids[b]), []).append(b)
    for e, blocks in blocks_of.items():
        if e < 0:
            continue
        ids = torch.cat([sorted_token_ids[b * block_m:(b + 1) * block_m] for b in blocks]).long()
        ids = ids[(ids // top_k) < M]
        if ids.numel() == 0:
            continue
        tok = ids // top_k
        w1_e = deinterleave_reference(w[e:e + 1].view(torch.uint8), 8)[0].view(torch.float8_e4m3fn)
        w1s_e = deinterleave_reference(w_scale[e:e + 1], 1)[0]
        up_sums = _up_sums_kblock(fp8_to_float(x[tok]), x_scale[tok], w1_e, w1s_e) if accumulate == "kblock" else None
        y = _expert_forward(xd_all[tok], w1_e, w1s_e, w2[e], w2_scale[e], up_sums, up_nudge)
        y = y * (tw_flat[ids] * float(scaling_factor)).unsqueeze(1)            # K.cu:997-1003
        acc.index_add_(0, tok, y)
    return (from_dev(out).float() + acc).bfloat16()


def fused_moe_dense(x, x_scale, w1_orig, w1_scale_orig, w2, w2_scale, topk_ids, topk_weights, scaling_factor):
    """Per-token loop over topk_ids on NON-interleaved weights; never touches the routing arrays."""
    M, K = x.shape
    xd_all = x.float() * x_scale.repeat_interleave(128, dim=1)
    acc = torch.zeros((M, K), dtype=torch.float32)
    for t in range(M):
        for s in range(topk_ids.shape[1]):
            e = int(topk_ids[t, s])
            y = _expert_forward(xd_all[t:t + 1], w1_orig[e], w1_scale_orig[e], w2[e], w2_scale[e])
            acc[t] += y[0] * float(topk_weights[t, s]) * float(scaling_factor)
    return acc.bfloat16()


def error_metrics(out: torch.Tensor, ref: torch.Tensor) -> dict:
    """Parity figures: max |err| over max |ref|, worst allclose-style relative error, cosine."""
    o, r = out.detach().float().cpu().flatten().double(), ref.detach().float().cpu().flatten().double()
    err = (o - r).abs()
    denom = r.abs().max().clamp_min(1e-30)
    cos = float((o @ r) / (o.norm() * r.norm()).clamp_min(1e-30))
    return {
        "max_abs": float(err.max()),
        "max_abs_over_max_ref": float(err.max() / denom),
        "cosine": cos,
        "allclose_2e-2_1e-1": bool(torch.allclose(o, r, atol=2e-2, rtol=1e-1)),
    }
