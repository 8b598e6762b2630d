"""ctypes loader for oracle/libmoe_oracle.so (the scalar C restatement).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return os.path.join(_HERE, "libmoe_oracle.so")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libmoe_oracle.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.moe_oracle_fp8_encode.restype = ctypes.c_uint8
        L.moe_oracle_fp8_encode.argtypes = [ctypes.c_float]
        L.moe_oracle_fp8_decode.restype = ctypes.c_float
        L.moe_oracle_fp8_decode.argtypes = [ctypes.c_uint8]
        L.moe_oracle_float_to_bf16.restype = ctypes.c_uint16
        L.moe_oracle_float_to_bf16.argtypes = [ctypes.c_float]
        L.moe_oracle_fused.restype = ctypes.c_int
        L.moe_oracle_fused.argtypes = [ctypes.c_void_p] * 11 + [ctypes.c_int] * 7 + [ctypes.c_float]
        _LIB = L
    return _LIB


def fused_moe_c(x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                topk_weights, out, top_k, block_m, scaling_factor):
    """Same arguments as the operator; returns a new bf16 tensor (``out`` is left alone)."""
    c = lambda t: t.detach().cpu().contiguous()
    x, x_scale, w, w_scale, w2, w2_scale = map(c, (x, x_scale, w, w_scale, w2, w2_scale))
    sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights = map(
        c, (sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights))
    res = c(out).clone()
    M, K = x.shape
    rc = lib().moe_oracle_fused(
        x.data_ptr(), x_scale.data_ptr(), w.data_ptr(), w_scale.data_ptr(), w2.data_ptr(), w2_scale.data_ptr(),
        res.data_ptr(), sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(),
        topk_weights.data_ptr(), int(top_k), M, K, w.shape[1], w.shape[0], sorted_token_ids.shape[0], int(block_m),
        float(scaling_factor))
    if rc != 0:
        raise RuntimeError(f"moe_oracle_fused returned {rc}")
    return res
