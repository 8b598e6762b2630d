"""``import alpha_moe`` registers ``torch.ops.alpha_moe.fused_moe_w8a8_up_down`` (as the reference's extension
module of the same name does, csrc/torch_interface.cpp:105-131) by loading the in-tree HIP libraries, together with
the two input-preparation operators ``per_token_group_quant_fp8`` and ``moe_align_block_size``.

There is no fallback: if the libraries are not built the import fails.
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the libraries below bind to)

_HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIBRARY = os.path.join(_HERE, "libalpha_moe_hip.so")
TORCH_LIBRARY = os.path.join(_HERE, "alpha_moe_torch.so")

for _p in (HIP_LIBRARY, TORCH_LIBRARY):
    if not os.path.exists(_p):
        raise ImportError(f"{_p} is missing: build it with `python alpha-moe_amd/build.py` (needs hipcc, gfx950)")

# the C ABI first (the binding links against it), then the binding, whose static initialiser registers the op
c_abi = ctypes.CDLL(HIP_LIBRARY, mode=ctypes.RTLD_GLOBAL)
torch.ops.load_library(TORCH_LIBRARY)

c_abi.alpha_moe_status_string.restype = ctypes.c_char_p
c_abi.alpha_moe_status_string.argtypes = [ctypes.c_int]
c_abi.alpha_moe_version.restype = ctypes.c_char_p
c_abi.alpha_moe_validate.restype = ctypes.c_int
c_abi.alpha_moe_validate.argtypes = [ctypes.c_int] * 10
c_abi.alpha_moe_fused_moe_w8a8_up_down.restype = ctypes.c_int
c_abi.alpha_moe_fused_moe_w8a8_up_down.argtypes = (
    [ctypes.c_void_p] * 11 + [ctypes.c_int] * 10 + [ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])
c_abi.alpha_moe_fused_moe_w8a8_up_down_store.restype = ctypes.c_int
c_abi.alpha_moe_fused_moe_w8a8_up_down_store.argtypes = c_abi.alpha_moe_fused_moe_w8a8_up_down.argtypes
c_abi.alpha_moe_fused_moe_w8a8_up_down_static.restype = ctypes.c_int
c_abi.alpha_moe_fused_moe_w8a8_up_down_static.argtypes = (
    [ctypes.c_void_p] * 11 + [ctypes.c_int] * 10 + [ctypes.c_float, ctypes.c_void_p])
c_abi.alpha_moe_fused_moe_w8a8_up_down_prepacked.restype = ctypes.c_int
c_abi.alpha_moe_fused_moe_w8a8_up_down_prepacked.argtypes = (
    [ctypes.c_void_p] * 11 + [ctypes.c_int] * 10 + [ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                                                   ctypes.c_void_p])
c_abi.alpha_moe_static_scratch_check.restype = ctypes.c_int
c_abi.alpha_moe_static_scratch_check.argtypes = [ctypes.c_void_p]
c_abi.alpha_moe_static_scratch_reset.restype = ctypes.c_int
c_abi.alpha_moe_static_scratch_reset.argtypes = [ctypes.c_void_p]
c_abi.alpha_moe_set_tunable.restype = ctypes.c_int
c_abi.alpha_moe_set_tunable.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_int]
c_abi.alpha_moe_workspace_check.restype = ctypes.c_int
c_abi.alpha_moe_workspace_check.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
c_abi.alpha_moe_workspace_zero_bytes.restype = ctypes.c_size_t
c_abi.alpha_moe_workspace_zero_bytes.argtypes = []
c_abi.alpha_moe_workspace_bytes.restype = ctypes.c_size_t
c_abi.alpha_moe_workspace_bytes.argtypes = [ctypes.c_int] * 7

c_abi.alpha_moe_per_token_group_quant_fp8.restype = ctypes.c_int
c_abi.alpha_moe_per_token_group_quant_fp8.argtypes = (
    [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])
c_abi.alpha_moe_align_workspace_bytes.restype = ctypes.c_size_t
c_abi.alpha_moe_align_workspace_bytes.argtypes = [ctypes.c_int] * 2
c_abi.alpha_moe_moe_align_block_size.restype = ctypes.c_int
c_abi.alpha_moe_moe_align_block_size.argtypes = (
    [ctypes.c_void_p] + [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                                              ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])

__version__ = c_abi.alpha_moe_version().decode()


def set_tunable(name: str, value=None) -> None:
    """Install (``value`` an int) or clear (``None``) one of the library's tuning overrides (experiments and tests)."""
    rc = c_abi.alpha_moe_set_tunable(name.encode(), 0 if value is None else int(value), 0 if value is None else 1)
    if rc != 0:
        raise ValueError(f"unknown tunable {name!r}")
