"""The C ABI library loads without a GPU, exports every function include/alpha_moe_hip.h declares, and its host-only
entry points (argument validation, workspace sizing, status strings) behave as documented."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "alpha_moe_hip.h")
LIB = os.path.join(ROOT, "alpha-moe_amd", "alpha_moe", "libalpha_moe_hip.so")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} is not built: run `python alpha-moe_amd/build.py`")
    L = ctypes.CDLL(LIB)
    L.alpha_moe_validate.restype = ctypes.c_int
    L.alpha_moe_validate.argtypes = [ctypes.c_int] * 10
    L.alpha_moe_workspace_bytes.restype = ctypes.c_size_t
    L.alpha_moe_workspace_bytes.argtypes = [ctypes.c_int] * 7
    L.alpha_moe_status_string.restype = ctypes.c_char_p
    L.alpha_moe_status_string.argtypes = [ctypes.c_int]
    L.alpha_moe_version.restype = ctypes.c_char_p
    L.alpha_moe_fused_moe_w8a8_up_down.restype = ctypes.c_int
    L.alpha_moe_fused_moe_w8a8_up_down.argtypes = (
        [ctypes.c_void_p] * 11 + [ctypes.c_int] * 10 + [ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])
    return L


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(alpha_moe_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = declared_functions()
    assert "alpha_moe_fused_moe_w8a8_up_down" in names and len(names) >= 5
    for name in names:
        assert getattr(lib, name) is not None, name


def test_status_codes_match_header(lib):
    text = open(HEADER).read()
    codes = dict((k, int(v)) for k, v in re.findall(r"(ALPHA_MOE_\w+)\s*=\s*(\d+)", text))
    assert codes["ALPHA_MOE_OK"] == 0 and len(set(codes.values())) == len(codes)
    for name, code in codes.items():
        msg = lib.alpha_moe_status_string(code).decode()
        assert msg and msg != "unknown status", name
    assert lib.alpha_moe_status_string(999).decode() == "unknown status"
    assert re.fullmatch(r"\d+\.\d+", lib.alpha_moe_version().decode())


def test_validate_accepts_the_reference_knob_space_and_rejects_the_rest(lib):
    ok = dict(top_k=9, M=64, K=7168, N=512, E=257, sorted_num=4431, block_m=16, block_n=64, warp_n=4, stages=3)

    def v(**kw):
        a = dict(ok, **kw)
        return lib.alpha_moe_validate(a["top_k"], a["M"], a["K"], a["N"], a["E"], a["sorted_num"], a["block_m"],
                                      a["block_n"], a["warp_n"], a["stages"])
    # csrc/torch_interface.cpp:62-64 of the reference: block_m 8..128 step 8, (64,4)|(32,8), stages 1..5
    for bm in range(8, 129, 8):
        for bn, wn in ((64, 4), (32, 8)):
            for st in range(1, 6):
                assert v(block_m=bm, block_n=bn, warp_n=wn, stages=st) == 0
    assert v(block_m=12) == 3 and v(block_m=0) == 3 and v(block_m=136) == 3
    assert v(block_n=64, warp_n=8) == 4 and v(block_n=128, warp_n=2) == 4
    assert v(stages=0) == 5 and v(stages=6) == 5
    assert v(K=7168 + 64) == 2 and v(N=384) == 2 and v(M=0) == 2 and v(top_k=0) == 2
    assert v(K=7168 + 128) == 0                       # K % 256 == 128 is supported (the reference drops columns there)


def test_null_pointers_and_small_workspace_are_refused_without_touching_a_device(lib):
    args = [None] * 11 + [9, 64, 7168, 512, 257, 4431, 16, 64, 4, 3, 2.5, None, 0, None]
    assert lib.alpha_moe_fused_moe_w8a8_up_down(*args) == 1
    fake = [ctypes.c_void_p(4096)] * 11
    assert lib.alpha_moe_fused_moe_w8a8_up_down(*fake, 9, 64, 7168, 512, 257, 4431, 16, 64, 4, 3, 2.5, None, 0, None) == 7
    assert lib.alpha_moe_fused_moe_w8a8_up_down(*fake, 9, 64, 7168, 512, 257, 4431, 16, 64, 4, 3, 2.5,
                                                ctypes.c_void_p(4096), 1024, None) == 7
    assert lib.alpha_moe_fused_moe_w8a8_up_down(*fake, 9, 64, 7168, 512, 257, 4431, 12, 64, 4, 3, 2.5,
                                                ctypes.c_void_p(4096), 1 << 40, None) == 3
    # the store variant runs the same checks
    lib.alpha_moe_fused_moe_w8a8_up_down_store.restype = ctypes.c_int
    lib.alpha_moe_fused_moe_w8a8_up_down_store.argtypes = lib.alpha_moe_fused_moe_w8a8_up_down.argtypes
    assert lib.alpha_moe_fused_moe_w8a8_up_down_store(*args) == 1
    assert lib.alpha_moe_fused_moe_w8a8_up_down_store(*fake, 9, 64, 7168, 512, 257, 4431, 16, 64, 4, 3, 2.5, None, 0,
                                                      None) == 7
    assert lib.alpha_moe_fused_moe_w8a8_up_down_store(*fake, 9, 64, 7168, 512, 257, 4431, 12, 64, 4, 3, 2.5,
                                                      ctypes.c_void_p(4096), 1 << 40, None) == 3


def test_workspace_check_refuses_a_null_workspace(lib):
    lib.alpha_moe_workspace_check.restype = ctypes.c_int
    lib.alpha_moe_workspace_check.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    assert lib.alpha_moe_workspace_check(None, None) == 1


def test_zeroed_prefix_is_small_and_inside_every_workspace(lib):
    lib.alpha_moe_workspace_zero_bytes.restype = ctypes.c_size_t
    lib.alpha_moe_workspace_zero_bytes.argtypes = []
    z = lib.alpha_moe_workspace_zero_bytes()
    assert z > 0 and z % 256 == 0 and z <= 4 << 20
    assert z <= lib.alpha_moe_workspace_bytes(2, 1, 128, 256, 1, 16, 16)


def test_workspace_bytes_is_monotone_and_covers_both_kernel_families(lib):
    small = lib.alpha_moe_workspace_bytes(9, 1, 7168, 512, 257, 9 + 257 * 15, 16)
    big = lib.alpha_moe_workspace_bytes(9, 64, 7168, 512, 257, 576 + 257 * 15, 16)
    assert 0 < small < big < (1 << 31)
    direct = lib.alpha_moe_workspace_bytes(9, 64, 7168, 512, 257, 576 + 257 * 127, 128)
    assert direct >= 64 * 7168 * 4
    assert lib.alpha_moe_workspace_bytes(9, 0, 7168, 512, 257, 100, 16) == 0


def test_prep_entry_points_refuse_bad_arguments_without_touching_a_device(lib):
    lib.alpha_moe_per_token_group_quant_fp8.restype = ctypes.c_int
    lib.alpha_moe_per_token_group_quant_fp8.argtypes = (
        [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])
    lib.alpha_moe_align_workspace_bytes.restype = ctypes.c_size_t
    lib.alpha_moe_align_workspace_bytes.argtypes = [ctypes.c_int] * 2
    lib.alpha_moe_moe_align_block_size.restype = ctypes.c_int
    lib.alpha_moe_moe_align_block_size.argtypes = (
        [ctypes.c_void_p] + [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                                                  ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])
    assert lib.alpha_moe_per_token_group_quant_fp8(None, 0, None, None, 4, 128, None) == 1      # null pointer
    assert lib.alpha_moe_per_token_group_quant_fp8(8, 0, 8, 8, 4, 130, None) == 2               # K % 128
    assert lib.alpha_moe_align_workspace_bytes(0, 8) == 0
    assert lib.alpha_moe_align_workspace_bytes(1024, 8) == 8 * 4
    assert lib.alpha_moe_align_workspace_bytes(1025, 8) == 2 * 8 * 4
    assert lib.alpha_moe_moe_align_block_size(None, 32, 8, 16, None, 0, None, 0, None, None, 0, None) == 1
    # sorted_num must be numel + E * (block - 1), n_blocks its ceiling quotient
    assert lib.alpha_moe_moe_align_block_size(8, 32, 8, 16, 8, 100, 8, 7, 8, None, 0, None) == 2
    assert lib.alpha_moe_moe_align_block_size(8, 32, 5000, 16, 8, 32 + 5000 * 15, 8, 4690, 8, None, 0, None) == 2
    # more than 4096 slots need the scratch buffer
    assert lib.alpha_moe_moe_align_block_size(8, 5000, 8, 16, 8, 5120, 8, 320, 8, None, 0, None) == 7
