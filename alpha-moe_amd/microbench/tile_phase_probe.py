"""Where a call of the tile (prefill) kernel spends its time: builds the library once per case with
-DALPHA_MOE_TILE_PROBE=<bits> (csrc/moe_tile.hip: parts of the kernel are then compiled out) and times the DeepSeek-V3
shard at one batch size with each.  The first case is the product's own code.  The results of the other calls are
wrong on purpose; this is a stopwatch, not a test.  Needs an MI355X, hipcc and torch (for device memory only).

    python alpha-moe_amd/microbench/tile_phase_probe.py [--shape ds] [--M 8192] [--block-m 128] [--calls 8]
"""
import argparse
import ctypes
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
sys.path.insert(0, PKG)

import torch  # noqa: E402
from alpha_moe_python.workloads import SHAPES, make_problem, make_weights  # noqa: E402

NO_UP, NO_DOWN, NO_Y, NO_REDUCE, ROW0, EXPERT8, NO_LOAD, NO_MMA = (1 << i for i in range(8))
CASES = [
    ("whole call", 0),
    ("tile kernel only (no reduce kernel)", NO_REDUCE),
    ("up/gate items only", NO_DOWN | NO_REDUCE),
    ("up/gate items only, operands cache-resident", NO_DOWN | NO_REDUCE | ROW0 | EXPERT8),
    ("up/gate items only, loads without matrix work", NO_DOWN | NO_REDUCE | NO_MMA),
    ("up/gate items only, loads without matrix work, cache-resident", NO_DOWN | NO_REDUCE | NO_MMA | ROW0 | EXPERT8),
    ("up/gate items only, matrix work without loads", NO_DOWN | NO_REDUCE | NO_LOAD),
    ("down items only, no result stores", NO_UP | NO_REDUCE | NO_Y),
    ("down items only, no result stores, loads without matrix work", NO_UP | NO_REDUCE | NO_Y | NO_MMA),
    ("down items only, with result stores", NO_UP | NO_REDUCE),
    ("neither item kind (queue walk + reduce kernel with no live rows)", NO_UP | NO_DOWN),
]


def build_probe_libraries(out_dir, masks):
    """One shared library per mask; only csrc/moe_tile.hip is compiled more than once."""
    import build as product_build   # the product's flags, so that nothing but the macro differs
    include = os.path.join(os.path.dirname(PKG), "include")
    jobs = []
    for src, extra in product_build.HIP_SOURCES.items():
        for mask in (masks if src == "moe_tile.hip" else [None]):
            obj = os.path.join(out_dir, src.replace(".hip", "") + ("" if mask is None else f"_{mask}") + ".o")
            cmd = [product_build.HIPCC] + product_build.HIP_FLAGS + extra + ["-I", include]
            if mask is not None:
                cmd.append(f"-DALPHA_MOE_TILE_PROBE={mask}")
            jobs.append((src, mask, obj, cmd + ["-c", os.path.join(PKG, "csrc", src), "-o", obj]))
    running = []
    for job in jobs:
        if len(running) == 12:
            if running.pop(0).wait() != 0:
                raise RuntimeError("probe build failed")
        running.append(subprocess.Popen(job[3], stderr=subprocess.DEVNULL))
    for pr in running:
        if pr.wait() != 0:
            raise RuntimeError("probe build failed")
    common = [j[2] for j in jobs if j[1] is None]
    libs = {}
    for src, mask, obj, _ in jobs:
        if mask is not None:
            libs[mask] = os.path.join(out_dir, f"libalpha_moe_probe_{mask}.so")
            subprocess.check_call([product_build.HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", libs[mask], obj]
                                  + common)
    return libs


def bind(path):
    lib = ctypes.CDLL(path)
    lib.alpha_moe_workspace_bytes.restype = ctypes.c_size_t
    lib.alpha_moe_workspace_bytes.argtypes = [ctypes.c_int] * 7
    lib.alpha_moe_fused_moe_w8a8_up_down.restype = ctypes.c_int
    lib.alpha_moe_fused_moe_w8a8_up_down.argtypes = ([ctypes.c_void_p] * 11 + [ctypes.c_int] * 10 +
                                                     [ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])
    return lib


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", default="ds")
    ap.add_argument("--M", type=int, default=8192)
    ap.add_argument("--block-m", type=int, default=128)
    ap.add_argument("--calls", type=int, default=8)
    ap.add_argument("--bits", type=int, nargs="*", help="only the cases with these bits (e.g. under rocprofv3 --pmc)")
    args = ap.parse_args()
    tmp = tempfile.mkdtemp(prefix="alpha_moe_probe_")
    cases = [c for c in CASES if args.bits is None or c[1] in args.bits]
    print("building one library per case ...", flush=True)
    libs = {mask: bind(path) for mask, path in build_probe_libraries(tmp, sorted({0} | {m for _, m in cases})).items()}
    lib = libs[0]
    dev = "cuda:0"
    W = make_weights(SHAPES[args.shape], device=dev, seed=0)
    P = make_problem(W, args.M, seed=0)
    sh = P.shape
    s_ids, e_ids, total = P.align(args.block_m)
    out = torch.zeros((args.M, sh.K), dtype=torch.bfloat16, device=dev)
    nbytes = lib.alpha_moe_workspace_bytes(sh.top_k, args.M, sh.K, sh.N, sh.E, s_ids.numel(), args.block_m)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    flush = torch.empty(1 << 27, dtype=torch.int32, device=dev)   # 512 MiB: evicts L2 and the Infinity Cache

    def call(lib):
        rc = lib.alpha_moe_fused_moe_w8a8_up_down(
            P.x.data_ptr(), P.x_scale.data_ptr(), W.w1.data_ptr(), W.w1_scale.data_ptr(), W.w2.data_ptr(),
            W.w2_scale.data_ptr(), out.data_ptr(), s_ids.data_ptr(), e_ids.data_ptr(), total.data_ptr(),
            P.topk_weights.data_ptr(), sh.top_k, args.M, sh.K, sh.N, sh.E, s_ids.numel(), args.block_m, 64, 4, 3,
            float(sh.scaling_factor), ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(f"status {rc}")

    print(f"{args.shape} M={args.M} block_m={args.block_m}: median of {args.calls} calls, each behind a 512 MiB fill")
    print(f"algorithmic flops {P.algorithmic_flops() / 1e9:.1f} G, bytes {P.algorithmic_bytes() / 1e6:.1f} MB")
    for name, mask in cases:
        call(libs[mask])
        torch.cuda.synchronize()
        ts = []
        for i in range(args.calls):
            flush.fill_(i)
            out.zero_()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            call(libs[mask])
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
        ts.sort()
        print(f"| {name} | {mask} | {ts[len(ts) // 2]:.1f} |", flush=True)


if __name__ == "__main__":
    main()
