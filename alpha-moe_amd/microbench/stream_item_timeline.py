"""Item timeline of the streaming (decode) kernel: builds the library once more with -DALPHA_MOE_STREAM_TRACE
(csrc/moe_stream.hip: every work item then leaves its start / wait-or-stream end / end times in a device array), runs
one cold call and prints, per item kind, when the items ran and how long they waited and worked, plus the bytes the
UP and DOWN items streamed per 10 us.  A stopwatch, not a test.  Needs an MI355X, hipcc and torch.

    python alpha-moe_amd/microbench/stream_item_timeline.py [--shape ds] [--M 64] [--knobs 16,64,4,4]
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

import numpy as np  # noqa: E402
import torch  # noqa: E402
from alpha_moe_python.workloads import SHAPES, make_problem, make_weights  # noqa: E402


def build_trace_library(out_dir):
    import build as product_build   # the product's flags, so that nothing but the macro differs
    include = os.path.join(os.path.dirname(PKG), "include")
    objs, procs = [], []
    for src, extra in product_build.HIP_SOURCES.items():
        obj = os.path.join(out_dir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [product_build.HIPCC] + product_build.HIP_FLAGS + extra + ["-I", include]
        if src == "moe_stream.hip":
            cmd.append("-DALPHA_MOE_STREAM_TRACE")
        procs.append(subprocess.Popen(cmd + ["-c", os.path.join(PKG, "csrc", src), "-o", obj], stderr=subprocess.DEVNULL))
    for pr in procs:
        if pr.wait() != 0:
            raise RuntimeError("trace build failed")
    lib = os.path.join(out_dir, "libalpha_moe_trace.so")
    subprocess.check_call([product_build.HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    return lib


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", default="ds")
    ap.add_argument("--M", type=int, default=64)
    ap.add_argument("--knobs", default="16,64,4,4")
    args = ap.parse_args()
    bm, bn, wn, st = (int(v) for v in args.knobs.split(","))
    print("building the trace library ...", flush=True)
    lib = ctypes.CDLL(build_trace_library(tempfile.mkdtemp(prefix="alpha_moe_trace_")))
    lib.alpha_moe_workspace_bytes.restype = ctypes.c_size_t
    lib.alpha_moe_workspace_bytes.argtypes = [ctypes.c_int] * 7
    lib.alpha_moe_fused_moe_w8a8_up_down.restype = ctypes.c_int
    lib.alpha_moe_fused_moe_w8a8_up_down.argtypes = ([ctypes.c_void_p] * 11 + [ctypes.c_int] * 10 +
                                                     [ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])
    lib.alpha_moe_debug_trace_read.restype = ctypes.c_int
    lib.alpha_moe_debug_trace_read.argtypes = [ctypes.c_void_p, ctypes.c_int]
    dev = "cuda:0"
    W = make_weights(SHAPES[args.shape], device=dev, seed=0)
    P = make_problem(W, args.M, seed=0)
    sh = P.shape
    s_ids, e_ids, total = P.align(bm)
    out = torch.zeros((args.M, sh.K), dtype=torch.bfloat16, device=dev)
    nbytes = lib.alpha_moe_workspace_bytes(sh.top_k, args.M, sh.K, sh.N, sh.E, s_ids.numel(), bm)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    flush = torch.empty(1 << 27, dtype=torch.int32, device=dev)   # 512 MiB: evicts L2 and the Infinity Cache
    buf = np.zeros((1 << 16, 4), dtype=np.uint64)
    n = 0
    for it in range(3):   # the last of three cold calls is the one looked at
        flush.fill_(it)
        out.zero_()
        torch.cuda.synchronize()
        lib.alpha_moe_debug_trace_read(buf.ctypes.data, 1 << 16)
        rc = lib.alpha_moe_fused_moe_w8a8_up_down(
            P.x.data_ptr(), P.x_scale.data_ptr(), W.w1.data_ptr(), W.w1_scale.data_ptr(), W.w2.data_ptr(),
            W.w2_scale.data_ptr(), out.data_ptr(), s_ids.data_ptr(), e_ids.data_ptr(), total.data_ptr(),
            P.topk_weights.data_ptr(), sh.top_k, args.M, sh.K, sh.N, sh.E, s_ids.numel(), bm, bn, wn, st,
            float(sh.scaling_factor), ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(f"status {rc}")
        torch.cuda.synchronize()
        n = lib.alpha_moe_debug_trace_read(buf.ctypes.data, 1 << 16)
    if n == 0:
        raise RuntimeError("no records: these knobs do not select the streaming kernel")
    r = buf[:n].astype(np.int64)
    kind = (r[:, 0] >> 56) & 0xff
    wg = (r[:, 0] >> 32) & 0xffffff
    t0, t1, t2 = r[:, 1], r[:, 2], r[:, 3]
    base = t0.min()

    def us(v):
        return (v - base) / 100.0

    print(f"{args.shape} M={args.M} knobs=({bm},{bn},{wn},{st}): {n} items on {len(np.unique(wg))} workgroups, "
          f"first item start to last item end {us(t2.max()):.1f} us")
    for k, name, first, second in ((1, "UP", "streaming", "hand-over"), (2, "DOWN", "prologue+wait", "streaming"),
                                   (3, "FIN", "wait", "work")):
        m = kind == k
        if not m.any():
            continue
        a, b = (t1[m] - t0[m]) / 100.0, (t2[m] - t1[m]) / 100.0
        print(f"| {name} | {int(m.sum())} | start {us(t0[m].min()):.1f} .. {us(t0[m].max()):.1f} | end {us(t2[m].min()):.1f} .. "
              f"{us(t2[m].max()):.1f} | {first} mean {a.mean():.1f} max {a.max():.1f} | {second} mean {b.mean():.1f} max {b.max():.1f} |")
    act = e_ids[: int(total.item()) // bm]
    n_units = int((act >= 0).sum().item()) * (sh.N // 256)
    up_bytes, down_bytes = n_units * 256 * sh.K, n_units * sh.K * 128
    n_upi, n_dni = max(int((kind == 1).sum()), 1), max(int((kind == 2).sum()), 1)
    nb = int(us(t2.max()) // 10) + 1
    per = np.zeros((nb, 3))
    for k, a, b, c in zip(kind, t0, t1, t2):
        if k == 1:
            lo, hi, by = us(a), us(b), up_bytes / n_upi
        elif k == 2:
            lo, hi, by = us(b), us(c), down_bytes / n_dni
        else:
            continue
        hi = max(hi, lo + 0.01)
        for i in range(int(lo // 10), min(int(hi // 10) + 1, nb)):
            per[i, k] += by * max(0.0, min(hi, (i + 1) * 10) - max(lo, i * 10)) / (hi - lo)
    print("| from us | UP TB/s | DOWN TB/s | workgroups in UP / DOWN items |")
    for i in range(nb):
        mid = i * 10 + 5
        n_up = int(((kind == 1) & (us(t0) <= mid) & (us(t2) > mid)).sum())
        n_dn = int(((kind == 2) & (us(t0) <= mid) & (us(t2) > mid)).sum())
        print(f"| {i * 10} | {per[i, 1] / 10 / 1e6:.2f} | {per[i, 2] / 10 / 1e6:.2f} | {n_up} / {n_dn} |")


if __name__ == "__main__":
    main()
