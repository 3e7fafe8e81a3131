"""Per-workgroup timelines of the decode kernel (gemv_fused_kernel) on the launch shapes of a Qwen2-1.5B token.

Needs the traced build of the library (`make -C mllm-advanced_amd/csrc trace`, which compiles the same sources
with -DW4A32_TRACE into libw4a32_hip_trace.so) and a GPU. Thread 0 of every workgroup stamps the 100 MHz wall
clock at seven points; for each launch shape this prints, over the workgroups of one launch on cold weights,
when each point was reached (ns after the first workgroup's start). Every stamp costs the kernel a few tens of
ns, so the traced launch runs about 0.3 us longer than the product's.

    python mllm-advanced_amd/trace_decode.py
"""
import ctypes
import importlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
pkg = importlib.import_module("mllm-advanced_amd")
pkg.LIB_PATH = os.path.join(HERE, "libw4a32_hip_trace.so")
L = pkg.lib()
L.w4a32_trace_dump.restype = ctypes.c_int
L.w4a32_trace_dump.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
POINTS = ["workgroup starts", "row arrived, range known", "quantisation parameters", "int8 row in LDS",
          "weights arrived, products done", "sums in LDS", "outputs stored"]


def trace(label, K, Ns, sets, nwg=None):
    g = torch.Generator(device="cuda").manual_seed(0)
    packs = [[pkg.quant_pack_rhs(torch.randn((n, K), generator=g, device="cuda") * 0.02) for n in Ns]
             for _ in range(sets)]                     # more weight sets than the 256 MB cache holds: cold every time
    x = torch.randn((1, K), generator=g, device="cuda")
    ys = [torch.empty((1, n), device="cuda") for n in Ns]
    ws = torch.empty(pkg.workspace_bytes(1, K), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    cnt = len(Ns)
    if nwg is None:
        nwg = sum((n + 15) // 16 for n in Ns)           # one workgroup per 16-row tile row of every Linear
    ya = (ctypes.c_void_p * cnt)(*[t.data_ptr() for t in ys])
    na = (ctypes.c_int * cnt)(*Ns)
    for _ in range(3):
        for p in packs:
            pa = (ctypes.c_void_p * cnt)(*[t.data_ptr() for t in p])
            assert L.w4a32_matmul_grouped(ya, x.data_ptr(), pa, na, cnt, ws.data_ptr(), 1, K, stream) == 0
    torch.cuda.synchronize()
    buf = np.zeros(8192 * 8, dtype=np.uint64)
    assert L.w4a32_trace_dump(buf.ctypes.data, buf.size) == 0
    t = buf.reshape(8192, 8)[:nwg, :7].astype(np.int64)
    rel = (t - t[:, 0].min()) * 10                      # ns
    print(f"== {label}: {nwg} workgroups; ns after the first workgroup's start")
    for i, name in enumerate(POINTS):
        c = rel[:, i]
        print(f"  {name:32s} min {c.min():5d}  p10 {int(np.percentile(c, 10)):5d}  median {int(np.median(c)):5d}"
              f"  p90 {int(np.percentile(c, 90)):5d}  max {c.max():5d}")
    d = np.diff(rel, axis=1)
    print("  step durations per workgroup, median ns:", [int(np.median(d[:, i])) for i in range(6)])


if __name__ == "__main__":
    # two Linears of equal N on one row run as a pair: a workgroup takes tile row nt of both
    trace("gate,up as a pair (K 1536, N 2 x 8960)", 1536, [8960, 8960], 20, nwg=8960 // 16)
    trace("o_proj (K 1536, N 1536)", 1536, [1536], 28)
    trace("q,k,v grouped (K 1536, N 1536 + 256 + 256)", 1536, [1536, 256, 256], 28)
    trace("down_proj unsplit, as w4a32_matmul runs it (K 8960, N 1536)", 8960, [1536], 28)
