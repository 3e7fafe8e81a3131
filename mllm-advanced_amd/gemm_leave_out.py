"""What the prefill kernel's steady-state loop waits for: times gate_proj (K = 1536, N = 8960) at M = 512 and
M = 2048 on a library whose loop lacks one of its parts.

    make -C mllm-advanced_amd/csrc leaveout LEAVE_OUT=<mask>      # 1 barriers, 2 dequantisation + LDS writes,
    python3 mllm-advanced_amd/gemm_leave_out.py <mask>            # 4 packed-weight loads, 8 activation loads,
                                                                  # 16 LDS fragment reads, 32 products, 64 half of
                                                                  # the activation loads (masks add)

With mask 0 (or none) the product library is timed. A build with a part left out computes wrong results: the
figures say how much of the launch waits for that part, nothing else. Run every mask in a process of its own
(a process maps one library), on the same box: boxes differ by several percent.
"""
import importlib
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
pkg = importlib.import_module("mllm-advanced_amd")


def main():
    mask = int(sys.argv[1]) if len(sys.argv) > 1 else 0
    if mask:
        pkg.LIB_PATH = os.path.join(HERE, f"libw4a32_hip_leaveout{mask}.so")
    pkg.lib()
    gen = torch.Generator(device="cuda").manual_seed(0)
    K, N = 1536, 8960
    packs = [pkg.quant_pack_rhs(torch.randn((N, K), generator=gen, device="cuda") * 0.02) for _ in range(6)]
    line = []
    for M in (512, 2048, 8192):
        ws = pkg.quant_lhs(torch.randn((M, K), generator=gen, device="cuda"))
        y = torch.empty((M, N), device="cuda")
        for p in packs[:2]:
            pkg.matmul_quantized(ws, p, M, K, N, out=y)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(4):
            for p in packs:
                pkg.matmul_quantized(ws, p, M, K, N, out=y)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (4 * len(packs))
        line.append(f"M = {M}: {us:.1f} us ({2.0 * M * N * K / us / 1e6:.0f} TFLOP/s if the results were right)")
    print(f"left out: {mask}  " + "  ".join(line))


if __name__ == "__main__":
    main()
