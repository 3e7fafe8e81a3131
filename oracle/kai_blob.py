"""TEST INFRASTRUCTURE, not a product path (only tests/ import this file).

PARITY UNPINNED. Byte layout of the weight blob that the reference's Arm quantizer stores in a
`.mllm` file for the W4A32 Linear, i.e. the output of
    kai_run_rhs_pack_nxk_qsi4c32p_qsu4c32s1s0(1, N, K, nr, kr, sr, bl=32, rhs_u4, K/2, bias, scales,
                                              nb*2, out, 0, {lhs_zero_point=1, rhs_zero_point=8, bf16})
called at mllm/Backends/Arm/Kernels/kai_linear.cpp:331-344. That routine lives in KleidiAI
(ARM-software/kleidiai), a git submodule that is an empty directory in the reference tree, whose
pinned revision cannot be read from it (no .git), and which needs arm_neon.h. The reference holds no
golden blob either. What follows restates the published packing loop from memory; nothing here can
check it against KleidiAI itself, so every consumer of this layout says "parity unpinned".

Layout as restated (nb = K/32 blocks per row, rows in groups of nr, N padded up to a multiple of nr):

  group g (rows g*nr .. g*nr+nr-1) occupies nr * (nb*18 + 8) bytes:
    for each block b:
      nr*16 data bytes: byte i of the block belongs to
          segment      s  = i // (nr*seg)           seg = kr // sr bytes (8 for kr=16, 4 for kr=8)
          row in group r  = (i // seg) % nr
          byte in seg  t  = i % seg
        its low nibble is the weight at k = 32*b + s*seg + t, its high nibble the one at k + 16,
        both as u4 (q + 8) XOR 8, i.e. the two's complement nibble of q (the byte is XORed with 0x88)
      nr bf16 scales (row order)
    nr f32 "rsum" = sum over blocks of scale * sum_k (u4 - 8)      (recomputed here, not consumed)
    nr f32 bias (0 when the layer has none)

Tile parameters of the reference's six W4A32 implementations (LinearOpImplType 3..8,
mllm/Core/AOps/LinearOp.hpp:21-26, ukernel table kai_linear.cpp:123-218): nr from "qsi4c32p<nr>x<..>",
kr/sr from the micro-kernel family: p4x8 / p8x8 -> kr 16, sr 2; p4x4 -> kr 8, sr 2.
"""
import numpy as np

TILE_PARAMS = {3: (4, 16, 2), 4: (8, 16, 2), 5: (4, 16, 2), 6: (4, 16, 2), 7: (8, 16, 2), 8: (4, 8, 2)}


def blob_bytes(N, K, nr):
    nb = K // 32
    return (N + nr - 1) // nr * nr * (nb * 18 + 8)


def _bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def pack(u4, scales_bf16, bias, nr, kr, sr):
    """u4: uint8 [N][K/2] (low nibble = even k), scales_bf16: uint16 [N][K/32], bias: f32 [N] or None.

    Written as the packing loop runs: over destination bytes, computing the two source positions."""
    N, half = u4.shape
    K, nb = 2 * half, half // 16
    assert K % 32 == 0 and scales_bf16.shape == (N, nb)
    seg = kr // sr
    groups = (N + nr - 1) // nr
    out = np.zeros(blob_bytes(N, K, nr), dtype=np.uint8)
    stride = nr * (nb * 18 + 8)
    nib = lambda n, k: int((u4[n, k // 2] >> (4 * (k & 1))) & 0xF)
    for g in range(groups):
        base = g * stride
        sums = np.zeros(nr, dtype=np.float32)
        p = base
        for b in range(nb):
            for i in range(nr * 16):
                block_idx, t = divmod(i, seg)
                s, r = divmod(block_idx, nr)
                k_adj = ((t + s * seg) // 16) * 16
                k0 = 32 * b + t + s * seg + k_adj
                k1 = k0 + 16
                n = min(g * nr + r, N - 1)               # rows past N repeat the last one
                lo, hi = nib(n, k0), nib(n, k1)
                sc = _bf16_to_f32(scales_bf16[n:n + 1, b])[0]
                sums[r] += np.float32((lo - 8) + (hi - 8)) * sc
                out[p] = (lo | (hi << 4)) ^ 0x88
                p += 1
            for r in range(nr):
                n = min(g * nr + r, N - 1)
                out[p:p + 2] = np.frombuffer(scales_bf16[n, b].tobytes(), dtype=np.uint8)
                p += 2
        out[p:p + 4 * nr] = sums.view(np.uint8)
        p += 4 * nr
        bz = np.zeros(nr, dtype=np.float32)
        for r in range(nr):
            if bias is not None and g * nr + r < N:
                bz[r] = bias[g * nr + r]
        out[p:p + 4 * nr] = bz.view(np.uint8)
    return out


def unpack(blob, N, K, nr, kr, sr):
    """The closed form of the same layout, vectorised: returns u4 [N][K/2], scales [N][nb], bias [N]."""
    nb, seg = K // 32, kr // sr
    groups = (N + nr - 1) // nr
    stride = nr * (nb * 18 + 8)
    b8 = np.asarray(blob, dtype=np.uint8).reshape(groups, stride)
    blocks = b8[:, :nb * nr * 18].reshape(groups, nb, nr * 18)
    data = blocks[:, :, :nr * 16] ^ 0x88                                  # back to u4 nibbles
    data = data.reshape(groups, nb, 16 // seg, nr, seg)                   # [g][b][s][r][t]
    lo = (data & 0xF).transpose(0, 3, 1, 2, 4).reshape(groups * nr, nb, 16)   # k = s*seg + t
    hi = (data >> 4).transpose(0, 3, 1, 2, 4).reshape(groups * nr, nb, 16)    # k + 16
    vals = np.concatenate([lo, hi], axis=2).reshape(groups * nr, K)[:N]
    u4 = (vals[:, 0::2] | (vals[:, 1::2] << 4)).astype(np.uint8)
    sc = blocks[:, :, nr * 16:].reshape(groups, nb, nr, 2)
    sc = np.ascontiguousarray(sc.transpose(0, 2, 1, 3)).reshape(groups * nr, nb, 2).copy().view(np.uint16)
    scales = sc.reshape(groups * nr, nb)[:N]
    tail = np.ascontiguousarray(b8[:, nb * nr * 18:]).view(np.float32).reshape(groups, 2, nr)
    bias = tail[:, 1, :].reshape(groups * nr)[:N].copy()
    rsum = tail[:, 0, :].reshape(groups * nr)[:N].copy()
    return u4, scales.copy(), bias, rsum
