"""CPU: the restated KleidiAI blob layout (parity unpinned: nothing in the reference tree can check it
against KleidiAI itself). What these tests can fix is that the packing loop, written over destination
bytes as the packer runs, and the closed form the decoders use are the same layout, that the sizes are
the ones the reference's quant_pack_rhs_size implies, and the nibble / sign conventions."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import kai_blob  # noqa: E402


def random_native(N, K, seed):
    rng = np.random.default_rng(seed)
    u4 = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    scales = (rng.standard_normal((N, K // 32)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    bias = rng.standard_normal(N).astype(np.float32)
    return u4, scales, bias


def test_blob_sizes_are_the_ones_of_quant_pack_rhs_size():
    # N * (0.5625 K + 8) for nr | N: the sizes of the 1.5B model's Linears
    assert kai_blob.blob_bytes(8960, 1536, 4) == 7_813_120
    assert kai_blob.blob_bytes(1536, 1536, 4) == 1_339_392
    assert kai_blob.blob_bytes(256, 1536, 8) == 223_232
    assert kai_blob.blob_bytes(1536, 8960, 4) == 7_753_728
    assert kai_blob.blob_bytes(50, 64, 4) == 52 * (2 * 18 + 8)      # N padded to nr


@pytest.mark.parametrize("impl", sorted(kai_blob.TILE_PARAMS))
@pytest.mark.parametrize("N,K", [(8, 64), (13, 96), (50, 256)])
def test_packing_loop_and_closed_form_agree(impl, N, K):
    nr, kr, sr = kai_blob.TILE_PARAMS[impl]
    u4, scales, bias = random_native(N, K, seed=impl * 100 + N)
    blob = kai_blob.pack(u4, scales, bias, nr, kr, sr)
    assert blob.size == kai_blob.blob_bytes(N, K, nr)
    u4b, scb, biasb, rsum = kai_blob.unpack(blob, N, K, nr, kr, sr)
    assert np.array_equal(u4b, u4) and np.array_equal(scb, scales) and np.array_equal(biasb, bias)
    # the row sums the packer leaves behind: sum_b scale_b * sum_k (u4 - 8)
    q = np.stack([(u4 & 0xF), (u4 >> 4)], axis=2).reshape(N, K).astype(np.int32) - 8
    sc = (scales.astype(np.uint32) << 16).view(np.float32)
    want = (q.reshape(N, K // 32, 32).sum(axis=2).astype(np.float32) * sc).sum(axis=1)
    assert np.allclose(rsum, want, rtol=1e-4, atol=1e-3)


def test_hand_placed_bytes_nr4_kr16():
    # one block, nr = 4, seg = 8: byte (s*4 + r)*8 + t holds k = 8s + t (low) and k + 16 (high) of row r
    N, K, nr, kr, sr = 4, 32, 4, 16, 2
    u4 = np.zeros((N, K // 2), dtype=np.uint8)
    setk = lambda n, k, v: u4.__setitem__((n, k // 2), u4[n, k // 2] | (v << (4 * (k & 1))))
    setk(2, 3, 0xF)        # row 2, k = 3  -> segment 0, byte (0*4+2)*8+3 = 19, low nibble
    setk(1, 27, 0x1)       # row 1, k = 27 = 16 + 8 + 3 -> segment 1, byte (1*4+1)*8+3 = 43, high nibble
    scales = np.full((N, 1), 0x3F80, dtype=np.uint16)
    blob = kai_blob.pack(u4, scales, None, nr, kr, sr)
    data = blob[:64] ^ 0x88
    assert data[19] == 0x0F and data[43] == 0x10 and int(data.sum()) == 0x1F
    assert blob[0] == 0x88                      # q = -8 in both nibbles is stored as 0x88
    assert bytes(blob[64:72]) == bytes([0x80, 0x3F] * 4)          # nr bf16 scales behind the data
    assert np.all(blob[72 + 16:] == 0)                              # no bias
