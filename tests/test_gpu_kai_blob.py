"""GPU: the device decoder of the Arm quantizer's blob (parity unpinned: checked against this
repository's own restatement of KleidiAI's packing, oracle/kai_blob.py) gives back the native arrays
bit for bit, and a Linear built from it multiplies like one built from the native arrays."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import kai_blob  # noqa: E402

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("impl", sorted(kai_blob.TILE_PARAMS))
@pytest.mark.parametrize("N,K", [(13, 64), (50, 256), (256, 1536)])
def test_unpack_kai_gives_back_the_native_arrays(pkg, impl, N, K):
    nr, kr, sr = kai_blob.TILE_PARAMS[impl]
    rng = np.random.default_rng(impl + N)
    u4 = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    scales = ((rng.standard_normal((N, K // 32)) * 0.01).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    bias = rng.standard_normal(N).astype(np.float32)
    blob = kai_blob.pack(u4, scales, bias, nr, kr, sr)
    assert blob.size == int(pkg.lib().w4a32_kai_blob_bytes(N, K, nr))
    u4d, scd, biasd = pkg.unpack_kai(dev(blob), N, K, nr, kr, sr)
    assert np.array_equal(u4d.cpu().numpy(), u4)
    assert np.array_equal(scd.cpu().numpy().view(np.uint16), scales)
    assert np.array_equal(biasd.cpu().numpy(), bias)
    # and the Linear on top of it
    packed_k = pkg.repack_native(u4d, scd, biasd, N, K)
    packed_n = pkg.repack_native(dev(u4), dev(scales.view(np.int16)), dev(bias), N, K)
    assert torch.equal(packed_k, packed_n)


def test_unpack_kai_rejects_bad_tile_parameters(pkg):
    blob = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError):
        pkg.unpack_kai(blob, 8, 64, 3, 16, 2)      # nr is 4 or 8
    with pytest.raises(RuntimeError):
        pkg.unpack_kai(blob, 8, 64, 4, 16, 3)      # kr must be a multiple of sr
    assert int(pkg.lib().w4a32_kai_blob_bytes(8, 48, 4)) == 0
