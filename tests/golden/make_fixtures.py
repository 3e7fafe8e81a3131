"""Writes tests/golden/w4a32_small.npz with this repository's CPU oracle.

The reference holds no stored vectors for the W4A32 path (its test draws inputs with rand()
at run time), so the fixture is produced by the oracle, which tests/test_oracle_pins.py pins
to closed forms. It freezes one small case (M=3, K=64, N=8, with bias) so that a later change
to the oracle or to the HIP path that alters any integer or output shows up as a diff.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import w4a32_oracle as orc  # noqa: E402


def main():
    m, k, n = 3, 64, 8
    rng = np.random.default_rng(20251125)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    w[1, :32] = 0.0                       # a zero block
    w[2, 32:] = 0.25                      # a constant block
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[1] *= 20.0                          # an outlier row
    x[2] = np.abs(x[2])                   # a one-sided row
    bias = (rng.standard_normal(n) * 0.02).astype(np.float32)
    u4, sc = orc.quant_rhs(w)
    aq, recip, neg_zp, _ = orc.quant_lhs(x)
    y = orc.linear(x, u4, sc, bias=bias)
    out = os.path.join(ROOT, "tests", "golden", "w4a32_small.npz")
    np.savez(out, m=m, k=k, n=n, w=w, x=x, bias=bias, u4=u4, scales=sc, aq=aq, recip=recip,
             neg_zp=neg_zp, y=y, dequant=orc.dequant(u4, sc, k))
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
