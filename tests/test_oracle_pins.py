"""Pins the CPU oracle to facts that do not depend on it.

The reference stores no golden vectors for this path (its test draws inputs with
rand() at run time), so each oracle function is pinned by closed forms, invariants,
brute force on tiny inputs and reductions to library routines, chosen so that a
dropped term, a wrong sign or index, a swapped nibble or a wrong rounding mode fails
at least one of them. Reference lines are cited next to the fact they fix.
"""
import numpy as np
import pytest
import torch

from conftest import make_acts, make_weights


# --------------------------------------------------------------------------- bf16

def test_bf16_trunc_is_upper_half_word(orc):
    # tests/Arm/KaiLinearTest.hpp:138-139
    vals = np.array([0.0, -0.0, 1.0, -1.0, 0.02, 3.14159, 1e-30, -7.25e12, 1.0 + 2**-8, 1.0 + 2**-7],
                    dtype=np.float32)
    for v in vals:
        assert orc.bf16_trunc(v) == int(np.array([v], np.float32).view(np.uint32)[0] >> 16)
    # round trip widens by a 16-bit shift (KaiLinearTest.hpp:144-149)
    assert orc.f32_from_bf16(0x3F80) == 1.0
    assert orc.f32_from_bf16(0xC000) == -2.0


def test_bf16_rne_matches_ieee_cast(orc):
    rng = np.random.default_rng(7)
    vals = np.concatenate([
        rng.standard_normal(2000).astype(np.float32) * 0.02,
        np.array([1.0 + 2**-8, 1.0 + 3 * 2**-8, 1.0 + 2**-8 + 2**-20, -(1.0 + 2**-8)], np.float32),
    ])
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([orc.bf16_rne(v) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    # the two ties above: 1+2^-8 -> even (down), 1+3*2^-8 -> even (up)
    assert orc.bf16_rne(np.float32(1.0 + 2**-8)) == 0x3F80
    assert orc.bf16_rne(np.float32(1.0 + 3 * 2**-8)) == 0x3F82
    assert orc.bf16_trunc(np.float32(1.0 + 3 * 2**-8)) == 0x3F81


# ---------------------------------------------------------------- weight quantizer

def nibbles(u4_row, k):
    out = np.empty(k, dtype=np.int32)
    out[0::2] = u4_row[: (k + 1) // 2] & 0x0F
    out[1::2] = (u4_row[: k // 2] >> 4)
    return out


def test_rhs_constant_block_maps_to_minus_eight(orc):
    # abs-max element / -8 is the scale, so a constant block c has every q = c/(c/-8) = -8
    for c in (0.5, -0.5, 3.0):
        w = np.full((1, 32), c, dtype=np.float32)
        u4, sc = orc.quant_rhs(w)
        assert np.all(u4 == 0x00)
        assert sc[0, 0] == orc.bf16_trunc(np.float32(c / -8.0))


def test_rhs_zero_block(orc):
    # max stays +0.0f, scale = 0.0f / -8.0 = -0.0f (bf16 0x8000, kai_linear.cpp:254), which is
    # falsy -> recip 0 (kai_linear.cpp:255) -> q = 0 -> u4 = 8 in both nibbles
    u4, sc = orc.quant_rhs(np.zeros((2, 64), np.float32))
    assert np.all(u4 == 0x88)
    assert np.all(sc == 0x8000)


def test_rhs_one_hot_block_and_nibble_order(orc):
    # one non-zero value v at position p: q[p] = -8 (u4 0), all others q = 0 (u4 8);
    # even k sits in the low nibble of byte k/2 (kai_linear.cpp:278-285)
    for p in (0, 1, 6, 31):
        w = np.zeros((1, 32), np.float32)
        w[0, p] = 1.25
        u4, _ = orc.quant_rhs(w)
        want = np.full(16, 0x88, np.uint8)
        want[p // 2] = 0x80 if p % 2 == 0 else 0x08
        assert np.array_equal(u4[0], want), p


def test_rhs_recovers_planted_integers(orc):
    # w = q * 2^-5 with a planted -8: scale is exactly 2^-5 and every q must come back,
    # at its own k (catches index/nibble swaps) and for each row/block separately.
    rng = np.random.default_rng(3)
    n, k = 3, 96
    q = rng.integers(-8, 8, size=(n, k)).astype(np.int32)
    e = rng.integers(-9, -2, size=(n, k // 32))
    for r in range(n):
        for b in range(k // 32):
            q[r, 32 * b + int(rng.integers(0, 32))] = -8
    w = (q * np.exp2(np.repeat(e, 32, axis=1))).astype(np.float32)
    u4, sc = orc.quant_rhs(w)
    for r in range(n):
        assert np.array_equal(nibbles(u4[r], k) - 8, q[r])
        for b in range(k // 32):
            assert orc.f32_from_bf16(sc[r, b]) == 2.0 ** e[r, b]


def test_rhs_negation_keeps_nibbles_flips_scale(orc):
    w = make_weights(4, 128, seed=11)
    u4a, sca = orc.quant_rhs(w)
    u4b, scb = orc.quant_rhs(-w)
    assert np.array_equal(u4a, u4b)
    assert np.array_equal(sca ^ 0x8000, scb)


def test_rhs_tie_keeps_first_maximum(orc):
    # |w[3]| == |w[7]|, strict '<' keeps index 3 (kai_linear.cpp:248): scale = a/-8 < 0,
    # q[3] = -8, q[7] = round(-a * -8/a) = 8 -> clamped to 7
    w = np.zeros((1, 32), np.float32)
    w[0, 3], w[0, 7] = 2.0, -2.0
    u4, sc = orc.quant_rhs(w)
    q = nibbles(u4[0], 32) - 8
    assert q[3] == -8 and q[7] == 7
    assert orc.f32_from_bf16(sc[0, 0]) == -0.25
    w[0, 3], w[0, 7] = -2.0, 2.0
    u4, sc = orc.quant_rhs(w)
    q = nibbles(u4[0], 32) - 8
    assert q[3] == -8 and q[7] == 7
    assert orc.f32_from_bf16(sc[0, 0]) == 0.25


def test_rhs_rounds_half_away_from_zero(orc):
    # scale = 2^-3 exactly (planted -1.0 = -8 * 2^-3); x/scale hits .5 exactly
    w = np.zeros((1, 32), np.float32)
    w[0, 0] = -1.0
    halves = {1: 0.5, 2: 1.5, 3: 2.5, 4: -0.5, 5: -2.5, 6: 6.5, 7: 7.5}
    for idx, t in halves.items():
        w[0, idx] = t * 0.125
    q = nibbles(orc.quant_rhs(w)[0][0], 32) - 8
    assert [q[i] for i in range(1, 8)] == [1, 2, 3, -1, -3, 7, 7]  # 7.5 -> 8 -> clamp 7


def test_rhs_reconstruction_bound_and_exact_max(orc):
    w = make_weights(16, 256, seed=5)
    u4, sc = orc.quant_rhs(w)
    for r in range(16):
        q = nibbles(u4[r], 256) - 8
        for b in range(8):
            blk = w[r, 32 * b: 32 * b + 32]
            j = int(np.argmax(np.abs(blk)))
            s = np.float32(blk[j]) / np.float32(-8.0)
            assert q[32 * b + j] == -8                      # the abs-max element is exactly -8 * s
            err = np.abs(blk.astype(np.float64) - q[32 * b: 32 * b + 32] * float(s))
            unclamped = q[32 * b: 32 * b + 32] < 7
            assert np.all(err[unclamped] <= abs(float(s)) * 0.5 * (1 + 1e-6))
            assert np.all(err <= abs(float(s)) * (1 + 1e-6))
            assert sc[r, b] == orc.bf16_trunc(s)


def test_rhs_k_tail_block(orc):
    # K = 40: second block has 8 elements (the loops stop at k, kai_linear.cpp:243,265)
    w = np.zeros((1, 40), np.float32)
    w[0, 32:40] = -4.0
    u4, sc = orc.quant_rhs(w)
    assert u4.shape == (1, 20) and sc.shape == (1, 2)
    assert np.all(u4[0, :16] == 0x88) and np.all(u4[0, 16:] == 0x00)
    assert orc.f32_from_bf16(sc[0, 1]) == 0.5


# ------------------------------------------------------------- activation quantizer

def test_lhs_zero_row(orc):
    # rmin == rmax -> scale 1; (-128+0)+(127+0) = -1 is not > 0 -> zp = 127 - 0
    # (KaiLinearTest.hpp:187,198-200): every a_q = 127 and a_q + offset = 0
    aq, recip, neg_zp, _ = orc.quant_lhs(np.zeros((1, 64), np.float32))
    assert recip[0] == 1.0 and neg_zp[0] == -127 and np.all(aq == 127)


def test_lhs_one_sided_rows(orc):
    x = np.zeros((2, 32), np.float32)
    x[0, 5] = 4.0          # rmin 0, rmax 4: zp = -128, a_q(4) = 255 - 128
    x[1, 9] = -4.0         # rmin -4, rmax 0: zp = 127, a_q(-4) = -255 + 127
    aq, recip, neg_zp, _ = orc.quant_lhs(x)
    assert neg_zp[0] == 128 and aq[0, 5] == 127 and np.all(np.delete(aq[0], 5) == -128)
    assert neg_zp[1] == -127 and aq[1, 9] == -128 and np.all(np.delete(aq[1], 9) == 127)
    assert recip[0] == np.float32(1.0) / (np.float32(255.0) / np.float32(4.0))


def test_lhs_symmetric_row_pins_rounding_modes(orc):
    # +-c with c = 2: scale = 63.75, zero point candidate 127 - 127.5 = -0.5 -> lrintf (nearest
    # even) -> 0; a half-away zero point would be -1.  Values: round(127.5) = 128 -> clamp 127,
    # round(-127.5) = -128 (round() is half away from zero; nearest-even would give 128/-128 too,
    # so also plant 0.5/scale-type ties below).
    x = np.zeros((1, 32), np.float32)
    x[0, 0], x[0, 1] = 2.0, -2.0
    aq, recip, neg_zp, _ = orc.quant_lhs(x)
    assert neg_zp[0] == 0
    assert aq[0, 0] == 127 and aq[0, 1] == -128 and np.all(aq[0, 2:] == 0)

    # range [-100, 155] -> scale exactly 1, zp = -128 + 100 = -28: ties x.5 round away from zero
    y = np.zeros((1, 32), np.float32)
    y[0, :6] = [-100.0, 155.0, 0.5, 1.5, -0.5, -2.5]
    aq, recip, neg_zp, _ = orc.quant_lhs(y)
    assert recip[0] == 1.0 and neg_zp[0] == 28
    assert list(aq[0, :6]) == [-128, 127, 1 - 28, 2 - 28, -1 - 28, -3 - 28]


def test_lhs_error_bound_and_range(orc):
    x = make_acts(8, 512, seed=2, outlier_frac=0.25)
    aq, recip, neg_zp, _ = orc.quant_lhs(x)
    for r in range(8):
        deq = (aq[r].astype(np.float64) + neg_zp[r]) * float(recip[r])
        inner = (aq[r] > -128) & (aq[r] < 127)
        assert np.all(np.abs(deq - x[r])[inner] <= 0.5 * recip[r] * (1 + 1e-5))
        assert np.abs(deq - x[r]).max() <= 1.0 * recip[r] * (1 + 1e-5)
        # zero is representable exactly: 0 -> a_q = zp
        assert -128 <= -neg_zp[r] <= 127
        # monotone
        order = np.argsort(x[r], kind="stable")
        assert np.all(np.diff(aq[r][order].astype(np.int32)) >= 0)


def test_lhs_row_header_layout(orc):
    # KaiLinearTest.hpp:208-214: f32 recip, i32 -zp, then k int8
    x = make_acts(3, 64, seed=4)
    aq, recip, neg_zp, raw = orc.quant_lhs(x)
    assert raw.shape == (3, 64 + 8)
    assert np.array_equal(raw[:, 8:], aq)
    assert np.array_equal(raw[:, :4].copy().view(np.float32).ravel(), recip)


# ------------------------------------------------------------------------ matmul

def exact_case(m, n, k, seed):
    """Inputs on which both quantizers are lossless, so the op equals a plain matmul."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-100, 156, size=(m, k)).astype(np.float32)
    x[:, 0], x[:, 1] = -100.0, 155.0          # pins scale = 255/255 = 1, zp = -28
    q = rng.integers(-8, 8, size=(n, k)).astype(np.int64)
    e = rng.integers(-7, -1, size=(n, k // 32))
    for r in range(n):
        for b in range(k // 32):
            q[r, 32 * b + int(rng.integers(0, 32))] = -8
    w = (q * np.exp2(np.repeat(e, 32, axis=1))).astype(np.float32)
    return x, w


@pytest.mark.parametrize("m,n,k", [(1, 8, 32), (3, 5, 64), (4, 16, 256), (2, 7, 1024)])
def test_matmul_equals_numpy_on_lossless_inputs(orc, m, n, k):
    x, w = exact_case(m, n, k, seed=m * 100 + n)
    u4, sc = orc.quant_rhs(w)
    y = orc.linear(x, u4, sc)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.array_equal(y.astype(np.float64), want)      # exact: all partial sums fit in 24 bits


def test_matmul_bias_is_added_after_scaling(orc):
    x, w = exact_case(3, 6, 64, seed=9)
    bias = np.arange(6, dtype=np.float32) * 4.0 - 8.0
    u4, sc = orc.quant_rhs(w)
    y0 = orc.linear(x, u4, sc)
    y1 = orc.linear(x, u4, sc, bias=bias)
    assert np.array_equal(y1, y0 + bias[None, :])


def test_matmul_brute_force_k32(orc):
    # one block, one output: redo the arithmetic with Python ints / numpy float32
    x = make_acts(1, 32, seed=21)
    w = make_weights(2, 32, seed=22)
    u4, sc = orc.quant_rhs(w)
    aq, recip, neg_zp, raw = orc.quant_lhs(x)
    y = orc.matmul_packed(raw, u4, sc)
    for c in range(2):
        q = nibbles(u4[c], 32) - 8
        iacc = sum((int(aq[0, i]) + int(neg_zp[0])) * int(q[i]) for i in range(32))
        s = np.float32(orc.f32_from_bf16(sc[c, 0]))
        want = np.float32(np.float32(np.float32(iacc) * s) * recip[0])
        assert y[0, c] == want


def test_matmul_rows_are_independent(orc):
    x = make_acts(5, 128, seed=31, outlier_frac=0.2)
    w = make_weights(9, 128, seed=32)
    u4, sc = orc.quant_rhs(w)
    y = orc.linear(x, u4, sc)
    perm = np.array([3, 0, 4, 1, 2])
    assert np.array_equal(orc.linear(x[perm], u4, sc), y[perm])
    for r in range(5):
        assert np.array_equal(orc.linear(x[r:r + 1], u4, sc)[0], y[r])
    cperm = np.random.default_rng(1).permutation(9)
    assert np.array_equal(orc.linear(x, u4[cperm], sc[cperm]), y[:, cperm])


def test_matmul_clamp(orc):
    x, w = exact_case(2, 4, 32, seed=5)
    u4, sc = orc.quant_rhs(w)
    _, _, _, raw = orc.quant_lhs(x)
    y = orc.matmul_packed(raw, u4, sc)
    yc = orc.matmul_packed(raw, u4, sc, lo=-1.0, hi=2.0)
    assert np.array_equal(yc, np.clip(y, -1.0, 2.0))


def test_matmul_threads_do_not_change_results(orc):
    x = make_acts(4, 256, seed=41)
    w = make_weights(33, 256, seed=42)
    u4, sc = orc.quant_rhs(w)
    assert np.array_equal(orc.linear(x, u4, sc, threads=1), orc.linear(x, u4, sc, threads=4))


def test_dequant_is_q_times_scale(orc):
    w = make_weights(4, 96, seed=6)
    u4, sc = orc.quant_rhs(w)
    d = orc.dequant(u4, sc, 96)
    for r in range(4):
        q = nibbles(u4[r], 96) - 8
        s = np.array([orc.f32_from_bf16(v) for v in sc[r]], np.float32)
        assert np.array_equal(d[r], (q.astype(np.float32) * np.repeat(s, 32)))


def test_reference_test_case_is_close_to_dense_matmul(orc):
    # The reference's own test protocol (KaiLinearTest.hpp:391-427, 473-476): M=1, K=N=1024,
    # uniform[-1,1] from srand(4568)/srand(4572). No stored outputs exist, so this checks the
    # quantized result against the dense product within the format's error budget, and the
    # generator against its definition.
    lhs = orc.fill_uniform_random(1, 1024, 4568)
    rhs = orc.fill_uniform_random(1024, 1024, 4572)
    assert lhs.min() >= -1.0 and lhs.max() <= 1.0 and abs(float(rhs.mean())) < 5e-3
    assert np.array_equal(lhs, orc.fill_uniform_random(1, 1024, 4568))
    u4, sc = orc.quant_rhs(rhs)
    y = orc.linear(lhs, u4, sc)
    dense = lhs.astype(np.float64) @ rhs.astype(np.float64).T
    # 4-bit weights: per-element error <= scale/2 ~ 1/16 of the block max; sum over 1024 terms
    rms = float(np.sqrt(np.mean((y - dense) ** 2)))
    assert rms < 0.06 * float(np.sqrt(np.mean(dense ** 2))) + 0.5
    assert np.corrcoef(y.ravel(), dense.ravel())[0, 1] > 0.995


def test_input_generator_is_glibc_rand_scaled_to_minus_one_one(orc):
    # glibc's rand() after srand(1) is a published sequence (1804289383, 846930886, 1681692777, 1714636915,
    # 1957747793, ...), and the reference's generator is (float)((double)rand() / RAND_MAX) * 2 - 1 filled
    # row by row (tests/Arm/KaiLinearTest.hpp:154-161): a known-answer pin that does not use the oracle.
    seq = [1804289383, 846930886, 1681692777, 1714636915, 1957747793, 424238335]
    want = np.array([np.float32(np.float32(v / 2147483647.0) * np.float32(2.0)) - np.float32(1.0) for v in seq],
                    dtype=np.float32)
    got = orc.fill_uniform_random(2, 3, 1)
    assert got.shape == (2, 3) and np.array_equal(got.ravel(), want)


# --------------------------------------------------------------------------- an independent library routine

def torch_dyn_quant_linear(x, u4, sc_bits, bias):
    """PyTorch's own W4 dynamic-quantised Linear (aten::_dyn_quant_pack_4bit_weight +
    aten::_dyn_quant_matmul_4bit, block 32, bf16 scales): on this x86 build its portable C++ path,
    written by the authors of the Arm kernels as the reference for the same qai8dxp x qsi4c32p
    scheme. Same input format as the oracle's: u4 [N][K/2] with the even k in the low nibble,
    bf16 scales [N][K/32], optional f32 bias."""
    n, k = u4.shape[0], u4.shape[1] * 2
    tw = torch.from_numpy(np.ascontiguousarray(u4))
    ts = torch.from_numpy(np.ascontiguousarray(sc_bits).view(np.int16)).view(torch.bfloat16)
    tb = None if bias is None else torch.from_numpy(np.ascontiguousarray(bias))
    packed = torch.ops.aten._dyn_quant_pack_4bit_weight(tw, ts, tb, 32, k, n)
    return torch.ops.aten._dyn_quant_matmul_4bit(torch.from_numpy(np.ascontiguousarray(x)), packed, 32, k,
                                                 n).numpy()


needs_torch_dynq = pytest.mark.skipif(not hasattr(torch.ops.aten, "_dyn_quant_matmul_4bit"),
                                      reason="this torch build has no aten::_dyn_quant_matmul_4bit")


@needs_torch_dynq
@pytest.mark.parametrize("m,k,n,has_bias", [(1, 32, 4, False), (1, 64, 8, True), (3, 128, 16, True),
                                            (8, 1536, 256, True), (4, 1536, 64, False), (2, 8960, 48, False),
                                            (5, 1280, 40, True)])
def test_oracle_equals_torch_dyn_quant_matmul(orc, m, k, n, has_bias):
    # Row quantiser, zero point, integer block dots, bf16 scales, lhs scale, bias and clamp of the whole op
    # against a routine this repository did not write: bit for bit, on random rows with outliers.
    w = make_weights(n, k, seed=k + n)
    x = make_acts(m, k, seed=m + k, outlier_frac=0.25)
    bias = (np.random.default_rng(n).standard_normal(n) * 0.02).astype(np.float32) if has_bias else None
    u4, sc = orc.quant_rhs(w)
    got = orc.linear(x, u4, sc, bias=bias)
    want = torch_dyn_quant_linear(x, u4, sc, bias)
    assert np.array_equal(got, want)


@needs_torch_dynq
def test_oracle_equals_torch_dyn_quant_matmul_on_corner_rows(orc):
    # the rows that pin the quantiser's special cases: all zero, constant, one-sided, symmetric (zero point
    # -0.5 -> ties to even), exact .5 ties of x * scale, a lone huge outlier, denormal-small values
    k, n = 128, 12
    rng = np.random.default_rng(3)
    rows = [np.zeros(k), np.full(k, 0.75), np.abs(rng.standard_normal(k)), -np.abs(rng.standard_normal(k)),
            np.where(np.arange(k) % 2 == 0, 1.5, -1.5), np.linspace(-1.0, 1.0, k) * 127.5 / 255.0,
            np.concatenate([[1000.0], rng.standard_normal(k - 1) * 1e-3]), rng.standard_normal(k) * 1e-30,
            np.concatenate([[0.0, 255.0], np.arange(k - 2) + 0.5])]
    x = np.stack(rows).astype(np.float32)
    w = make_weights(n, k, seed=11)
    w[0, :32] = 0.0                       # a zero block: scale -0.0, nibbles 8
    w[1, 32:64] = 0.3                     # a constant block: every q = -8
    u4, sc = orc.quant_rhs(w)
    bias = np.linspace(-1.0, 1.0, n).astype(np.float32)
    assert np.array_equal(orc.linear(x, u4, sc, bias=bias), torch_dyn_quant_linear(x, u4, sc, bias))
    assert np.array_equal(orc.linear(x, u4, sc), torch_dyn_quant_linear(x, u4, sc, None))


@needs_torch_dynq
def test_reference_test_protocol_equals_torch_dyn_quant_matmul(orc):
    # the reference's own test case (KaiLinearTest.hpp:391-427: M=1, K=N=1024, uniform[-1,1] from
    # srand(4568) / srand(4572), no bias), which it compares with the Arm kernel to 1e-4
    lhs = orc.fill_uniform_random(1, 1024, 4568)
    rhs = orc.fill_uniform_random(1024, 1024, 4572)
    u4, sc = orc.quant_rhs(rhs)
    assert np.array_equal(orc.linear(lhs, u4, sc), torch_dyn_quant_linear(lhs, u4, sc, None))


@needs_torch_dynq
def test_oracle_equals_torch_dyn_quant_matmul_on_many_small_cases(orc):
    # 120 seeded cases: shapes with K = 32..416 (every multiple of 32), N = 1..24, M = 1..6; rows drawn from
    # normal, uniform, heavy-tailed and sparse distributions at scales 1e-6..1e4; weights likewise
    rng = np.random.default_rng(2026)
    for case in range(120):
        k = 32 * int(rng.integers(1, 14))
        n, m = int(rng.integers(1, 25)), int(rng.integers(1, 7))
        kind = case % 4
        if kind == 0:
            x = rng.standard_normal((m, k))
        elif kind == 1:
            x = rng.uniform(-1.0, 1.0, (m, k))
        elif kind == 2:
            x = rng.standard_cauchy((m, k))
        else:
            x = rng.standard_normal((m, k)) * (rng.uniform(0, 1, (m, k)) < 0.1)
        x = (x * 10.0 ** rng.uniform(-6, 4, (m, 1))).astype(np.float32)
        w = (rng.standard_normal((n, k)) * 10.0 ** rng.uniform(-4, 1, (n, 1))).astype(np.float32)
        if case % 5 == 0:
            w[:, :32] = 0.0
        bias = rng.standard_normal(n).astype(np.float32) if case % 2 else None
        u4, sc = orc.quant_rhs(w)
        got = orc.linear(x, u4, sc, bias=bias)
        want = torch_dyn_quant_linear(x, u4, sc, bias)
        assert np.array_equal(got, want), (case, m, k, n, kind)


# ---- the AVX-512 VNNI form of the product (benchmark's CPU-baseline leg) ----
@pytest.mark.parametrize("m,k,n,bias,threads", [
    (1, 32, 5, False, 1),        # one block: the masked tail group alone
    (3, 96, 17, True, 2),        # three blocks: one partial group of four
    (2, 160, 33, True, 3),       # a whole group and a one-block tail
    (1, 1536, 256, True, 4),     # k/v_proj
    (4, 1280, 64, False, 1),     # ViT width (40 blocks)
    (1, 8960, 48, False, 2),     # down_proj's K
])
def test_vnni_product_is_bit_identical_to_the_scalar_one(orc, m, k, n, bias, threads):
    if not orc.has_vnni():
        pytest.skip("CPU without AVX-512 VNNI")
    rng = np.random.default_rng(1000 + k + n)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    w[0, :32] = 0.0                                   # an all-zero block (scale 0, every u4 = 8)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[0, ::7] *= 20.0                                 # outliers: a wide range, large |zero point|
    if m > 1:
        x[1] = np.abs(x[1])                           # one-sided row: offset at the end of its range
    b = (rng.standard_normal(n) * 0.1).astype(np.float32) if bias else None
    u4, sc = orc.quant_rhs(w)
    ref = orc.linear(x, u4, sc, bias=b, threads=1)
    got = orc.linear_vnni(x, u4, sc, bias=b, threads=threads)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))
