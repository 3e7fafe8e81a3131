"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same inputs.

Integer/byte results (weight nibbles, bf16 scales, int8 activations, zero points, the
repacked blob's round trip, dequantised weights) must be bit-exact. f32 outputs must be
within max|y - ref| / max|ref| <= 1e-3 for the decode kernels (M <= 8) and <= 2e-3 for the
prefill kernels, the tolerances the target states; since the block sums are exact integers
on both sides the observed error is near 1e-6, and the tests also hold it to 2e-5.
"""
import numpy as np
import pytest
import torch

from conftest import make_acts, make_weights, max_abs_rel

pytestmark = pytest.mark.gpu

GEMV_TOL = 1e-3
GEMM_TOL = 2e-3
TIGHT = 2e-5

# (name, K, N, has_bias) - the Qwen2-1.5B linears, lm_head, and the Qwen2-VL ViT linears
DECODER_SHAPES = [
    ("q_proj", 1536, 1536, True),
    ("kv_proj", 1536, 256, True),
    ("o_proj", 1536, 1536, False),
    ("gate_up", 1536, 8960, False),
    ("down", 8960, 1536, False),
]
LM_HEAD = ("lm_head", 1536, 151936, False)
VIT_SHAPES = [
    ("vit_qkv", 1280, 3840, True),
    ("vit_proj", 1280, 1280, True),
    ("vit_fc1", 1280, 5120, True),
    ("vit_fc2", 5120, 1280, True),
]
# the Qwen2-VL patch merger: four patches' 1280 features side by side -> 5120 -> 1536, both with bias
# (mllm/Models/qwen2vl/modeling_qwen2vl.hpp:112-137); 1024 patches give 256 rows
MERGER_SHAPES = [
    ("merger_fc1", 5120, 5120, True),
    ("merger_fc2", 5120, 1536, True),
]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def bias_for(n, has_bias, seed=2):
    if not has_bias:
        return None
    return (np.random.default_rng(seed).standard_normal(n) * 0.02).astype(np.float32)


# ------------------------------------------------------------------- weights (offline)

SPECIAL_W = "special"


def special_weights():
    """Blocks that exercise the quantizer's corner rules."""
    w = make_weights(32, 256, seed=13)
    w[0, :32] = 0.0                       # zero block -> scale -0.0, bytes 0x88
    w[1, :32] = 0.5                       # constant block -> all -8
    w[2, :32] = 0.0
    w[2, 3], w[2, 7] = 2.0, -2.0          # tie: the first maximum wins, q[7] clamps to 7
    w[3, :32] = 0.0
    w[3, 0] = -1.0                        # scale 2^-3; exact .5 ties round away from zero
    w[3, 1:8] = np.array([0.5, 1.5, 2.5, -0.5, -2.5, 6.5, 7.5], np.float32) * 0.125
    w[4, 32:64] = -w[5, 32:64]            # negated block: same nibbles, flipped scale
    return w


@pytest.mark.parametrize("n,k,seed", [(32, 256, SPECIAL_W), (64, 128, 0), (1536, 1536, 1),
                                      (256, 8960, 2), (50, 96, 3)])
@pytest.mark.parametrize("mode", [0, 1])
def test_quant_rhs_bit_exact(pkg, orc, n, k, seed, mode):
    w = special_weights() if seed == SPECIAL_W else make_weights(n, k, seed=seed)
    u4_ref, sc_ref = orc.quant_rhs(w, bf16_rne_mode=bool(mode))
    u4, sc = pkg.quant_rhs_native(dev(w), bf16_mode=mode)
    assert np.array_equal(host(u4), u4_ref)
    assert np.array_equal(host(sc).view(np.uint16), sc_ref)


@pytest.mark.parametrize("n,k", [(16, 128), (50, 96), (1536, 1536), (256, 8960), (3, 32)])
def test_repack_round_trip_and_dequant_bit_exact(pkg, orc, n, k):
    rng = np.random.default_rng(n * 7 + k)
    u4 = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)           # any byte pattern
    sc = (rng.standard_normal((n, k // 32)).astype(np.float32) * 0.01).view(np.uint32) >> 16
    sc = sc.astype(np.uint16)
    bias = rng.standard_normal(n).astype(np.float32)
    packed = pkg.repack_native(dev(u4), dev(sc.view(np.int16)), dev(bias), n, k)
    assert packed.numel() == pkg.packed_bytes(n, k)
    u4_b, sc_b, bias_b = pkg.unpack_native(packed, n, k)
    assert np.array_equal(host(u4_b), u4)
    assert np.array_equal(host(sc_b).view(np.uint16), sc)
    assert np.array_equal(host(bias_b), bias)
    deq = host(pkg.dequant(packed, n, k))
    assert np.array_equal(deq.view(np.uint32), orc.dequant(u4, sc, k).view(np.uint32))


def test_quant_pack_equals_two_steps(pkg, orc):
    w = make_weights(48, 256, seed=4)
    b = bias_for(48, True)
    one = pkg.quant_pack_rhs(dev(w), dev(b))
    u4, sc = pkg.quant_rhs_native(dev(w))
    two = pkg.repack_native(u4, sc, dev(b), 48, 256)
    assert torch.equal(one, two)
    u4_ref, sc_ref = orc.quant_rhs(w)
    deq = host(pkg.dequant(one, 48, 256))
    assert np.array_equal(deq.view(np.uint32), orc.dequant(u4_ref, sc_ref, 256).view(np.uint32))


# ------------------------------------------------------------ activations (every forward)

def special_acts(k):
    x = make_acts(12, k, seed=5)
    x[0] = 0.0                                   # zero row: scale 1, zp 127
    x[1] = 0.0
    x[1, 5] = 4.0                                # one-sided positive: zp -128
    x[2] = 0.0
    x[2, 9] = -4.0                               # one-sided negative: zp 127
    x[3] = 0.0
    x[3, 0], x[3, 1] = 2.0, -2.0                 # symmetric: zp -0.5 -> nearest even -> 0
    x[4] = 0.0
    x[4, :6] = [-100.0, 155.0, 0.5, 1.5, -0.5, -2.5]   # scale 1: .5 ties round away from zero
    x[5] *= 20.0                                 # outlier row
    x[6] = np.abs(x[6])                          # all positive
    x[7] = -np.abs(x[7])                         # all negative
    x[8] *= 1e-6                                 # tiny
    x[9] *= 1e6                                  # huge
    return x


@pytest.mark.parametrize("m,k,seed", [(12, 1536, "special"), (12, 32, "special"), (1, 1536, 1),
                                      (8, 8960, 2), (64, 1280, 3), (300, 5120, 4)])
def test_quant_lhs_bit_exact(pkg, orc, m, k, seed):
    x = special_acts(k) if seed == "special" else make_acts(m, k, seed=seed, outlier_frac=0.05)
    aq_ref, recip_ref, negzp_ref, _ = orc.quant_lhs(x)
    ws = pkg.quant_lhs(dev(x))
    aq, recip, negzp = pkg.export_lhs(ws, x.shape[0], k)
    assert np.array_equal(host(negzp), negzp_ref)
    assert np.array_equal(host(recip).view(np.uint32), recip_ref.view(np.uint32))
    assert np.array_equal(host(aq), aq_ref)


# ------------------------------------------------------------------------- products

def run_linear(pkg, orc, m, k, n, has_bias, wseed=0, xseed=1, outliers=0.0, threads=8, rows=None):
    w = make_weights(n, k, seed=wseed)
    x = make_acts(m, k, seed=xseed, outlier_frac=outliers)
    bias = bias_for(n, has_bias)
    u4, sc = orc.quant_rhs(w)
    packed = pkg.repack_native(dev(u4), dev(sc.view(np.int16)), None if bias is None else dev(bias),
                               n, k)
    y = host(pkg.matmul(dev(x), packed, n))
    if rows is None:
        ref = orc.linear(x, u4, sc, bias=bias, threads=threads)
        return y, ref
    ref = orc.linear(x[rows], u4, sc, bias=bias, threads=threads)   # rows are independent
    return y[rows], ref


@pytest.mark.parametrize("name,k,n,has_bias", DECODER_SHAPES + VIT_SHAPES)
@pytest.mark.parametrize("m", [1, 4, 8])
def test_gemv_matches_oracle(pkg, orc, name, k, n, has_bias, m):
    y, ref = run_linear(pkg, orc, m, k, n, has_bias)
    err = max_abs_rel(y, ref)
    assert err <= GEMV_TOL and err <= TIGHT, (name, m, err)


@pytest.mark.parametrize("m", [2, 3, 5, 6, 7])
def test_gemv_every_m(pkg, orc, m):
    y, ref = run_linear(pkg, orc, m, 1536, 256, True, outliers=0.3)
    assert max_abs_rel(y, ref) <= TIGHT


@pytest.mark.parametrize("m,k,n", [(1, 1536, 8960), (8, 1536, 256), (1, 8960, 1536), (3, 5120, 1280),
                                   (2, 64, 40), (8, 32, 16)])
def test_fused_decode_kernel_equals_two_step_path(pkg, orc, m, k, n):
    # w4a32_matmul quantises inside the decode kernel when M*K is small; the two-step path
    # (w4a32_quant_lhs, then the GEMV on the workspace) must give the same bits, and the
    # quantised rows it exports must be the oracle's
    w = make_weights(n, k, seed=k + n)
    x = make_acts(m, k, seed=m, outlier_frac=0.3)
    bias = bias_for(n, True)
    packed = pkg.quant_pack_rhs(dev(w), dev(bias))
    xd = dev(x)
    fused = host(pkg.matmul(xd, packed, n))
    ws = pkg.quant_lhs(xd)
    two_step = host(pkg.matmul_quantized(ws, packed, m, k, n, kernel=pkg.KERNEL_GEMV))
    assert np.array_equal(fused, two_step)
    u4, sc = orc.quant_rhs(w)
    assert max_abs_rel(fused, orc.linear(x, u4, sc, bias=bias, threads=4)) <= TIGHT


@pytest.mark.parametrize("m,k,ns", [(1, 1536, [1536, 256, 256]), (8, 1536, [1536, 256, 256]),
                                    (1, 1536, [8960, 8960]), (4, 1536, [8960, 8960]), (8, 1536, [8960, 8960]),
                                    # two Linears of equal N: one workgroup per tile row of both (M <= 8)
                                    (3, 256, [48, 48]), (2, 64, [40, 40]), (5, 1280, [1280, 1280]),
                                    (1, 8960, [1536, 1536]),
                                    (1, 8960, [1536]), (4, 8960, [1536, 50]), (12, 256, [64, 48, 16, 100]),
                                    (2, 64, [40, 16]), (40, 256, [64, 48, 16, 100]),
                                    (130, 96, [50, 16]), (300, 1536, [1536, 256, 256]),
                                    (512, 1536, [8960, 8960]), (1024, 1280, [1280, 1280, 1280])])
def test_grouped_linears_equal_separate_calls(pkg, m, k, ns):
    # q/k/v and gate/up take the same rows: one grouped call must give, bit for bit, what one
    # w4a32_matmul per Linear gives (covers the one-launch decode path, the quantise-once fallback
    # and, from M = 33 on, the prefill kernel's one launch over all the Linears)
    x = dev(make_acts(m, k, seed=7, outlier_frac=0.25))
    packed = [pkg.quant_pack_rhs(dev(make_weights(n, k, seed=10 + i)), dev(bias_for(n, True, seed=i)))
              for i, n in enumerate(ns)]
    grouped = pkg.matmul_grouped(x, packed, ns)
    for p, n, yg in zip(packed, ns, grouped):
        assert np.array_equal(host(yg), host(pkg.matmul(x, p, n)))


@pytest.mark.parametrize("m", [1, 4, 8])
def test_gemv_lm_head(pkg, orc, m):
    name, k, n, has_bias = LM_HEAD
    y, ref = run_linear(pkg, orc, m, k, n, has_bias)
    err = max_abs_rel(y, ref)
    assert err <= GEMV_TOL and err <= TIGHT, err


@pytest.mark.parametrize("m,k,n", [(1, 32, 16), (3, 64, 5), (8, 96, 50), (1, 1024, 1024),
                                   # several rows on a short K: a workgroup takes many tile rows
                                   (8, 256, 512), (7, 384, 256), (5, 128, 300), (8, 96, 400), (6, 32, 1000),
                                   (4, 4096, 100), (8, 3072, 48), (3, 2048, 33)])
def test_gemv_ragged_shapes(pkg, orc, m, k, n):
    # N not a multiple of 16, K not a multiple of 128: padding inside the tiles must be inert
    y, ref = run_linear(pkg, orc, m, k, n, True, wseed=m + k, xseed=n)
    assert max_abs_rel(y, ref) <= TIGHT


def exact_case(m, n, k, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(-100, 156, size=(m, k)).astype(np.float32)
    x[:, 0], x[:, 1] = -100.0, 155.0
    q = rng.integers(-8, 8, size=(n, k)).astype(np.int64)
    e = rng.integers(-7, -1, size=(n, k // 32))
    for r in range(n):
        for b in range(k // 32):
            q[r, 32 * b + int(rng.integers(0, 32))] = -8
    return x, (q * np.exp2(np.repeat(e, 32, axis=1))).astype(np.float32)


@pytest.mark.parametrize("m,n,k", [(1, 48, 256), (8, 33, 512), (40, 64, 256), (130, 20, 128)])
def test_lossless_inputs_give_the_exact_dense_product(pkg, m, n, k):
    # Inputs both quantizers represent exactly, with every partial sum below 2^24: the op
    # must equal a float64 matmul bit for bit. Fails on any wrong index, sign, nibble order,
    # scale pairing or operand layout, independently of the oracle.
    x, w = exact_case(m, n, k, seed=m + n)
    packed = pkg.quant_pack_rhs(dev(w))
    y = host(pkg.matmul(dev(x), packed, n)).astype(np.float64)
    assert np.array_equal(y, x.astype(np.float64) @ w.astype(np.float64).T)


@pytest.mark.parametrize("name,k,n,has_bias", DECODER_SHAPES)
@pytest.mark.parametrize("m", [128, 512])
def test_gemm_matches_oracle(pkg, orc, name, k, n, has_bias, m):
    # 1 % of rows scaled x20 stresses the per-row activation scales
    rows = None if m * n * k <= 2 ** 31 else np.unique(
        np.concatenate([np.arange(0, m, 37), [m - 1]]))
    y, ref = run_linear(pkg, orc, m, k, n, has_bias, outliers=0.01, rows=rows)
    err = max_abs_rel(y, ref)
    assert err <= GEMM_TOL and err <= TIGHT, (name, m, err)


@pytest.mark.parametrize("name,k,n,has_bias", DECODER_SHAPES + VIT_SHAPES)
def test_gemm_large_m_on_sampled_rows(pkg, orc, name, k, n, has_bias):
    # M = 2048 (ViT: 1024): rows are independent, so the oracle checks a sample of them
    m = 1024 if name.startswith("vit") else 2048
    rows = np.unique(np.concatenate([np.arange(0, m, 101), [m - 1, m - 2, 63, 64, 65]]))
    y, ref = run_linear(pkg, orc, m, k, n, has_bias, outliers=0.01, rows=rows)
    err = max_abs_rel(y, ref)
    assert err <= GEMM_TOL and err <= TIGHT, (name, err)


@pytest.mark.parametrize("name,k,n,has_bias", MERGER_SHAPES)
@pytest.mark.parametrize("m", [1, 256, 1024])
def test_merger_linears_match_oracle(pkg, orc, name, k, n, has_bias, m):
    # M = 256 is the image of the vision config (1024 patches merged four to one); 1 and 1024 bracket it
    rows = None if m == 1 else np.unique(np.concatenate([np.arange(0, m, 29), [m - 1, 31, 32, 33]]))
    y, ref = run_linear(pkg, orc, m, k, n, has_bias, outliers=0.0 if m == 1 else 0.01, rows=rows)
    err = max_abs_rel(y, ref)
    assert err <= (GEMV_TOL if m <= 8 else GEMM_TOL) and err <= TIGHT, (name, m, err)


@pytest.mark.parametrize("m", [9, 15, 16, 17, 32, 33, 63, 65, 100, 129, 257, 300])
def test_gemm_ragged_m(pkg, orc, m):
    y, ref = run_linear(pkg, orc, m, 256, 50, True, outliers=0.1)
    assert max_abs_rel(y, ref) <= TIGHT


@pytest.mark.parametrize("kernel", ["i8", "f16"] + [f"f16:{i}" for i in range(10)])
@pytest.mark.parametrize("m,k,n", [(9, 32, 16), (40, 96, 50), (200, 160, 330), (128, 1536, 256),
                                   (300, 1280, 3840), (512, 8960, 1536), (1024, 5120, 1280),
                                   # a last 64-k stage that is half empty, behind whole and behind
                                   # ragged unrolled iterations of the main loop
                                   (70, 1760, 80), (150, 1632, 200)])
def test_gemm_each_kernel_matches_oracle(pkg, orc, kernel, m, k, n):
    # both prefill kernels (and each tile shape of the f16 one) on the same inputs; K = 32, 96 and 160
    # leave padding inside a stage (an odd number of 32-k blocks: the second k-half of the last stage
    # is all padding); N = 330 ends inside a 160- and a 128-column tile
    w = make_weights(n, k, seed=k)
    x = make_acts(m, k, seed=m, outlier_frac=0.02)
    bias = bias_for(n, True)
    u4, sc = orc.quant_rhs(w)
    packed = pkg.repack_native(dev(u4), dev(sc.view(np.int16)), dev(bias), n, k)
    ws = pkg.quant_lhs(dev(x))
    if kernel == "i8":
        sel = pkg.KERNEL_GEMM_I8
    elif kernel == "f16":
        sel = pkg.KERNEL_GEMM_F16
    else:  # every tile shape of the f16 kernel, whatever the size-based choice would be
        sel = pkg.KERNEL_GEMM_F16_TILE0 + int(kernel.split(":")[1])
    y = host(pkg.matmul_quantized(ws, packed, m, k, n, kernel=sel))
    rows = np.unique(np.concatenate([np.arange(0, m, 41), [m - 1]]))
    ref = orc.linear(x[rows], u4, sc, bias=bias, threads=8)
    err = max_abs_rel(y[rows], ref)
    assert err <= GEMM_TOL and err <= TIGHT, (kernel, err)


@pytest.mark.parametrize("m,k,n", [(512, 8960, 1536), (100, 8960, 50), (16, 8960, 1536), (300, 6144, 272),
                                   (1024, 8960, 1536),
                                   (1100, 6144, 1536), (64, 256, 64), (64, 6208, 96)])
def test_splitk_matches_oracle_and_plain(pkg, orc, m, k, n):
    # few tiles and a long K: the k range of a tile is dealt to several workgroups and the parts are
    # added by a second kernel; K = 256 is one the library does not split (falls through); K = 6208 is an
    # odd number of stages (the ranges are whole pairs of stages, the last one ends on the odd stage)
    w = make_weights(n, k, seed=n)
    x = make_acts(m, k, seed=m, outlier_frac=0.02)
    bias = bias_for(n, True)
    u4, sc = orc.quant_rhs(w)
    packed = pkg.repack_native(dev(u4), dev(sc.view(np.int16)), dev(bias), n, k)
    ws = pkg.quant_lhs(dev(x))
    split = int(pkg.lib().w4a32_splitk_scratch_bytes(m, k, n)) > 0
    assert split == (k >= 6144)
    y = host(pkg.matmul_quantized_splitk(ws, packed, m, k, n))
    plain = host(pkg.matmul_quantized(ws, packed, m, k, n))
    rows = np.unique(np.concatenate([np.arange(0, m, 37), [m - 1]]))
    ref = orc.linear(x[rows], u4, sc, bias=bias, threads=8)
    assert max_abs_rel(y[rows], ref) <= TIGHT
    assert max_abs_rel(y, plain) <= 1e-6          # same products, another f32 summation order
    if not split:
        assert np.array_equal(y, plain)
    # too little scratch: the plain kernel runs
    import torch
    tiny = torch.empty((16,), dtype=torch.uint8, device="cuda")
    assert np.array_equal(host(pkg.matmul_quantized_splitk(ws, packed, m, k, n, scratch=tiny)), plain)


@pytest.mark.parametrize("m,k,n", [(512, 8960, 1536), (128, 8960, 1536), (100, 8960, 50), (64, 256, 64), (4, 8960, 1536)])
def test_whole_op_with_a_sized_workspace_takes_the_split_form_itself(pkg, orc, m, k, n):
    # w4a32_matmul_ws: one call per Linear; with room for the partial sums behind the activation workspace the
    # library deals a long k range to several workgroups itself, with the plain workspace it is w4a32_matmul
    import torch
    w = make_weights(n, k, seed=n + 3)
    x = make_acts(m, k, seed=m + 1, outlier_frac=0.02)
    bias = bias_for(n, True)
    u4, sc = orc.quant_rhs(w)
    packed = pkg.repack_native(dev(u4), dev(sc.view(np.int16)), dev(bias), n, k)
    xd = dev(x)
    L = pkg.lib()
    small, large = int(L.w4a32_workspace_bytes(m, k)), int(L.w4a32_workspace_bytes_n(m, k, n))
    scratch = int(L.w4a32_splitk_scratch_bytes(m, k, n))
    assert large == (small + 255) // 256 * 256 + scratch and (scratch > 0) == (m > 8 and k >= 6144)
    y = host(pkg.matmul_ws(xd, packed, n))
    plain = host(pkg.matmul(xd, packed, n))
    rows = np.unique(np.concatenate([np.arange(0, m, 37), [m - 1]]))
    assert max_abs_rel(y[rows], orc.linear(x[rows], u4, sc, bias=bias, threads=8)) <= TIGHT
    if scratch:
        split = host(pkg.matmul_quantized_splitk(pkg.quant_lhs(xd), packed, m, k, n))
        assert np.array_equal(y, split) and max_abs_rel(y, plain) <= 1e-6
    else:
        assert np.array_equal(y, plain)
    # the plain workspace: w4a32_matmul, bit for bit; a shorter one is refused
    ws_small = torch.empty((small,), dtype=torch.uint8, device="cuda")
    assert np.array_equal(host(pkg.matmul_ws(xd, packed, n, ws=ws_small)), plain)
    with pytest.raises(pkg.W4A32Error):
        pkg.matmul_ws(xd, packed, n, ws=ws_small[: small - 256])


@pytest.mark.parametrize("m,k,n", [(9, 64, 48), (33, 64, 48), (130, 160, 100), (256, 1536, 8960), (512, 1536, 8960),
                                   (1100, 1280, 5120), (300, 4096, 2560)])
def test_silu_pair_matches_the_three_operators(pkg, orc, m, k, n):
    # gate Linear, up Linear, silu(gate) * up in one launch: against the separate operators of the library
    # (same products, same f32 expression) and against the oracle's two Linears; N = 48 and 100 end inside
    # a tile's half, K = 160 leaves padding in the last stage; the shapes cover the three tile choices
    wg, wu = make_weights(n, k, seed=n), make_weights(n, k, seed=n + 1)
    x = make_acts(m, k, seed=m, outlier_frac=0.02)
    bg, bu = bias_for(n, True, seed=3), bias_for(n, True, seed=4)
    (u4g, scg), (u4u, scu) = orc.quant_rhs(wg), orc.quant_rhs(wu)
    pg = pkg.repack_native(dev(u4g), dev(scg.view(np.int16)), dev(bg), n, k)
    pu = pkg.repack_native(dev(u4u), dev(scu.view(np.int16)), dev(bu), n, k)
    ws = pkg.quant_lhs(dev(x))
    got = host(pkg.matmul_quantized_silu_pair(ws, pg, pu, m, k, n))
    yg = pkg.matmul_quantized(ws, pg, m, k, n, kernel=pkg.KERNEL_GEMM_F16_TILE0 + 2)
    yu = pkg.matmul_quantized(ws, pu, m, k, n, kernel=pkg.KERNEL_GEMM_F16_TILE0 + 2)
    sep = host(pkg.op_silu_mul(yg, yu))
    assert np.array_equal(got, sep)
    rows = np.unique(np.concatenate([np.arange(0, m, 53), [m - 1]]))
    rg = orc.linear(x[rows], u4g, scg, bias=bg, threads=8).astype(np.float64)
    ru = orc.linear(x[rows], u4u, scu, bias=bu, threads=8).astype(np.float64)
    ref = (rg / (1.0 + np.exp(-rg)) * ru).astype(np.float32)
    assert max_abs_rel(got[rows], ref) <= TIGHT


@pytest.mark.skipif(not hasattr(torch.ops.aten, "_dyn_quant_matmul_4bit"),
                    reason="this torch build has no aten::_dyn_quant_matmul_4bit")
@pytest.mark.parametrize("m,k,n", [(1, 1536, 256), (8, 8960, 64), (64, 1536, 320), (300, 1280, 160)])
def test_hip_path_matches_torch_dyn_quant_matmul(pkg, orc, m, k, n):
    # the HIP op against PyTorch's own CPU routine for the same scheme (block 32, bf16 scales, dynamic
    # per-row int8 activations), without the oracle in between; weights quantised by the HIP quantiser
    w = make_weights(n, k, seed=n)
    x = make_acts(m, k, seed=m, outlier_frac=0.05)
    bias = bias_for(n, True)
    u4d, scd = pkg.quant_rhs_native(dev(w))
    packed = pkg.repack_native(u4d, scd, dev(bias), n, k)
    y = host(pkg.matmul(dev(x), packed, n))
    u4, sc = host(u4d), host(scd).view(np.uint16)
    tw = torch.from_numpy(u4)
    ts = torch.from_numpy(sc.view(np.int16)).view(torch.bfloat16)
    tp = torch.ops.aten._dyn_quant_pack_4bit_weight(tw, ts, torch.from_numpy(bias), 32, k, n)
    want = torch.ops.aten._dyn_quant_matmul_4bit(torch.from_numpy(x), tp, 32, k, n).numpy()
    assert max_abs_rel(y, want) <= TIGHT


def test_f16_kernel_with_wide_scale_range(pkg, orc):
    # rows whose block scales differ by many octaves, and rows that are tiny or huge overall:
    # the per-row power-of-two normalisation must keep the f16 operands exact
    n, k, m = 64, 256, 48
    rng = np.random.default_rng(8)
    w = make_weights(n, k, seed=8)
    for r in range(n):
        w[r] *= np.float32(2.0) ** rng.integers(-30, 30)
        for b in range(k // 32):
            w[r, 32 * b:32 * b + 32] *= np.float32(2.0) ** rng.integers(-12, 1)
    x = make_acts(m, k, seed=9)
    u4, sc = orc.quant_rhs(w)
    packed = pkg.repack_native(dev(u4), dev(sc.view(np.int16)), None, n, k)
    ws = pkg.quant_lhs(dev(x))
    y = host(pkg.matmul_quantized(ws, packed, m, k, n, kernel=pkg.KERNEL_GEMM_F16))
    ref = orc.linear(x, u4, sc, threads=4)
    # per output column (its own row of weights), relative to that column's largest output
    col_err = np.abs(y - ref).max(axis=0) / np.abs(ref).max(axis=0)
    assert col_err.max() <= TIGHT, col_err.max()


def test_gemm_rows_agree_with_gemv(pkg):
    # size-independent property at a full prefill size: each row of the M=512 product equals
    # the M=1 product of that row (different kernels, same integer block sums)
    k, n, m = 1536, 8960, 512
    w = make_weights(n, k, seed=0)
    x = dev(make_acts(m, k, seed=1, outlier_frac=0.01))
    packed = pkg.quant_pack_rhs(dev(w))
    big = pkg.matmul(x, packed, n)
    for r in (0, 5, 255, 511):
        one = pkg.matmul(x[r:r + 1].contiguous(), packed, n)
        assert max_abs_rel(host(one), host(big[r:r + 1])) <= TIGHT


def test_weight_row_permutation_permutes_outputs(pkg):
    k, n = 1536, 1536
    w = make_weights(n, k, seed=3)
    perm = np.random.default_rng(0).permutation(n)
    x = dev(make_acts(4, k, seed=2))
    y = host(pkg.matmul(x, pkg.quant_pack_rhs(dev(w)), n))
    yp = host(pkg.matmul(x, pkg.quant_pack_rhs(dev(w[perm])), n))
    assert np.array_equal(yp, y[:, perm])


def test_golden_fixture(pkg):
    g = np.load(__import__("os").path.join(__import__("os").path.dirname(__file__), "golden",
                                           "w4a32_small.npz"))
    packed = pkg.repack_native(dev(g["u4"]), dev(g["scales"].view(np.int16)), dev(g["bias"]),
                               int(g["n"]), int(g["k"]))
    ws = pkg.quant_lhs(dev(g["x"]))
    aq, recip, negzp = pkg.export_lhs(ws, int(g["m"]), int(g["k"]))
    assert np.array_equal(host(aq), g["aq"])
    assert np.array_equal(host(negzp), g["neg_zp"])
    assert np.array_equal(host(recip), g["recip"])
    u4, sc = pkg.quant_rhs_native(dev(g["w"]))
    assert np.array_equal(host(u4), g["u4"]) and np.array_equal(host(sc).view(np.uint16), g["scales"])
    y = host(pkg.matmul(dev(g["x"]), packed, int(g["n"])))
    assert max_abs_rel(y, g["y"]) <= TIGHT


def test_f16_kernel_forms_agree_with_the_integer_kernel_on_random_shapes(pkg):
    # The f16 kernel's main loop exists in three forms (advancing pointers while every load is in range,
    # clamped addresses, a last iteration that skips what lies past the end) and which stages run in which
    # depends on K, the tile shape and the split. gemm_i8_kernel shares none of that code and was checked
    # against the oracle above: 40 seeded shapes x (7 tile shapes, split-K, grouped, gate/up pair) against it.
    import random
    rnd = random.Random(1)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    L = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream
    ks = [32, 96, 160, 224, 288, 352, 480, 544, 736, 1056, 1568, 1632, 1760, 2080, 3104, 6176, 6208, 6240]
    for _ in range(40):
        k, m = rnd.choice(ks), rnd.choice([9, 31, 33, 100, 129, 300, 513])
        n = rnd.choice([16, 40, 100, 160, 330, 700])
        w1, w2 = (torch.randn((n, k), generator=gen, device="cuda") * 0.05 for _ in range(2))
        p1, p2 = pkg.quant_pack_rhs(w1), pkg.quant_pack_rhs(w2)
        ws = pkg.quant_lhs(torch.randn((m, k), generator=gen, device="cuda"))
        r1 = pkg.matmul_quantized(ws, p1, m, k, n, kernel=pkg.KERNEL_GEMM_I8)
        r2 = pkg.matmul_quantized(ws, p2, m, k, n, kernel=pkg.KERNEL_GEMM_I8)
        den = float(r1.abs().max())

        def close(y, r, what, tol=2e-6):
            err = float((y - r).abs().max()) / den
            assert err <= tol, (what, m, k, n, err)   # (a NaN fails the comparison too)

        y = torch.empty_like(r1)
        for t in range(pkg.GEMM_F16_TILES):
            y.fill_(float("nan"))
            assert L.w4a32_matmul_quantized_ex(y.data_ptr(), ws.data_ptr(), p1.data_ptr(), m, k, n,
                                               pkg.KERNEL_GEMM_F16_TILE0 + t, stream) == 0
            close(y, r1, f"tile {t}")
        close(pkg.matmul_quantized_splitk(ws, p1, m, k, n), r1, "split-K")
        for o, r in zip(pkg.matmul_quantized_grouped(ws, [p1, p2], [n, n], m, k), (r1, r2)):
            close(o, r, "grouped")
        act = pkg.matmul_quantized_silu_pair(ws, p1, p2, m, k, n)
        want = torch.nn.functional.silu(r1) * r2
        assert float((act - want).abs().max()) <= 1e-4 * float(want.abs().max()), ("pair", m, k, n)


def test_bad_arguments_return_error_codes(pkg):
    L = pkg.lib()
    x = torch.zeros((1, 48), device="cuda")
    assert L.w4a32_packed_bytes(16, 48) == 0                      # K % 32 != 0
    assert L.w4a32_quant_lhs(x.data_ptr(), 1, 48, 48, x.data_ptr(), None) == -2
    assert L.w4a32_quant_lhs(None, 1, 64, 64, x.data_ptr(), None) == -1
    assert L.w4a32_matmul_quantized(None, None, None, 1, 64, 16, None) == -1
    ws = torch.zeros(pkg.workspace_bytes(4, 64), dtype=torch.uint8, device="cuda")
    pk = torch.zeros(pkg.packed_bytes(16, 64), dtype=torch.uint8, device="cuda")
    y = torch.zeros((16, 16), device="cuda")
    args = (y.data_ptr(), ws.data_ptr(), pk.data_ptr())
    assert L.w4a32_matmul_quantized_ex(*args, 4, 64, 16, pkg.KERNEL_GEMM_F16, None) == -2
    assert L.w4a32_matmul_quantized_ex(*args, 16, 64, 16, pkg.KERNEL_GEMV, None) == -2
    assert L.w4a32_matmul_quantized_ex(*args, 4, 64, 16, 99, None) == -1
    # one past the last named tile shape of the f16 kernel
    assert L.w4a32_matmul_quantized_ex(*args, 16, 64, 16, pkg.KERNEL_GEMM_F16_TILE0 + pkg.GEMM_F16_TILES,
                                       None) == -1
    # the pair launch: decode row counts have no f16 activation copy; null and misaligned operands
    act = torch.zeros((16, 16), device="cuda")
    assert L.w4a32_matmul_quantized_silu_pair(act.data_ptr(), ws.data_ptr(), pk.data_ptr(), pk.data_ptr(),
                                              8, 64, 16, None) == -2
    assert L.w4a32_matmul_quantized_silu_pair(act.data_ptr(), ws.data_ptr(), None, pk.data_ptr(),
                                              16, 64, 16, None) == -1
    assert L.w4a32_matmul_quantized_silu_pair(act.data_ptr(), ws.data_ptr(), pk.data_ptr() + 4, pk.data_ptr(),
                                              16, 64, 16, None) == -1
    assert L.w4a32_matmul_quantized_silu_pair(act.data_ptr(), ws.data_ptr(), pk.data_ptr(), pk.data_ptr(),
                                              16, 48, 16, None) == -2
    # split-K: shapes the library does not split ask for no scratch
    assert L.w4a32_splitk_scratch_bytes(8, 8960, 1536) == 0
    assert L.w4a32_splitk_scratch_bytes(512, 1536, 1536) == 0
    assert L.w4a32_splitk_scratch_bytes(512, 8960, 1536) == 5 * 512 * 1536 * 4
    with pytest.raises(pkg.W4A32Error):
        pkg._check(-2, "probe")
