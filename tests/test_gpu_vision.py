"""GPU: the vision patch embedding (Conv3D without padding, stride = kernel) as im2col + the W4A32
Linear, the way the reference's ArmConv3DOp::forward does it (Conv3DOp.cpp:48-188)."""
import numpy as np
import pytest
import torch

from conftest import max_abs_rel

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def im2col_ref(a, kernel, stride):
    """numpy restatement of im2col_conv3d_p0_d1_activation_fp32 (conv3d.cpp:15-78)."""
    B, C, T, H, W = a.shape
    (kt, kh, kw), (st, sh, sw) = kernel, stride
    OT, OH, OW = (T - kt) // st + 1, (H - kh) // sh + 1, (W - kw) // sw + 1
    z = np.empty((B * OT * OH * OW, C * kt * kh * kw), dtype=a.dtype)
    r = 0
    for b in range(B):
        for ot in range(OT):
            for oh in range(OH):
                for ow in range(OW):
                    patch = a[b, :, ot * st:ot * st + kt, oh * sh:oh * sh + kh, ow * sw:ow * sw + kw]
                    z[r] = patch.reshape(-1)
                    r += 1
    return z


@pytest.mark.parametrize("shape,kernel,stride", [
    ((1, 3, 2, 56, 56), (2, 14, 14), (2, 14, 14)),      # Qwen2-VL patch embed geometry, small image
    ((2, 3, 4, 28, 42), (2, 14, 14), (2, 14, 14)),
    ((1, 2, 3, 9, 10), (2, 3, 4), (1, 2, 3)),           # overlapping windows
])
def test_im2col_is_exact_and_zero_padded(pkg, shape, kernel, stride):
    rng = np.random.default_rng(0)
    a = rng.standard_normal(shape).astype(np.float32)
    ref = im2col_ref(a, kernel, stride)
    got = pkg.op_im2col_conv3d(dev(a), kernel, stride).cpu().numpy()
    cols = ref.shape[1]
    assert got.shape == (ref.shape[0], (cols + 31) // 32 * 32)
    assert np.array_equal(got[:, :cols], ref)
    assert not got[:, cols:].any()
    # torch's unfold-free check of the column order: a conv3d with a one-hot filter picks one column
    w = np.zeros((1,) + (shape[1],) + kernel, dtype=np.float32)
    w.reshape(-1)[cols // 3] = 1.0
    conv = torch.nn.functional.conv3d(torch.from_numpy(a), torch.from_numpy(w), stride=stride)
    assert np.array_equal(conv.permute(0, 2, 3, 4, 1).reshape(-1).numpy(), ref[:, cols // 3])


def test_patch_embed_conv3d_as_w4a32_linear(pkg, orc):
    """out_channels x (3*2*14*14 = 1176) filters: K is padded to 1184 with zeros on both operands, which
    leaves every row's quantisation range and every sum unchanged: the HIP product must match the oracle on
    the same padded operands, the padding must not disturb the quantised weights, and the result must stay
    close to the f32 convolution."""
    rng = np.random.default_rng(1)
    B, C, T, H, W, OC = 1, 3, 2, 112, 112, 1280
    kernel = stride = (2, 14, 14)
    a = rng.standard_normal((B, C, T, H, W)).astype(np.float32)
    w = (rng.standard_normal((OC, C) + kernel) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(OC) * 0.02).astype(np.float32)
    K = C * 2 * 14 * 14
    Kp = (K + 31) // 32 * 32
    wp = np.zeros((OC, Kp), dtype=np.float32)
    wp[:, :K] = w.reshape(OC, K)

    cols = pkg.op_im2col_conv3d(dev(a), kernel, stride)                 # [64][1184]
    packed = pkg.quant_pack_rhs(dev(wp), dev(bias))
    y = pkg.matmul(cols, packed, OC).cpu().numpy()                      # [b,ot,oh,ow][oc]

    zp = np.zeros((cols.shape[0], Kp), dtype=np.float32)
    zp[:, :K] = im2col_ref(a, kernel, stride)
    u4, sc = orc.quant_rhs(wp)
    ref = orc.linear(zp, u4, sc, bias=bias)
    assert max_abs_rel(y, ref) <= 2e-3
    # the zero padding is invisible: the last (partial) block of every weight row quantises as if the
    # row ended at K (its scale comes from the real values), and the activation rows keep their range
    u4_np, sc_np = orc.quant_rhs(np.ascontiguousarray(wp[:, :K - K % 32]))
    assert np.array_equal(u4[:, :(K - K % 32) // 2], u4_np)
    # against the f32 convolution: 4-bit weights and 8-bit activations, a few percent at most
    conv = torch.nn.functional.conv3d(torch.from_numpy(a), torch.from_numpy(w), torch.from_numpy(bias),
                                      stride=stride).permute(0, 2, 3, 4, 1).reshape(-1, OC).numpy()
    assert max_abs_rel(y, conv) < 0.1


def test_patch_embed_at_the_configuration_s_image_size(pkg, orc):
    """One 448 x 448 image (two frames), 14 x 14 patches: 1024 rows of K = 1176 (padded to 1184) through the
    1280 filters, as configuration 5 names it. The product against the oracle on sampled rows."""
    rng = np.random.default_rng(2)
    B, C, T, H, W, OC = 1, 3, 2, 448, 448, 1280
    kernel = stride = (2, 14, 14)
    a = rng.standard_normal((B, C, T, H, W)).astype(np.float32)
    w = (rng.standard_normal((OC, C) + kernel) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(OC) * 0.02).astype(np.float32)
    K = C * 2 * 14 * 14
    Kp = (K + 31) // 32 * 32
    wp = np.zeros((OC, Kp), dtype=np.float32)
    wp[:, :K] = w.reshape(OC, K)
    cols = pkg.op_im2col_conv3d(dev(a), kernel, stride)
    assert tuple(cols.shape) == (1024, Kp)
    y = pkg.matmul(cols, pkg.quant_pack_rhs(dev(wp), dev(bias)), OC).cpu().numpy()
    assert y.shape == (1024, OC) and np.isfinite(y).all()
    rows = np.unique(np.concatenate([np.arange(0, 1024, 41), [1023]]))
    ref_cols = im2col_ref(a, kernel, stride)
    assert np.array_equal(cols.cpu().numpy()[:, :K], ref_cols) and not cols.cpu().numpy()[:, K:].any()
    zp = np.zeros((len(rows), Kp), dtype=np.float32)
    zp[:, :K] = ref_cols[rows]
    u4, sc = orc.quant_rhs(wp)
    assert max_abs_rel(y[rows], orc.linear(zp, u4, sc, bias=bias, threads=8)) <= 2e-3
