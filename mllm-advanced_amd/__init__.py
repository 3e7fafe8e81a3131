"""MI355X-native W4A32 quantized Linear: Python binding of the C ABI (include/w4a32_hip.h).

The product is libw4a32_hip.so (hand-written gfx950 kernels behind a C ABI) and the C++
operator layer in host/. This module is plumbing: it loads the library with ctypes and
passes torch tensors' device pointers through. There is no CPU fallback: if the library
is missing or a call fails, an exception is raised.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libw4a32_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")
HOST_DIR = os.path.join(_HERE, "host")

BLOCK_LEN = 32
GEMV_MAX_M = 8
BF16_TRUNC = 0
BF16_RNE = 1
KERNEL_AUTO, KERNEL_GEMV, KERNEL_GEMM_I8, KERNEL_GEMM_F16 = 0, 1, 2, 3
KERNEL_GEMM_F16_TILE0, GEMM_F16_TILES = 16, 10  # + i: the f16 kernel with tile shape i
DENSE_F32, DENSE_F16 = 1, 2  # element types of a dense (unquantised) operand

#: every symbol include/w4a32_hip.h declares, with (restype, argtypes)
_vp, _ci, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
ABI = {
    "w4a32_error_string": (ctypes.c_char_p, [_ci]),
    "w4a32_abi_version": (_ci, []),
    "w4a32_packed_bytes": (_sz, [_ci, _ci]),
    "w4a32_workspace_bytes": (_sz, [_ci, _ci]),
    "w4a32_native_u4_bytes": (_sz, [_ci, _ci]),
    "w4a32_native_scale_bytes": (_sz, [_ci, _ci]),
    "w4a32_quant_rhs_native": (_ci, [_vp, _ci, _ci, _vp, _vp, _ci, _vp]),
    "w4a32_repack_native": (_ci, [_vp, _vp, _vp, _ci, _ci, _vp, _vp]),
    "w4a32_quant_pack_rhs": (_ci, [_vp, _vp, _ci, _ci, _vp, _vp, _ci, _vp]),
    "w4a32_unpack_native": (_ci, [_vp, _ci, _ci, _vp, _vp, _vp, _vp]),
    "w4a32_dequant": (_ci, [_vp, _ci, _ci, _vp, _vp]),
    "w4a32_quant_lhs": (_ci, [_vp, _ci, _ci, _ci, _vp, _vp]),
    "w4a32_export_lhs": (_ci, [_vp, _ci, _ci, _vp, _vp, _vp, _vp]),
    "w4a32_matmul_quantized": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a32_matmul_quantized_ex": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp]),
    "w4a32_matmul_quantized_grouped": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a32_quant_lhs_norm": (_ci, [_vp, _vp, _vp, ctypes.c_float, _vp, _ci, _ci, _vp, _vp]),
    "w4a32_quant_lhs_silu_mul": (_ci, [_vp, _vp, _ci, _ci, _vp, _vp]),
    "w4a32_kai_blob_bytes": (_sz, [_ci, _ci, _ci]),
    "w4a32_unpack_kai": (_ci, [_vp, _ci, _ci, _ci, _ci, _ci, _vp, _vp, _vp, _vp]),
    "w4a32_splitk_scratch_bytes": (_sz, [_ci, _ci, _ci]),
    "w4a32_matmul_quantized_splitk": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a32_matmul_quantized_splitk_parts": (_ci, [_vp, _vp, _ci, _ci, _ci, _vp, _sz, _vp, _vp]),
    "w4a32_quant_lhs_norm_parts": (_ci, [_vp, _vp, _ci, _vp, _ci, _vp, ctypes.c_float, _vp, _ci, _ci, _vp, _vp]),
    "w4a32_matmul": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a32_matmul_grouped": (_ci, [_vp, _vp, _vp, _vp, _ci, _vp, _ci, _ci, _vp]),
    "w4a32_matmul_static_ws": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a32_workspace_bytes_n": (_sz, [_ci, _ci, _ci]),
    "w4a32_matmul_ws": (_ci, [_vp, _vp, _vp, _vp, _sz, _ci, _ci, _ci, _vp]),
    # include/w4a32_decoder.h
    "w4a32_op_embedding": (_ci, [_vp, _vp, _ci, _ci, _ci, _vp, _vp]),
    "w4a32_op_rmsnorm": (_ci, [_vp, _vp, _vp, _ci, _ci, ctypes.c_float, _vp, _vp, _vp]),
    "w4a32_op_add": (_ci, [_vp, _vp, _vp, _sz, _vp]),
    "w4a32_op_silu_mul": (_ci, [_vp, _vp, _vp, _sz, _vp]),
    "w4a32_op_rope_table": (_ci, [_vp, _vp, _ci, _ci, ctypes.c_float, _vp]),
    "w4a32_op_rope_kv": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _ci, _vp]),
    "w4a32_op_im2col_conv3d": (_ci, [_vp, _vp] + [_ci] * 12 + [_vp]),
    "w4a32_op_scratch_bytes": (_sz, [_ci]),
    "w4a32_op_scratch_init": (_ci, [_vp, _ci, _vp]),
    "w4a32_op_attention": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _ci, _vp, _vp]),
    "w4a32_matmul_quantized_silu_pair": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a32_op_attention_prefill_scratch_bytes": (_sz, [_ci, _ci]),
    "w4a32_op_attention_prefill": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _ci, _vp, _sz,
                                         _vp]),
    "w4a32_op_attention_prefill_bf16x3_scratch_bytes": (_sz, [_ci, _ci]),
    "w4a32_op_attention_prefill_bf16x3": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a32_op_rope_attention_prefill_bf16x3": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci,
                                                     _ci, _vp, _sz, _vp]),
    "w4a32_op_rope_attention_decode": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci,
                                             _vp, _ci, _vp, _vp]),
    "w4a32_op_rope_attention_decode_linear": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _vp, _ci, _ci,
                                                    _ci, _ci, _vp, _ci, _vp, _vp]),
    "w4a32_op_argmax": (_ci, [_vp, _ci, _vp, _vp, _vp, _vp]),
    "w4a32_op_silu": (_ci, [_vp, _vp, _sz, _vp]),
    "w4a32_op_mul": (_ci, [_vp, _vp, _vp, _sz, _vp]),
    "w4a32_op_rope": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp]),
    "w4a32_op_attention_bshd": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _vp]),
    "w4a32_op_matmul_f32_nt": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a32_op_matmul_nt": (_ci, [_vp, _vp, _ci, _vp, _ci, _ci, _ci, _vp]),
    "w4a32_op_f16_to_f32": (_ci, [_vp, _vp, _sz, _vp]),
    "w4a32_decode_linear": (_ci, [_vp, _vp]),
    "w4a32_decode_kparts": (_ci, [_ci, _ci]),
    "w4a32_decoder_state_bytes": (_sz, [_vp]),
    "w4a32_decoder_state_offset": (_sz, [_vp, _ci]),
    "w4a32_decoder_init": (_ci, [_vp, _vp, _vp]),
    "w4a32_decoder_prefill": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _vp, _vp]),
    "w4a32_decoder_step": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp]),
}


class DecodeLinearArgs(ctypes.Structure):
    """w4a32_decode_linear_args"""
    _fields_ = [("d_x", ctypes.c_void_p), ("d_delta", ctypes.c_void_p), ("d_sum_out", ctypes.c_void_p),
                ("d_norm_weight", ctypes.c_void_p), ("norm_eps", ctypes.c_float), ("K", ctypes.c_int),
                ("count", ctypes.c_int), ("d_packed", ctypes.c_void_p * 4), ("N", ctypes.c_int * 4),
                ("d_y", ctypes.c_void_p * 4), ("silu_pair", ctypes.c_int), ("in_parts", ctypes.c_int),
                ("out_parts", ctypes.c_int)]


class DecoderConfig(ctypes.Structure):
    """w4a32_decoder_config"""
    _fields_ = [(n, ctypes.c_int) for n in ("hidden", "n_heads", "n_kv_heads", "head_dim", "intermediate",
                                            "n_layers", "vocab", "max_seq", "max_batch_tokens")] + \
               [("rope_theta", ctypes.c_float), ("rms_eps", ctypes.c_float)]


class LayerWeights(ctypes.Structure):
    """w4a32_layer_weights"""
    _fields_ = [(n, ctypes.c_void_p) for n in ("q", "k", "v", "o", "gate", "up", "down", "attn_norm",
                                               "ffn_norm")]


class DecoderWeights(ctypes.Structure):
    """w4a32_decoder_weights"""
    _fields_ = [("embedding", ctypes.c_void_p), ("final_norm", ctypes.c_void_p),
                ("lm_head", ctypes.c_void_p), ("layers", ctypes.POINTER(LayerWeights)),
                ("lm_head_dense", ctypes.c_void_p), ("lm_head_dense_dtype", ctypes.c_int)]


class W4A32Error(RuntimeError):
    pass


def build(force=True):
    """Compile the HIP library for gfx950 with hipcc (cross-compiles without a GPU)."""
    cmd = ["make", "-C", CSRC_DIR, "-j8"] + (["-B"] if force else [])
    subprocess.check_call(cmd)
    return LIB_PATH


_lib = None


def lib():
    """The loaded C-ABI library. Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise W4A32Error(
                f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; "
                "g.build()'). This package has no CPU or PyTorch fallback.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in ABI.items():
            fn = getattr(L, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _check(code, what):
    if code != 0:
        msg = lib().w4a32_error_string(code).decode()
        raise W4A32Error(f"{what} failed: {msg} (code {code})")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    import torch

    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def packed_bytes(N, K):
    return int(lib().w4a32_packed_bytes(N, K))


def workspace_bytes(M, K):
    return int(lib().w4a32_workspace_bytes(M, K))


def _dev_empty(nbytes, dtype=None):
    import torch

    return torch.empty(nbytes, dtype=dtype or torch.uint8, device="cuda")


def quant_rhs_native(w, bf16_mode=BF16_TRUNC):
    """f32 cuda tensor [N,K] -> (u4 uint8 [N,K/2], scales int16-view-of-bf16 [N,K/32])."""
    import torch

    N, K = w.shape
    assert w.is_cuda and w.dtype == torch.float32 and w.is_contiguous()
    u4 = torch.empty((N, K // 2), dtype=torch.uint8, device="cuda")
    sc = torch.empty((N, K // BLOCK_LEN), dtype=torch.int16, device="cuda")
    _check(lib().w4a32_quant_rhs_native(_ptr(w), N, K, _ptr(u4), _ptr(sc), bf16_mode, _stream()),
           "w4a32_quant_rhs_native")
    return u4, sc


def repack_native(u4, sc, bias, N, K):
    packed = _dev_empty(packed_bytes(N, K))
    _check(lib().w4a32_repack_native(_ptr(u4), _ptr(sc), _ptr(bias), N, K, _ptr(packed), _stream()),
           "w4a32_repack_native")
    return packed


def quant_pack_rhs(w, bias=None, bf16_mode=BF16_TRUNC):
    N, K = w.shape
    L = lib()
    packed = _dev_empty(packed_bytes(N, K))
    tmp = _dev_empty(int(L.w4a32_native_u4_bytes(N, K)) + int(L.w4a32_native_scale_bytes(N, K)))
    _check(L.w4a32_quant_pack_rhs(_ptr(w), _ptr(bias), N, K, _ptr(packed), _ptr(tmp), bf16_mode,
                                  _stream()), "w4a32_quant_pack_rhs")
    return packed


def unpack_native(packed, N, K, want_bias=True):
    import torch

    u4 = torch.empty((N, K // 2), dtype=torch.uint8, device="cuda")
    sc = torch.empty((N, K // BLOCK_LEN), dtype=torch.int16, device="cuda")
    bias = torch.empty((N,), dtype=torch.float32, device="cuda") if want_bias else None
    _check(lib().w4a32_unpack_native(_ptr(packed), N, K, _ptr(u4), _ptr(sc), _ptr(bias), _stream()),
           "w4a32_unpack_native")
    return u4, sc, bias


def dequant(packed, N, K):
    import torch

    out = torch.empty((N, K), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_dequant(_ptr(packed), N, K, _ptr(out), _stream()), "w4a32_dequant")
    return out


def quant_lhs(x, ws=None):
    M, K = x.shape
    if ws is None:
        ws = _dev_empty(workspace_bytes(M, K))
    _check(lib().w4a32_quant_lhs(_ptr(x), M, K, x.stride(0), _ptr(ws), _stream()), "w4a32_quant_lhs")
    return ws


def quant_lhs_norm(h, weight, eps, delta=None, ws=None):
    """Residual add + RMSNorm + row quantiser in one launch: returns (ws, h + delta or None)."""
    import torch

    M, K = h.shape
    if ws is None:
        ws = _dev_empty(workspace_bytes(M, K))
    h_out = torch.empty_like(h) if delta is not None else None
    _check(lib().w4a32_quant_lhs_norm(_ptr(h), _ptr(delta), _ptr(weight), eps, _ptr(h_out), M, K,
                                      _ptr(ws), _stream()), "w4a32_quant_lhs_norm")
    return ws, h_out


def quant_lhs_silu_mul(gate, up, ws=None):
    """silu(gate) * up + row quantiser in one launch."""
    M, K = gate.shape
    if ws is None:
        ws = _dev_empty(workspace_bytes(M, K))
    _check(lib().w4a32_quant_lhs_silu_mul(_ptr(gate), _ptr(up), M, K, _ptr(ws), _stream()),
           "w4a32_quant_lhs_silu_mul")
    return ws


def unpack_kai(blob, N, K, nr, kr, sr):
    """Blob of the reference's Arm quantizer (parity unpinned) -> native u4, bf16 scales, bias."""
    import torch

    u4 = torch.empty((N, K // 2), dtype=torch.uint8, device="cuda")
    scales = torch.empty((N, K // 32), dtype=torch.int16, device="cuda")
    bias = torch.empty((N,), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_unpack_kai(_ptr(blob), N, K, nr, kr, sr, _ptr(u4), _ptr(scales), _ptr(bias),
                                  _stream()), "w4a32_unpack_kai")
    return u4, scales, bias


def export_lhs(ws, M, K):
    import torch

    aq = torch.empty((M, K), dtype=torch.int8, device="cuda")
    recip = torch.empty((M,), dtype=torch.float32, device="cuda")
    neg_zp = torch.empty((M,), dtype=torch.int32, device="cuda")
    _check(lib().w4a32_export_lhs(_ptr(ws), M, K, _ptr(aq), _ptr(recip), _ptr(neg_zp), _stream()),
           "w4a32_export_lhs")
    return aq, recip, neg_zp


def matmul_quantized(ws, packed, M, K, N, out=None, kernel=KERNEL_AUTO):
    import torch

    y = out if out is not None else torch.empty((M, N), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_matmul_quantized_ex(_ptr(y), _ptr(ws), _ptr(packed), M, K, N, kernel,
                                           _stream()), "w4a32_matmul_quantized_ex")
    return y


def matmul_quantized_grouped(ws, packed_list, Ns, M, K, outs=None):
    """Several Linears on rows already quantised into ws (one launch at M > 8)."""
    import torch

    n = len(Ns)
    ys = outs if outs is not None else [torch.empty((M, N), dtype=torch.float32, device="cuda") for N in Ns]
    yarr = (ctypes.c_void_p * n)(*[y.data_ptr() for y in ys])
    parr = (ctypes.c_void_p * n)(*[p.data_ptr() for p in packed_list])
    narr = (ctypes.c_int * n)(*Ns)
    _check(lib().w4a32_matmul_quantized_grouped(yarr, _ptr(ws), parr, narr, n, M, K, _stream()),
           "w4a32_matmul_quantized_grouped")
    return ys


def matmul_quantized_silu_pair(ws, gate, up, M, K, N, out=None):
    """silu(gate Linear) * (up Linear) on rows already quantised into ws, one launch (M > 8)."""
    import torch

    y = out if out is not None else torch.empty((M, N), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_matmul_quantized_silu_pair(_ptr(y), _ptr(ws), _ptr(gate), _ptr(up), M, K, N, _stream()),
           "w4a32_matmul_quantized_silu_pair")
    return y


def matmul_quantized_splitk(ws, packed, M, K, N, scratch=None, out=None):
    """matmul_quantized() with scratch memory lent for partial sums (allocated here when absent)."""
    import torch

    y = out if out is not None else torch.empty((M, N), dtype=torch.float32, device="cuda")
    need = int(lib().w4a32_splitk_scratch_bytes(M, K, N))
    if scratch is None and need:
        scratch = _dev_empty(need)
    _check(lib().w4a32_matmul_quantized_splitk(_ptr(y), _ptr(ws), _ptr(packed), M, K, N,
                                               _ptr(scratch) if scratch is not None else None,
                                               scratch.numel() * scratch.element_size() if scratch is not None else 0,
                                               _stream()), "w4a32_matmul_quantized_splitk")
    return y


def matmul_quantized_splitk_parts(ws, packed, M, K, N):
    """The split-K product without the kernel that adds its parts up: returns (scratch, parts)."""
    need = int(lib().w4a32_splitk_scratch_bytes(M, K, N))
    scratch = _dev_empty(max(need, 16))
    parts = ctypes.c_int(0)
    _check(lib().w4a32_matmul_quantized_splitk_parts(_ptr(ws), _ptr(packed), M, K, N, _ptr(scratch), need,
                                                     ctypes.byref(parts), _stream()),
           "w4a32_matmul_quantized_splitk_parts")
    return scratch, parts.value


def quant_lhs_norm_parts(h, scratch, parts, packed, K_linear, weight, eps, ws=None):
    """quant_lhs_norm() with delta = the sum of a split-K Linear's parts + its bias: returns (ws, h + delta)."""
    import torch

    M, K = h.shape
    if ws is None:
        ws = _dev_empty(workspace_bytes(M, K))
    h_out = torch.empty_like(h)
    _check(lib().w4a32_quant_lhs_norm_parts(_ptr(h), _ptr(scratch), parts, _ptr(packed), K_linear, _ptr(weight),
                                            eps, _ptr(h_out), M, K, _ptr(ws), _stream()),
           "w4a32_quant_lhs_norm_parts")
    return ws, h_out


def matmul(x, packed, N, ws=None, out=None):
    """The whole op on a contiguous f32 cuda tensor x [M,K]."""
    import torch

    M, K = x.shape
    assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()
    if ws is None:
        ws = _dev_empty(workspace_bytes(M, K))
    y = out if out is not None else torch.empty((M, N), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_matmul(_ptr(y), _ptr(x), _ptr(packed), _ptr(ws), M, K, N, _stream()),
           "w4a32_matmul")
    return y


def matmul_ws(x, packed, N, ws=None, out=None):
    """The whole op with a workspace of stated size (w4a32_workspace_bytes_n by default: the library may then
    deal a long k range to several workgroups, as for down_proj at prefill sizes)."""
    import torch

    M, K = x.shape
    if ws is None:
        ws = _dev_empty(int(lib().w4a32_workspace_bytes_n(M, K, N)))
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_matmul_ws(_ptr(out), _ptr(x), _ptr(packed), _ptr(ws), ws.numel() * ws.element_size(), M, K, N,
                                 _stream()), "w4a32_matmul_ws")
    return out


def matmul_grouped(x, packed_list, n_list, ws=None):
    """Several Linears on the same rows x [M,K]; returns one output tensor per Linear."""
    import torch

    M, K = x.shape
    cnt = len(packed_list)
    if ws is None:
        ws = _dev_empty(workspace_bytes(M, K))
    ys = [torch.empty((M, n), dtype=torch.float32, device="cuda") for n in n_list]
    y_arr = (ctypes.c_void_p * cnt)(*[y.data_ptr() for y in ys])
    p_arr = (ctypes.c_void_p * cnt)(*[p.data_ptr() for p in packed_list])
    n_arr = (ctypes.c_int * cnt)(*n_list)
    _check(lib().w4a32_matmul_grouped(y_arr, _ptr(x), p_arr, n_arr, cnt, _ptr(ws), M, K, _stream()),
           "w4a32_matmul_grouped")
    return ys


# ---- decoder operators and runner (include/w4a32_decoder.h) ---------------------------------

def op_embedding(ids, table):
    import torch

    M, (V, D) = ids.numel(), table.shape
    out = torch.empty((M, D), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_embedding(_ptr(ids), _ptr(table), M, D, V, _ptr(out), _stream()),
           "w4a32_op_embedding")
    return out


def op_rmsnorm(h, weight, eps, delta=None):
    """Returns y, or (h + delta, y) when delta is given."""
    import torch

    M, D = h.shape
    y = torch.empty_like(h)
    h_out = torch.empty_like(h) if delta is not None else None
    _check(lib().w4a32_op_rmsnorm(_ptr(h), _ptr(delta), _ptr(weight), M, D, eps, _ptr(h_out), _ptr(y),
                                  _stream()), "w4a32_op_rmsnorm")
    return y if delta is None else (h_out, y)


def op_add(a, b):
    import torch

    out = torch.empty_like(a)
    _check(lib().w4a32_op_add(_ptr(a), _ptr(b), _ptr(out), a.numel(), _stream()), "w4a32_op_add")
    return out


def op_silu_mul(gate, up):
    import torch

    out = torch.empty_like(gate)
    _check(lib().w4a32_op_silu_mul(_ptr(gate), _ptr(up), _ptr(out), gate.numel(), _stream()),
           "w4a32_op_silu_mul")
    return out


def op_rope_table(max_pos, head_dim, base):
    import torch

    sin = torch.empty((max_pos, head_dim // 2), dtype=torch.float32, device="cuda")
    cos = torch.empty_like(sin)
    _check(lib().w4a32_op_rope_table(_ptr(sin), _ptr(cos), max_pos, head_dim, base, _stream()),
           "w4a32_op_rope_table")
    return sin, cos


def op_rope_kv(q, k, v, sin, cos, kcache, vcache, n_heads, n_kv_heads, head_dim, pos0, d_pos0=None):
    """q is rotated in place; kcache/vcache [n_kv_heads][max_seq][head_dim] receive rows pos0.."""
    M = q.shape[0]
    _check(lib().w4a32_op_rope_kv(_ptr(q), _ptr(k), _ptr(v), _ptr(sin), _ptr(cos), _ptr(kcache),
                                  _ptr(vcache), M, n_heads, n_kv_heads, head_dim, kcache.shape[1],
                                  _ptr(d_pos0), pos0, _stream()), "w4a32_op_rope_kv")


def op_im2col_conv3d(x, kernel, stride, ld_out=None):
    """x [B][C][T][H][W] f32 -> [B*OT*OH*OW][ld_out] (columns beyond C*kt*kh*kw are zero)."""
    import torch

    B, C, T, H, W = x.shape
    (kt, kh, kw), (st, sh, sw) = kernel, stride
    rows = B * ((T - kt) // st + 1) * ((H - kh) // sh + 1) * ((W - kw) // sw + 1)
    cols = C * kt * kh * kw
    ld = ld_out or (cols + 31) // 32 * 32
    out = torch.empty((rows, ld), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_im2col_conv3d(_ptr(x), _ptr(out), B, C, T, H, W, kt, kh, kw, st, sh, sw, ld,
                                        _stream()), "w4a32_op_im2col_conv3d")
    return out


def op_silu(x):
    import torch

    out = torch.empty_like(x)
    _check(lib().w4a32_op_silu(_ptr(x), _ptr(out), x.numel(), _stream()), "w4a32_op_silu")
    return out


def op_mul(a, b):
    import torch

    out = torch.empty_like(a)
    _check(lib().w4a32_op_mul(_ptr(a), _ptr(b), _ptr(out), a.numel(), _stream()), "w4a32_op_mul")
    return out


def op_rope(x, sin, cos, n_heads, head_dim, pos0):
    """Rows x [M][n_heads*head_dim] rotated at positions pos0.. (a new tensor)."""
    import torch

    out = torch.empty_like(x)
    _check(lib().w4a32_op_rope(_ptr(x), _ptr(out), _ptr(sin), _ptr(cos), x.shape[0], n_heads, head_dim, pos0,
                               sin.shape[0], _stream()), "w4a32_op_rope")
    return out


def op_attention_bshd(q, k, v, n_heads, n_kv_heads, head_dim, pos0):
    """Causal attention on k, v laid out [n_keys][n_kv_heads][head_dim]; q [M][n_heads*head_dim]."""
    import torch

    M, n_keys = q.shape[0], k.shape[0]
    out = torch.empty((M, n_heads * head_dim), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_attention_bshd(_ptr(q), _ptr(k), _ptr(v), _ptr(out), M, n_heads, n_kv_heads, head_dim,
                                         n_keys, pos0, _stream()), "w4a32_op_attention_bshd")
    return out


def op_matmul_f32_nt(a, b):
    """a [M][K] x b [N][K]^T, dense f32."""
    import torch

    (M, K), N = a.shape, b.shape[0]
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_matmul_f32_nt(_ptr(a), _ptr(b), _ptr(out), M, N, K, _stream()),
           "w4a32_op_matmul_f32_nt")
    return out


def _dense_dtype(b):
    import torch

    if b.dtype == torch.float16:
        return DENSE_F16
    if b.dtype == torch.float32:
        return DENSE_F32
    raise W4A32Error(f"a dense operand is f16 or f32, not {b.dtype}")


def op_matmul_nt(a, b):
    """a f32 [M][K] x b [N][K]^T with b held as f16 or f32; products and sums in f32."""
    import torch

    (M, K), N = a.shape, b.shape[0]
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_matmul_nt(_ptr(a), _ptr(b), _dense_dtype(b), _ptr(out), M, N, K, _stream()),
           "w4a32_op_matmul_nt")
    return out


def op_f16_to_f32(x):
    import torch

    out = torch.empty(x.shape, dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_f16_to_f32(_ptr(x), _ptr(out), x.numel(), _stream()), "w4a32_op_f16_to_f32")
    return out


def op_scratch(n_heads):
    sc = _dev_empty(int(lib().w4a32_op_scratch_bytes(n_heads)))
    _check(lib().w4a32_op_scratch_init(_ptr(sc), n_heads, _stream()), "w4a32_op_scratch_init")
    return sc


def op_attention(q, kcache, vcache, n_heads, n_kv_heads, head_dim, pos0, scratch=None, d_pos0=None):
    import torch

    M = q.shape[0]
    out = torch.empty((M, n_heads * head_dim), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_attention(_ptr(q), _ptr(kcache), _ptr(vcache), _ptr(out), M, n_heads,
                                    n_kv_heads, head_dim, kcache.shape[1], _ptr(d_pos0), pos0,
                                    _ptr(scratch), _stream()), "w4a32_op_attention")
    return out


def op_attention_prefill(q, kcache, vcache, n_heads, n_kv_heads, head_dim, pos0, d_pos0=None, part=None):
    """Causal attention of M rows with the keys of each query block dealt to several workgroups; `part`
    is the scratch (allocated here when not given)."""
    import torch

    M = q.shape[0]
    if part is None:
        need = int(lib().w4a32_op_attention_prefill_scratch_bytes(M, n_heads))
        part = torch.empty((max(need, 16),), dtype=torch.uint8, device="cuda")
    out = torch.empty((M, n_heads * head_dim), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_attention_prefill(_ptr(q), _ptr(kcache), _ptr(vcache), _ptr(out), M, n_heads,
                                            n_kv_heads, head_dim, kcache.shape[1], _ptr(d_pos0), pos0,
                                            _ptr(part), part.numel(), _stream()),
           "w4a32_op_attention_prefill")
    return out


def op_attention_prefill_bf16x3(q, kcache, vcache, n_heads, n_kv_heads, head_dim, pos0):
    """The prefill attention with its products on the bf16 matrix pipe (three terms per f32 operand)."""
    import torch

    M = q.shape[0]
    out = torch.empty((M, n_heads * head_dim), dtype=torch.float32, device="cuda")
    scratch = _dev_empty(int(lib().w4a32_op_attention_prefill_bf16x3_scratch_bytes(pos0 + M, n_kv_heads)))
    _check(lib().w4a32_op_attention_prefill_bf16x3(_ptr(q), _ptr(kcache), _ptr(vcache), _ptr(out), M, n_heads,
                                                   n_kv_heads, head_dim, kcache.shape[1], pos0, _ptr(scratch),
                                                   scratch.numel(), _stream()),
           "w4a32_op_attention_prefill_bf16x3")
    return out


def op_rope_attention_prefill_bf16x3(q, k, v, sin, cos, kcache, vcache, n_heads, n_kv_heads, head_dim, pos0):
    """op_rope_kv (q rotated in place, k and v appended to the caches at pos0..) + op_attention_prefill_bf16x3 with
    the rotation and the append done by the launch that splits K and V."""
    import torch

    M = q.shape[0]
    out = torch.empty((M, n_heads * head_dim), dtype=torch.float32, device="cuda")
    scratch = _dev_empty(int(lib().w4a32_op_attention_prefill_bf16x3_scratch_bytes(pos0 + M, n_kv_heads)))
    _check(lib().w4a32_op_rope_attention_prefill_bf16x3(_ptr(q), _ptr(k), _ptr(v), _ptr(sin), _ptr(cos),
                                                        _ptr(kcache), _ptr(vcache), _ptr(out), M, n_heads,
                                                        n_kv_heads, head_dim, kcache.shape[1], pos0,
                                                        _ptr(scratch), scratch.numel(), _stream()),
           "w4a32_op_rope_attention_prefill_bf16x3")
    return out


def op_rope_attention_decode(q, k, v, sin, cos, kcache, vcache, n_heads, n_kv_heads, head_dim, pos0,
                             scratch, d_pos0=None):
    """RoPE + cache append + attention of one token in one launch (q, k, v un-rotated)."""
    import torch

    out = torch.empty((1, n_heads * head_dim), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_rope_attention_decode(_ptr(q), _ptr(k), _ptr(v), _ptr(sin), _ptr(cos),
                                                _ptr(kcache), _ptr(vcache), _ptr(out), n_heads,
                                                n_kv_heads, head_dim, kcache.shape[1], _ptr(d_pos0), pos0,
                                                _ptr(scratch), _stream()),
           "w4a32_op_rope_attention_decode")
    return out


def op_rope_attention_decode_linear(q, k, v, sin, cos, kcache, vcache, packed, N, n_heads, n_kv_heads,
                                    head_dim, pos0, scratch, d_pos0=None):
    """op_rope_attention_decode followed by the Linear that reads it (o_proj), as the decoder's step issues
    them: the attention's key slices are merged by the Linear's row load. Returns y [1][N]."""
    import torch

    y = torch.empty((1, N), dtype=torch.float32, device="cuda")
    _check(lib().w4a32_op_rope_attention_decode_linear(
        _ptr(q), _ptr(k), _ptr(v), _ptr(sin), _ptr(cos), _ptr(kcache), _ptr(vcache), _ptr(packed), N, _ptr(y),
        n_heads, n_kv_heads, head_dim, kcache.shape[1], _ptr(d_pos0), pos0, _ptr(scratch), _stream()),
        "w4a32_op_rope_attention_decode_linear")
    return y


def op_argmax(logits, scratch, d_pos=None):
    import torch

    tok = torch.empty((1,), dtype=torch.int64, device="cuda")
    _check(lib().w4a32_op_argmax(_ptr(logits), logits.numel(), _ptr(scratch), _ptr(tok), _ptr(d_pos),
                                 _stream()), "w4a32_op_argmax")
    return tok


def decode_linear(x, packed_list, n_list, norm_weight=None, eps=1e-6, delta=None, want_sum=False,
                  silu_pair=False, in_parts=0, out_parts=0):
    """One f32 row x [1][K] through 1..4 Linears with the decoder's fusions (see w4a32_decode_linear).
    Returns (outputs, sum) where sum is x + delta when want_sum. in_parts > 1: x (delta with a norm) holds
    that many partial rows [in_parts][K]; out_parts > 1: the single output is [out_parts][N] partial rows."""
    import torch

    K = x.shape[-1]
    cnt = len(packed_list)
    ys = [torch.empty((max(out_parts, 1), n), dtype=torch.float32, device="cuda") for n in n_list]
    if silu_pair:
        ys = ys[:1]
    total = torch.empty((1, K), dtype=torch.float32, device="cuda") if want_sum else None
    a = DecodeLinearArgs()
    a.d_x, a.d_delta, a.d_sum_out = x.data_ptr(), _ptr(delta), _ptr(total)
    a.d_norm_weight, a.norm_eps, a.K, a.count, a.silu_pair = _ptr(norm_weight), eps, K, cnt, int(silu_pair)
    a.in_parts, a.out_parts = in_parts, out_parts
    for i in range(cnt):
        a.d_packed[i], a.N[i] = packed_list[i].data_ptr(), n_list[i]
        a.d_y[i] = ys[i].data_ptr() if i < len(ys) else None
    _check(lib().w4a32_decode_linear(ctypes.byref(a), _stream()), "w4a32_decode_linear")
    return ys, total


class Decoder:
    """Plumbing around the decoder runner: owns the state buffer and the argument structs.

    `layers` is a list of dicts with the packed blobs q,k,v,o,gate,up,down and the f32 norm weights
    attn_norm, ffn_norm (cuda tensors); embedding f32 [vocab][hidden]; lm_head a packed blob, or (with
    lm_head_dense=True) a dense f16 / f32 [vocab][hidden] tensor applied as the reference applies it."""

    def __init__(self, hidden, n_heads, n_kv_heads, intermediate, vocab, layers, embedding, final_norm,
                 lm_head, max_seq=1024, max_batch_tokens=512, rope_theta=1e6, rms_eps=1e-6, head_dim=128,
                 lm_head_dense=False):
        import torch

        self.cfg = DecoderConfig(hidden, n_heads, n_kv_heads, head_dim, intermediate, len(layers), vocab,
                                 max_seq, max_batch_tokens, rope_theta, rms_eps)
        self._keep = (layers, embedding, final_norm, lm_head)
        arr = (LayerWeights * len(layers))()
        for i, lw in enumerate(layers):
            for name, _ in LayerWeights._fields_:
                setattr(arr[i], name, lw[name].data_ptr())
        self._layers = arr
        if lm_head_dense:
            self.weights = DecoderWeights(embedding.data_ptr(), final_norm.data_ptr(), None, arr,
                                          lm_head.data_ptr(), _dense_dtype(lm_head))
        else:
            self.weights = DecoderWeights(embedding.data_ptr(), final_norm.data_ptr(), lm_head.data_ptr(), arr,
                                          None, 0)
        nbytes = int(lib().w4a32_decoder_state_bytes(ctypes.byref(self.cfg)))
        if nbytes == 0:
            raise W4A32Error("w4a32_decoder_state_bytes: invalid configuration")
        self.state = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        self.token = torch.zeros((1,), dtype=torch.int64, device="cuda")
        _check(lib().w4a32_decoder_init(ctypes.byref(self.cfg), _ptr(self.state), _stream()),
               "w4a32_decoder_init")

    def _view(self, which, count, dtype):
        off = int(lib().w4a32_decoder_state_offset(ctypes.byref(self.cfg), which))
        return self.state[off:off + count * dtype.itemsize].view(dtype)

    @property
    def position(self):
        import torch

        return int(self._view(0, 1, torch.int32).item())

    @property
    def logits(self):
        import torch

        return self._view(1, self.cfg.vocab, torch.float32)

    def prefill(self, tokens, pos0=0):
        """tokens: int64 cuda tensor [n]. Leaves the greedy next token in self.token."""
        _check(lib().w4a32_decoder_prefill(ctypes.byref(self.cfg), ctypes.byref(self.weights),
                                           _ptr(self.state), _ptr(tokens), tokens.numel(), pos0,
                                           _ptr(self.token), _stream()), "w4a32_decoder_prefill")
        self._host_pos = pos0 + tokens.numel()
        return self.token

    def step(self):
        """One greedy step: consumes self.token, replaces it with the next token. The position lives in device
        memory; this object also counts the steps it issues (or records into a graph) and refuses the one that
        would run past the cache. A caller that replays a captured step keeps count itself: past the end the
        kernels stay inside the cache (the last row is overwritten) but the tokens are meaningless."""
        if getattr(self, "_host_pos", 0) >= self.cfg.max_seq:
            raise W4A32Error(f"decoder step at position {self._host_pos}: the cache holds {self.cfg.max_seq}")
        self._host_pos = getattr(self, "_host_pos", 0) + 1
        _check(lib().w4a32_decoder_step(ctypes.byref(self.cfg), ctypes.byref(self.weights),
                                        _ptr(self.state), _ptr(self.token), _ptr(self.token), _stream()),
               "w4a32_decoder_step")
        return self.token
