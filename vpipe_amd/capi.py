"""ctypes binding of libvpq.so for tests and the benchmark.

torch supplies device memory and the stream; every call goes through the C ABI
of include/vpq.h with raw device pointers.  There is no fallback: a missing
library or a non-zero status raises.

Tensor conventions: packed codes are int32 tensors viewed as uint32 words
[N, K/8]; bf16 data are torch.bfloat16 tensors (or int16 tensors holding the
bit patterns).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libvpq.so")
_lib = None

VPQ_GATE_SWIGLU, VPQ_GATE_GEGLU = 1, 2
VPQ_QMV_AUTO, VPQ_QMV_SIMPLE, VPQ_QMV_MFMA, VPQ_QMV_STREAM, VPQ_QMV_RING, VPQ_QMV_ROWS, VPQ_QMV_FLOW = 0, 1, 2, 4, 5, 6, 7
VPQ_QMV_RING_SPLITK = 8

# Every symbol include/vpq.h declares: (name, restype, argtypes).
_vp, _i, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
SYMBOLS = [
    ("vpq_version", _i, []),
    ("vpq_status_string", ctypes.c_char_p, [_i]),
    ("vpq_last_device_error", ctypes.c_char_p, []),
    ("vpq_init", _i, []),
    ("vpq_device_cu_count", _i, []),
    ("vpq_dequant_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_embed_gather_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_dequant_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_qmv_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i]),
    ("vpq_qmv_w4g32_f32out", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_qmv_gated_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    ("vpq_qmm_dense_route_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i]),
    ("vpq_linear_workspace_bytes", _sz, [_i, _i, _i]),
    ("vpq_argmax_workspace_bytes", _sz, [_i, _i]),
    ("vpq_argmax_bf16", _i, [_vp, _vp, _vp, _i, _i, _vp, _sz]),
    ("vpq_argmax_bf16_static", _i, [_vp, _vp, _vp, _i, _i]),
    ("vpq_argmax_partial_bf16", _i, [_vp, _vp, _vp, _i, _i]),
    ("vpq_argmax_combine", _i, [_vp, _vp, _vp, _i]),
    ("vpq_gather_qmv_gated_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _i, _i, _i, _i]),
    ("vpq_gather_down_qmv_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _i, _i]),
    ("vpq_qmm_grouped_block_rows", _i, []),
    ("vpq_moe_sort_workspace_bytes", _sz, [_i]),
    ("vpq_moe_sort_pairs", _i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _sz]),
    ("vpq_qmm_grouped_gated_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i, _i]),
    ("vpq_qmm_grouped_down_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i]),
    ("vpq_sample_topp_bf16", _i, [_vp, _vp, _vp, _i, _f, _f, ctypes.c_uint32, _vp, _i, _f, _f, _i, _f, _vp]),
    ("vpq_sample_hist_workspace_bytes", _sz, [_i]),
    ("vpq_sample_hist_bf16", _i, [_vp, _vp, _vp, _i, _f, _f, ctypes.c_uint32, _vp, _f, _f, _i, _f, _vp, _i, _vp, _sz]),
    ("vpq_qmv_grouped_gated_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i]),
    ("vpq_qmv_grouped_down_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i]),
    ("vpq_moe_scatter_back_bf16", _i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_qmv_grouped_gated_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i]),
    ("vpq_qmv_grouped_down_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i]),
    ("vpq_qmv_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _sz, _i]),
    ("vpq_qmv_w4g64_f32out", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _sz, _i]),
    ("vpq_qmv_workspace_bytes", _sz, [_i, _i, _i]),
    ("vpq_qmm_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _f, _vp]),
    ("vpq_qmm_tiled_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _f, _vp, _i]),
    ("vpq_qmm_workspace_bytes", _sz, [_i, _i, _i]),
    ("vpq_qmm_splitk_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _sz]),
    ("vpq_qmm_dense_route_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i]),
    ("vpq_qmm_dense_route_lora_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _f, _vp]),
    ("vpq_lora_a_bf16", _i, [_vp, _vp, _vp, _vp, _i, _i, _i, _f]),
    ("vpq_linear_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _sz]),
    ("vpq_qmv_group_w4g64_bf16", _i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i]),
    ("vpq_qmv_group_w4g64_f16", _i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i]),
    ("vpq_qmv_group_w4g32_bf16", _i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i]),
    ("vpq_qmv_group_w8g64_bf16", _i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i]),
    ("vpq_rmsnorm_bf16", _i, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    ("vpq_dequant_w8g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_qmv_w8g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    ("vpq_requant_w8_to_w4_g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_qmv_gelu_mul_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    ("vpq_qmv_gelu_mul_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _i]),
    ("vpq_qmm_dense_route_w8g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i]),
    ("vpq_qmv_qkv_rms_bf16", _i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _f, _vp]),
    ("vpq_dequant_w8_f16", _i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_qmm_dense_route_w8_f16", _i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i]),
    ("vpq_qmm_dense_route_lora_bf16", _i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _f, _vp]),
    ("vpq_interleave_rows", _i, [_vp, _vp, _vp, _vp, _sz, _sz]),
    ("vpq_qmv_swiglu_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_qmv_swiglu_w4g64_f32out", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_qmm_swiglu_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    ("vpq_linear_swiglu_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_qmv_gated_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    ("vpq_qmv_gated_w4g64_f32out", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    ("vpq_qmm_gated_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
    ("vpq_linear_gated_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_dequant_w4g64_f16", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_qmv_w4g64_f16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    ("vpq_qmv_w4g64_f16_f32out", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_qmv_gated_w4g64_f16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_qmm_dense_route_w4g64_f16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i]),
    ("vpq_qmm_w4g64_f16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_lora_a_f16", _i, [_vp, _vp, _vp, _vp, _i, _i, _i, _f]),
    ("vpq_qmv_gelu_mul_w4g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    ("vpq_moe_gate_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_qmm_lora_w4g64_f16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _f, _vp]),
    ("vpq_qmm_tiled_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    ("vpq_qmm_tiled_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    ("vpq_dequant_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i]),
    ("vpq_qmv_gated_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_qmm_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_linear_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_linear_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_qmm_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_qmm_gated_w4g32_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    ("vpq_qmm_gated_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
    ("vpq_qmm_grouped_gated_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i, _i]),
    ("vpq_qmm_grouped_down_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i]),
    ("vpq_gather_qmv_gated_split_bf16", _i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _vp, _i, _i, _i, _i]),
    ("vpq_gather_qmv_gated_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _i, _i, _i, _i]),
    ("vpq_gather_down_qmv_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _i, _i]),
    ("vpq_qmv_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    ("vpq_qmv_w8g64_f32out", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    ("vpq_qmm_dense_route_w8g64_bf16", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i]),
    ("vpq_quantize_w4g64", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _f]),
    ("vpq_quantize", _i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _f]),
    ("vpq_f16_to_bf16", _i, [_vp, _vp, _vp, _sz]),
    ("vpq_profile_enable", _i, [_i]),
    ("vpq_profile_read", _i, [_vp, _i]),
    ("vpq_profile_empty_kernel", _i, [_vp, _vp]),
    ("vpq_profile_read_kernel", _i, [_vp, _vp, _sz, _vp]),
    ("vpq_weight_bytes", _sz, [_i, _i]),
    ("vpq_scale_bytes", _sz, [_i, _i]),
]


VPQ_ERR_WORKSPACE = -4
VPQ_ARGMAX_STATIC_MAX_ROWS = 64


class VpqError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = load().vpq_status_string(status).decode()
        dev = load().vpq_last_device_error().decode()
        super().__init__("%s: %s (%d)%s" % (where, msg, status, (" [" + dev + "]") if dev else ""))


def lib_path():
    return _SO


def build_id():
    """First 12 hex digits of the SHA-256 of the built library: names the build a measurement was taken on."""
    import hashlib
    with open(_SO, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:12]


def load():
    """dlopen libvpq.so (built by `python -m vpipe_amd.build`); raises if absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise FileNotFoundError(
                "%s is missing: build it with `python -m vpipe_amd.build` (hipcc, gfx950)" % _SO)
        import torch  # noqa: F401  -- loads the HIP runtime libvpq.so binds to
        L = ctypes.CDLL(_SO)
        for name, res, args in SYMBOLS:
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(st, where):
    if st != 0:
        raise VpqError(st, where)


def qmv_workspace(K, N, M, device="cuda"):
    """Scratch for the split of K across workgroups in qmv_w4g64 (reusable across calls on one stream)."""
    import torch
    nbytes = load().vpq_qmv_workspace_bytes(K, N, M)
    return torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=device)


def dequant_w4g64(w, scales, biases, K, N, out=None):
    import torch
    if out is None:
        out = torch.empty((N, K), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_dequant_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(out), K, N),
           "vpq_dequant_w4g64_bf16")
    return out


def embed_gather_w4g64(ids, w, scales, biases, H, vocab, out=None):
    """ids: int32 device tensor [T] -> bf16 [T, H], rows of the dequantized table."""
    import torch
    T = ids.numel()
    if out is None:
        out = torch.empty((T, H), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_embed_gather_w4g64_bf16(_stream(), _ptr(ids), _ptr(w), _ptr(scales), _ptr(biases), _ptr(out),
                                              H, T, vocab), "vpq_embed_gather_w4g64_bf16")
    return out


def dequant_w4g32(w, scales, biases, K, N, out=None):
    import torch
    if out is None:
        out = torch.empty((N, K), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_dequant_w4g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(out), K, N),
           "vpq_dequant_w4g32_bf16")
    return out


def qmv_w4g32(w, scales, biases, x, K, N, M, out=None, residual=None, f32out=False, scale_only=False, activation=0):
    """group-32 QMV; biases may be None with scale_only; activation != 0: interleaved gate|up pack -> [M, N/2]."""
    import torch
    L = load()
    so = 1 if scale_only else 0
    if activation:
        if out is None:
            out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=w.device)
        _check(L.vpq_qmv_gated_w4g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                          activation, so), "vpq_qmv_gated_w4g32_bf16")
        return out
    if f32out:
        if out is None:
            out = torch.empty((M, N), dtype=torch.float32, device=w.device)
        _check(L.vpq_qmv_w4g32_f32out(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M, so),
               "vpq_qmv_w4g32_f32out")
        return out
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _check(L.vpq_qmv_w4g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                _ptr(residual), so), "vpq_qmv_w4g32_bf16")
    return out


def qmm_dense_route_w4g32(w, scales, biases, x, K, N, M, w_deq=None, expand=True, out=None):
    import torch
    if w_deq is None:
        w_deq = torch.empty((N, K), dtype=torch.bfloat16, device=w.device)
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmm_dense_route_w4g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                                 _ptr(w_deq), 1 if expand else 0), "vpq_qmm_dense_route_w4g32_bf16")
    return out


def argmax_bf16(logits, out=None, two_stage=True):
    """bf16 [rows, V] (or [V]) -> int32 [rows]: lowest index of the largest logit of each row."""
    import torch
    L = load()
    rows, V = (1, logits.numel()) if logits.dim() == 1 else logits.shape
    if out is None:
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    ws, ws_bytes = None, 0
    if two_stage:
        ws_bytes = L.vpq_argmax_workspace_bytes(V, rows)
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=logits.device)
    _check(L.vpq_argmax_bf16(_stream(), _ptr(logits), _ptr(out), V, rows, _ptr(ws), ws_bytes), "vpq_argmax_bf16")
    return out


def sample_topp_bf16(logits, seen, temp, top_p, seed, ws=None, out=None, n_iter=24, rep=1.0, pres=0.0, top_k=0, min_p=0.0):
    """One row of bf16 logits [V] and its seen flags (uint8 [V], updated in place) -> int32 [1] with the drawn token."""
    import torch
    V = logits.numel()
    if ws is None:
        ws = torch.empty((V,), dtype=torch.bfloat16, device=logits.device)
    if out is None:
        out = torch.empty((1,), dtype=torch.int32, device=logits.device)
    _check(load().vpq_sample_topp_bf16(_stream(), _ptr(logits), _ptr(out), V, temp, top_p, seed, _ptr(ws), n_iter, rep, pres,
                                       top_k, min_p, _ptr(seen)), "vpq_sample_topp_bf16")
    return out


def sample_hist_slabs(V):
    """A slab count for vpq_sample_hist_bf16: about 4096 logits per workgroup, at most 64 workgroups."""
    return max(1, min(64, (V + 4095) // 4096), (V + 65534) // 65535)


def sample_hist_bf16(logits, seen, temp, top_p, seed, ws=None, out=None, work=None, n_slabs=0, rep=1.0, pres=0.0, top_k=0,
                     min_p=0.0):
    """As sample_topp_bf16 over n_slabs workgroups with the thresholds read off a histogram of the weights."""
    import torch
    V = logits.numel()
    if n_slabs <= 0:
        n_slabs = sample_hist_slabs(V)
    L = load()
    if ws is None:
        ws = torch.empty((V,), dtype=torch.bfloat16, device=logits.device)
    if out is None:
        out = torch.empty((1,), dtype=torch.int32, device=logits.device)
    need = int(L.vpq_sample_hist_workspace_bytes(n_slabs))
    if work is None:
        work = torch.empty((max(need, 4) // 4,), dtype=torch.float32, device=logits.device)
    _check(L.vpq_sample_hist_bf16(_stream(), _ptr(logits), _ptr(out), V, temp, top_p, seed, _ptr(ws), rep, pres, top_k, min_p,
                                  _ptr(seen), n_slabs, _ptr(work), work.numel() * work.element_size()),
           "vpq_sample_hist_bf16")
    return out


def argmax_bf16_static(logits, out):
    """As argmax_bf16(two_stage=True) through the entry point that allocates nothing: `out` (int32 [rows]) is the
    caller's, the slab pairs go to the library's static device scratch."""
    rows, V = (1, logits.numel()) if logits.dim() == 1 else logits.shape
    _check(load().vpq_argmax_bf16_static(_stream(), _ptr(logits), _ptr(out), V, rows), "vpq_argmax_bf16_static")
    return out


def gather_qmv_gated_w4g64(w, scales, biases, x, K, N, pair_eid, top_k, n_experts, out=None, activation=VPQ_GATE_SWIGLU):
    """Expert batch [E, N=2*inner, ...], x [M, K], pair_eid int32 [npair] -> bf16 [npair, N/2]."""
    import torch
    npair = pair_eid.numel()
    if out is None:
        out = torch.empty((npair, N // 2), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_gather_qmv_gated_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                  _ptr(pair_eid), npair, top_k, n_experts, activation),
           "vpq_gather_qmv_gated_w4g64_bf16")
    return out


def gather_down_qmv_w4g64(w, scales, biases, x, K, N, pair_eid, n_experts, out=None):
    """Expert batch [E, N, ...], x [npair, K], pair_eid int32 [npair] -> bf16 [npair, N]."""
    import torch
    npair = pair_eid.numel()
    if out is None:
        out = torch.empty((npair, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_gather_down_qmv_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                 _ptr(pair_eid), npair, n_experts), "vpq_gather_down_qmv_w4g64_bf16")
    return out


def grouped_block_rows():
    return int(load().vpq_qmm_grouped_block_rows())


def moe_max_tiles(npair, n_experts, block_rows):
    """Blocks to provide for npair pairs: every expert's share rounded up to whole blocks."""
    return (npair + block_rows - 1) // block_rows + min(n_experts, npair)


def moe_sort_pairs(pair_eid, top_k, n_experts, block_rows=None, max_tiles=None):
    """pair_eid int32 [npair] -> (tile2e [max_tiles], srow [npad], sdst [npad], ntiles [1]), device int32."""
    import torch
    L = load()
    npair = pair_eid.numel()
    if block_rows is None:
        block_rows = grouped_block_rows()
    if max_tiles is None:
        max_tiles = moe_max_tiles(npair, n_experts, block_rows)
    dev = pair_eid.device
    npad = max_tiles * block_rows
    t2e = torch.empty(max_tiles, dtype=torch.int32, device=dev)
    srow = torch.empty(npad, dtype=torch.int32, device=dev)
    sdst = torch.empty(npad, dtype=torch.int32, device=dev)
    ntiles = torch.empty(1, dtype=torch.int32, device=dev)
    ws_bytes = int(L.vpq_moe_sort_workspace_bytes(n_experts))
    ws = torch.empty(ws_bytes // 4, dtype=torch.int32, device=dev)
    _check(L.vpq_moe_sort_pairs(_stream(), _ptr(pair_eid), npair, top_k, n_experts, block_rows, max_tiles, _ptr(t2e),
                                _ptr(srow), _ptr(sdst), _ptr(ntiles), _ptr(ws), ws_bytes), "vpq_moe_sort_pairs")
    return t2e, srow, sdst, ntiles


def qmm_grouped_gated_w4g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out=None, activation=VPQ_GATE_SWIGLU):
    """Expert batch [E, N=2*inner, ...], x [rows_x, K], sorted slots -> bf16 [npad, N/2] in slot order."""
    import torch
    npad = srow.numel()
    if out is None:
        out = torch.empty((npad, N // 2), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmm_grouped_gated_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                   npad, _ptr(tile2e), _ptr(srow), n_experts, x.shape[0], activation),
           "vpq_qmm_grouped_gated_w4g64_bf16")
    return out


def qmm_grouped_down_w4g64(w, scales, biases, x, K, N, tile2e, sdst, n_experts, out):
    """Expert batch [E, N, ...], x [npad, K] in slot order -> rows of out [npair, N] in pair order."""
    npad = sdst.numel()
    _check(load().vpq_qmm_grouped_down_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                  npad, _ptr(tile2e), _ptr(sdst), n_experts, out.shape[0]),
           "vpq_qmm_grouped_down_w4g64_bf16")
    return out


VPQ_QMV_GROUPED_SLOTS = 2


def qmv_grouped_gated_w4g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out, activation=VPQ_GATE_SWIGLU, bits=4):
    """Expert batch [E, N=2*inner, ...], x [rows_x, K], tiles of two sorted slots -> live rows of out [npad, N/2]."""
    npad = srow.numel()
    name = "vpq_qmv_grouped_gated_w%dg64_bf16" % bits
    _check(getattr(load(), name)(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                 npad, _ptr(tile2e), _ptr(srow), n_experts, activation), name)
    return out


def qmv_grouped_down_w4g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out, bits=4):
    """Expert batch [E, N, ...], x [npad, K] in slot order -> live rows of out [npad, N] in slot order."""
    npad = srow.numel()
    name = "vpq_qmv_grouped_down_w%dg64_bf16" % bits
    _check(getattr(load(), name)(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                 npad, _ptr(tile2e), _ptr(srow), n_experts), name)
    return out


def moe_scatter_back(dsorted, sdst, npair, out=None):
    """Sorted rows [npad, H] -> pair order [npair, H] (rows no slot points at are left as they are)."""
    import torch
    npad, H = dsorted.shape
    if out is None:
        out = torch.zeros((npair, H), dtype=dsorted.dtype, device=dsorted.device)
    _check(load().vpq_moe_scatter_back_bf16(_stream(), _ptr(dsorted), _ptr(sdst), _ptr(out), npad, H, npair),
           "vpq_moe_scatter_back_bf16")
    return out


def qmv_grouped_gated_w8g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out, activation=VPQ_GATE_SWIGLU):
    return qmv_grouped_gated_w4g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out, activation, bits=8)


def qmv_grouped_down_w8g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out):
    return qmv_grouped_down_w4g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out, bits=8)


def qmv_w4g64(w, scales, biases, x, K, N, M, out=None, residual=None, ws=None, variant=0, f32out=False):
    import torch
    L = load()
    ws_bytes = 0 if ws is None else ws.numel() * ws.element_size()
    if f32out:
        if out is None:
            out = torch.empty((M, N), dtype=torch.float32, device=w.device)
        _check(L.vpq_qmv_w4g64_f32out(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                      K, N, M, _ptr(ws), ws_bytes, variant), "vpq_qmv_w4g64_f32out")
        return out
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _check(L.vpq_qmv_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                K, N, M, _ptr(residual), _ptr(ws), ws_bytes, variant), "vpq_qmv_w4g64_bf16")
    return out


def interleave_gate_up(gate, up):
    """(w, scales, biases) of gate and of up, each [ffn, ...] -> the interleaved pack [2*ffn, ...]."""
    import torch
    outs = []
    for a, b in zip(gate, up):
        assert a.shape == b.shape and a.dtype == b.dtype and a.is_contiguous() and b.is_contiguous()
        out = torch.empty((2 * a.shape[0],) + tuple(a.shape[1:]), dtype=a.dtype, device=a.device)
        row_bytes = a.stride(0) * a.element_size()
        _check(load().vpq_interleave_rows(_stream(), _ptr(a), _ptr(b), _ptr(out), row_bytes, a.shape[0]),
               "vpq_interleave_rows")
        outs.append(out)
    return tuple(outs)


def qmv_swiglu_w4g64(w, scales, biases, x, K, N, M, out=None, variant=0, f32out=False, activation=VPQ_GATE_SWIGLU):
    """y [M, N/2] = act(gate) * up over an interleaved gate|up pack [N, K] (SwiGLU unless `activation` says GEGLU)."""
    import torch
    L = load()
    if f32out:
        if out is None:
            out = torch.empty((M, N // 2), dtype=torch.float32, device=w.device)
        if activation == VPQ_GATE_SWIGLU:
            st = L.vpq_qmv_swiglu_w4g64_f32out(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M, variant)
        else:
            st = L.vpq_qmv_gated_w4g64_f32out(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                              variant, activation)
        _check(st, "vpq_qmv_gated_w4g64_f32out")
        return out
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=w.device)
    if activation == VPQ_GATE_SWIGLU:
        st = L.vpq_qmv_swiglu_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M, variant)
    else:
        st = L.vpq_qmv_gated_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M, variant,
                                        activation)
    _check(st, "vpq_qmv_gated_w4g64_bf16")
    return out


def qmm_swiglu_w4g64(w, scales, biases, x, K, N, M, out=None, out_stride=0, out_off=0, activation=VPQ_GATE_SWIGLU):
    import torch
    if out is None:
        out = torch.empty((M, out_stride if out_stride > 0 else N // 2), dtype=torch.bfloat16, device=w.device)
    if activation == VPQ_GATE_SWIGLU:
        st = load().vpq_qmm_swiglu_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                              out_stride, out_off)
    else:
        st = load().vpq_qmm_gated_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                             out_stride, out_off, activation)
    _check(st, "vpq_qmm_gated_w4g64_bf16")
    return out


def linear_swiglu_w4g64(w, scales, biases, x, K, N, M, out=None, activation=VPQ_GATE_SWIGLU):
    import torch
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=w.device)
    if activation == VPQ_GATE_SWIGLU:
        st = load().vpq_linear_swiglu_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M)
    else:
        st = load().vpq_linear_gated_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                                activation)
    _check(st, "vpq_linear_gated_w4g64_bf16")
    return out


def qmm_splitk_w4g64(w, scales, biases, x, K, N, M, splits=0, ws=None, out=None):
    """Split-K QMM; ws: uint8 tensor of vpq_qmm_workspace_bytes (allocated here if None)."""
    import torch
    L = load()
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    if ws is None:
        need = max(L.vpq_qmm_workspace_bytes(K, N, M), (splits if splits > 1 else 0) * M * N * 4, 256)
        ws = torch.empty(need, dtype=torch.uint8, device=w.device)
    _check(L.vpq_qmm_splitk_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M, splits,
                                       _ptr(ws), ws.numel()), "vpq_qmm_splitk_w4g64_bf16")
    return out


def gather_qmv_gated_split(gate, gate_bits, up, up_bits, x, K, ffn, pair_eid, top_k, n_experts, out=None,
                           activation=VPQ_GATE_SWIGLU):
    """gate, up: (w, scales, biases) of separate (batched) packs at their own widths; pair_eid None: rows of x."""
    import torch
    rows = x.shape[0] if pair_eid is None else pair_eid.numel()
    if out is None:
        out = torch.empty((rows, ffn), dtype=torch.bfloat16, device=x.device)
    _check(load().vpq_gather_qmv_gated_split_bf16(_stream(), _ptr(gate[0]), _ptr(gate[1]), _ptr(gate[2]), gate_bits,
                                                  _ptr(up[0]), _ptr(up[1]), _ptr(up[2]), up_bits, _ptr(x), _ptr(out), K, ffn,
                                                  _ptr(pair_eid), rows, top_k, n_experts, activation),
           "vpq_gather_qmv_gated_split_bf16")
    return out


def linear_twin(kind, w, scales, biases, x, K, N, M, out=None):
    """kind: "w8g64" or "w4g32": the size-based entrance of that format."""
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    fn = getattr(load(), "vpq_linear_%s_bf16" % kind)
    _check(fn(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M), "vpq_linear_%s_bf16" % kind)
    return out


def qmm_w4g32(w, scales, biases, x, K, N, M, out=None, activation=0, tile_n=0):
    """Fused group-32 GEMM; activation != 0: interleaved gate|up pack -> [M, N/2].  tile_n: 0 = the library's
    choice; 128 the 256x128 tile kernel; -128 / 192 / 256 the large-tile kernel at that width."""
    import torch
    if out is None:
        out = torch.empty((M, N // 2 if activation else N), dtype=torch.bfloat16, device=w.device)
    if tile_n:
        _check(load().vpq_qmm_tiled_w4g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                               activation, tile_n), "vpq_qmm_tiled_w4g32_bf16")
        return out
    _check(load().vpq_qmm_gated_w4g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                           activation), "vpq_qmm_gated_w4g32_bf16")
    return out


def qmm_w8g64(w, scales, biases, x, K, N, M, out=None, activation=0, out_stride=0, out_off=0, tile_n=0):
    """Fused 8-bit GEMM; activation != 0: interleaved gate|up pack -> [M, N/2].  tile_n: 0 = the library's choice;
    128 the 256x128 tile kernel; -128 / 192 the large-tile kernel at that width."""
    import torch
    if out is None:
        out = torch.empty((M, N // 2 if activation else N), dtype=torch.bfloat16, device=w.device)
    if tile_n:
        _check(load().vpq_qmm_tiled_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                               activation, tile_n), "vpq_qmm_tiled_w8g64_bf16")
        return out
    _check(load().vpq_qmm_gated_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                           out_stride, out_off, activation), "vpq_qmm_gated_w8g64_bf16")
    return out


def qmm_grouped_gated_w8g64(w, scales, biases, x, K, N, tile2e, srow, n_experts, out=None, activation=VPQ_GATE_SWIGLU):
    import torch
    npad = srow.numel()
    if out is None:
        out = torch.empty((npad, N // 2), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmm_grouped_gated_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                   npad, _ptr(tile2e), _ptr(srow), n_experts, x.shape[0], activation),
           "vpq_qmm_grouped_gated_w8g64_bf16")
    return out


def qmm_grouped_down_w8g64(w, scales, biases, x, K, N, tile2e, sdst, n_experts, out):
    npad = sdst.numel()
    _check(load().vpq_qmm_grouped_down_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                  npad, _ptr(tile2e), _ptr(sdst), n_experts, out.shape[0]),
           "vpq_qmm_grouped_down_w8g64_bf16")
    return out


def qmv_gated_w8g64(w, scales, biases, x, K, N, M, out=None, activation=VPQ_GATE_SWIGLU):
    """8-bit interleaved gate|up pack [N=2*ffn, K/4], x [M, K] -> bf16 [M, N/2]."""
    import torch
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmv_gated_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                           activation), "vpq_qmv_gated_w8g64_bf16")
    return out


def gather_qmv_gated_w8g64(w, scales, biases, x, K, N, pair_eid, top_k, n_experts, out=None, activation=VPQ_GATE_SWIGLU):
    """8-bit expert batch [E, N=2*inner, K/4], x [M, K], pair_eid int32 [npair] -> bf16 [npair, N/2]."""
    import torch
    npair = pair_eid.numel()
    if out is None:
        out = torch.empty((npair, N // 2), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_gather_qmv_gated_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                  _ptr(pair_eid), npair, top_k, n_experts, activation),
           "vpq_gather_qmv_gated_w8g64_bf16")
    return out


def gather_down_qmv_w8g64(w, scales, biases, x, K, N, pair_eid, n_experts, out=None):
    """8-bit expert batch [E, N, K/4], x [npair, K], pair_eid int32 [npair] -> bf16 [npair, N]."""
    import torch
    npair = pair_eid.numel()
    if out is None:
        out = torch.empty((npair, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_gather_down_qmv_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                 _ptr(pair_eid), npair, n_experts), "vpq_gather_down_qmv_w8g64_bf16")
    return out


def dequant_w4g64_f16(w, scales, biases, K, N, out=None):
    """binary16 scales / biases (torch.float16) -> float16 [N, K]."""
    import torch
    if out is None:
        out = torch.empty((N, K), dtype=torch.float16, device=w.device)
    _check(load().vpq_dequant_w4g64_f16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(out), K, N),
           "vpq_dequant_w4g64_f16")
    return out


def qmv_w4g64_f16(w, scales, biases, x, K, N, M, out=None, residual=None, f32out=False, activation=0):
    """float16 elements; activation != 0: interleaved gate|up pack -> [M, N/2]."""
    import torch
    L = load()
    if activation:
        if out is None:
            out = torch.empty((M, N // 2), dtype=torch.float16, device=w.device)
        _check(L.vpq_qmv_gated_w4g64_f16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                         activation), "vpq_qmv_gated_w4g64_f16")
        return out
    if f32out:
        if out is None:
            out = torch.empty((M, N), dtype=torch.float32, device=w.device)
        _check(L.vpq_qmv_w4g64_f16_f32out(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M),
               "vpq_qmv_w4g64_f16_f32out")
        return out
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=w.device)
    _check(L.vpq_qmv_w4g64_f16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                               _ptr(residual)), "vpq_qmv_w4g64_f16")
    return out


def qmm_dense_route_w4g64_f16(w, scales, biases, x, K, N, M, w_deq, expand=True, out=None):
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=w.device)
    _check(load().vpq_qmm_dense_route_w4g64_f16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                                _ptr(w_deq), 1 if expand else 0), "vpq_qmm_dense_route_w4g64_f16")
    return out


def qmm_w4g64_f16(w, scales, biases, x, K, N, M, activation=0, out=None):
    """The fused GEMM on IEEE binary16 elements (the large-tile kernel: K % 512 == 0); activation 1 / 2 gives
    the SwiGLU / GEGLU store of an interleaved gate|up pack, y [M, N/2]."""
    import torch
    if out is None:
        out = torch.empty((M, N // 2 if activation else N), dtype=torch.float16, device=w.device)
    _check(load().vpq_qmm_w4g64_f16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                    activation), "vpq_qmm_w4g64_f16")
    return out


def qmv_gelu_mul_w4g64(w, scales, biases, x, K, N, mul, out=None):
    """y[n] = bf16(gelu_tanh(bf16(W x)[n]) * mul[n]) for one row of x."""
    import torch
    if out is None:
        out = torch.empty((1, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmv_gelu_mul_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                              _ptr(mul)), "vpq_qmv_gelu_mul_w4g64_bf16")
    return out


def qmv_gelu_mul_w8g64(w, scales, biases, x, K, N, mul, out=None):
    """The 8-bit twin of qmv_gelu_mul_w4g64."""
    import torch
    if out is None:
        out = torch.empty((1, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmv_gelu_mul_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                              _ptr(mul)), "vpq_qmv_gelu_mul_w8g64_bf16")
    return out


def qmv_gelu_mul_w4g32(w, scales, biases, x, K, N, mul, out=None, scale_only=False):
    """The group-32 twin of qmv_gelu_mul_w4g64."""
    import torch
    if out is None:
        out = torch.empty((1, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmv_gelu_mul_w4g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases) if biases is not None else None,
                                              _ptr(x), _ptr(out), K, N, _ptr(mul), int(scale_only)),
           "vpq_qmv_gelu_mul_w4g32_bf16")
    return out


def requant_w8_to_w4(w8, s8, b8, K, N):
    """8-bit group-64 pack -> (w4 uint32 [N, K/8] viewed as int32, s4, b4 bf16 [N, K/64])."""
    import torch
    w4 = torch.empty((N, K // 8), dtype=torch.int32, device=w8.device)
    s4 = torch.empty((N, K // 64), dtype=torch.bfloat16, device=w8.device)
    b4 = torch.empty((N, K // 64), dtype=torch.bfloat16, device=w8.device)
    _check(load().vpq_requant_w8_to_w4_g64_bf16(_stream(), _ptr(w8), _ptr(s8), _ptr(b8), _ptr(w4), _ptr(s4), _ptr(b4),
                                                K, N), "vpq_requant_w8_to_w4_g64_bf16")
    return w4, s4, b4


def moe_gate_w8g64(w, scales, biases, x, K, M, out=None):
    """gate[m] = bf16(sigmoid(W[1,K] . x[m])) over a one-row 8-bit pack."""
    import torch
    if out is None:
        out = torch.empty((M,), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_moe_gate_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, M),
           "vpq_moe_gate_w8g64_bf16")
    return out


def lora_a_f16(x, A, M, K, r, alpha, out=None):
    import torch
    if out is None:
        out = torch.empty((M, r), dtype=torch.float16, device=x.device)
    _check(load().vpq_lora_a_f16(_stream(), _ptr(x), _ptr(A), _ptr(out), M, K, r, alpha), "vpq_lora_a_f16")
    return out


def qmm_lora_w4g64_f16(w, scales, biases, x, K, N, M, lora_A, lora_B, r, alpha, out=None, t_ws=None):
    """The fused binary16 GEMM with a runtime adapter (A [r,K], B [N,r], binary16)."""
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=w.device)
    if t_ws is None:
        t_ws = torch.empty((M, r), dtype=torch.float16, device=w.device)
    _check(load().vpq_qmm_lora_w4g64_f16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                         _ptr(lora_A), _ptr(lora_B), r, alpha, _ptr(t_ws)), "vpq_qmm_lora_w4g64_f16")
    return out


def dequant_w8g64(w, scales, biases, K, N, out=None):
    import torch
    if out is None:
        out = torch.empty((N, K), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_dequant_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(out), K, N),
           "vpq_dequant_w8g64_bf16")
    return out


def qmv_w8g64(w, scales, biases, x, K, N, M, out=None, residual=None, f32out=False):
    import torch
    L = load()
    if f32out:
        if out is None:
            out = torch.empty((M, N), dtype=torch.float32, device=w.device)
        _check(L.vpq_qmv_w8g64_f32out(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M),
               "vpq_qmv_w8g64_f32out")
        return out
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _check(L.vpq_qmv_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                _ptr(residual)), "vpq_qmv_w8g64_bf16")
    return out


def qmm_dense_route_w8g64(w, scales, biases, x, K, N, M, w_deq, expand=True, out=None):
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmm_dense_route_w8g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                                 K, N, M, _ptr(w_deq), 1 if expand else 0), "vpq_qmm_dense_route_w8g64_bf16")
    return out


def lora_a(x, A, M, K, r, alpha, out=None):
    import torch
    if out is None:
        out = torch.empty((M, r), dtype=torch.bfloat16, device=x.device)
    _check(load().vpq_lora_a_bf16(_stream(), _ptr(x), _ptr(A), _ptr(out), M, K, r, alpha), "vpq_lora_a_bf16")
    return out


def qmm_w4g64(w, scales, biases, x, K, N, M, out=None, lora_A=None, lora_B=None, r=0, alpha=0.0, t_ws=None, tile_n=0):
    """tile_n: 0 = the library's choice; 128 the 256x128 tile kernel; 192 / 256 the large-tile kernel."""
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    if lora_A is not None and t_ws is None:
        t_ws = torch.empty((M, r), dtype=torch.bfloat16, device=w.device)
    if tile_n:
        _check(load().vpq_qmm_tiled_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                               K, N, M, _ptr(lora_A), _ptr(lora_B), r, alpha, _ptr(t_ws), tile_n),
               "vpq_qmm_tiled_w4g64_bf16")
        return out
    _check(load().vpq_qmm_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                     K, N, M, _ptr(lora_A), _ptr(lora_B), r, alpha, _ptr(t_ws)),
           "vpq_qmm_w4g64_bf16")
    return out


def qmm_dense_route_w4g64(w, scales, biases, x, K, N, M, w_deq, expand=True, out=None, lora_A=None, lora_B=None, r=0,
                          alpha=0.0, t_ws=None):
    """Dequant-once route: w_deq is bf16 [N,K] scratch (or the kept expansion when expand=False); with lora_A / lora_B
    the runtime adapter of qmm_w4g64 in the dense GEMM's accumulators."""
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    if lora_A is None:
        _check(load().vpq_qmm_dense_route_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                                     K, N, M, _ptr(w_deq), 1 if expand else 0),
               "vpq_qmm_dense_route_w4g64_bf16")
        return out
    if t_ws is None:
        t_ws = torch.empty((M, r), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmm_dense_route_lora_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                                      K, N, M, _ptr(w_deq), 1 if expand else 0, _ptr(lora_A), _ptr(lora_B),
                                                      r, alpha, _ptr(t_ws)), "vpq_qmm_dense_route_lora_w4g64_bf16")
    return out


def linear_w4g64(w, scales, biases, x, K, N, M, out=None, ws=None):
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    ws_bytes = 0 if ws is None else ws.numel() * ws.element_size()
    _check(load().vpq_linear_w4g64_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out),
                                        K, N, M, _ptr(ws), ws_bytes), "vpq_linear_w4g64_bf16")
    return out


class QmvGroup:
    """The pointer tables of a grouped launch, built once for a fixed set of tensors so that a
    launch costs one foreign call (a decode loop launches the same groups every token)."""

    def __init__(self, packs, x, K, M, outs, f16=False, entry=None, extra=()):
        self.entry = entry or ("vpq_qmv_group_w4g64_f16" if f16 else "vpq_qmv_group_w4g64_bf16")
        self.extra = tuple(extra)
        n = len(packs)
        PA = ctypes.c_void_p * n
        self.keep = (packs, x, outs)       # the tables hold raw pointers: keep the tensors alive
        self.n, self.K, self.M = n, K, M
        self.w = PA(*[p[0].data_ptr() for p in packs])
        self.s = PA(*[p[1].data_ptr() for p in packs])
        self.b = PA(*[p[2].data_ptr() for p in packs])
        self.y = PA(*[o.data_ptr() for o in outs])
        self.N = (ctypes.c_int * n)(*[int(p[3]) for p in packs])
        self.x = _ptr(x)
        self.outs = outs

    def launch(self):
        _check(getattr(load(), self.entry)(_stream(), self.n, self.w, self.s, self.b, self.x, self.y, self.K,
                                           self.N, self.M, *self.extra), self.entry)
        return self.outs


def qmv_group_w4g64(packs, x, K, M, outs=None):
    """packs: list of (w, scales, biases, N), 1..4 of them sharing x [M,K]; one launch."""
    import torch
    if outs is None:
        outs = [torch.empty((M, p[3]), dtype=torch.bfloat16, device=x.device) for p in packs]
    return QmvGroup(packs, x, K, M, outs).launch()


def qmv_group_w4g32(packs, x, K, M, outs=None, scale_only=False):
    """The grouped launch over 4-bit group-32 packs (scales / biases [N, K/32])."""
    import torch
    if outs is None:
        outs = [torch.empty((M, p[3]), dtype=torch.bfloat16, device=x.device) for p in packs]
    return QmvGroup(packs, x, K, M, outs, entry="vpq_qmv_group_w4g32_bf16", extra=(1 if scale_only else 0,)).launch()


def qmv_group_w8g64(packs, x, K, M, outs=None):
    """The grouped call over 8-bit group-64 packs (w uint32 [N, K/4])."""
    import torch
    if outs is None:
        outs = [torch.empty((M, p[3]), dtype=torch.bfloat16, device=x.device) for p in packs]
    return QmvGroup(packs, x, K, M, outs, entry="vpq_qmv_group_w8g64_bf16").launch()


def dequant_w8g32(w, scales, biases, K, N, out=None):
    import torch
    if out is None:
        out = torch.empty((N, K), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_dequant_w8g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(out), K, N),
           "vpq_dequant_w8g32_bf16")
    return out


def qmv_w8g32(w, scales, biases, x, K, N, M, out=None, residual=None):
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmv_w8g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                     _ptr(residual)), "vpq_qmv_w8g32_bf16")
    return out


def qmm_dense_route_w8g32(w, scales, biases, x, K, N, M, w_deq, expand=True, out=None):
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmm_dense_route_w8g32_bf16(_stream(), _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                                 _ptr(w_deq), 1 if expand else 0), "vpq_qmm_dense_route_w8g32_bf16")
    return out


def rmsnorm_bf16(x, norm_w, K, M, eps, out=None):
    import torch
    if out is None:
        out = torch.empty((M, K), dtype=torch.bfloat16, device=x.device)
    _check(load().vpq_rmsnorm_bf16(_stream(), _ptr(x), _ptr(norm_w), _ptr(out), K, M, eps), "vpq_rmsnorm_bf16")
    return out


VPQ_FORMAT_W4G64, VPQ_FORMAT_W4G32, VPQ_FORMAT_W8G64, VPQ_FORMAT_W8G32 = 0, 1, 2, 3


def qmv_qkv_rms(fmt, packs, x, norm_w, K, eps, outs=None, x_norm_ws=None):
    """RMSNorm of the row x [1,K], then the grouped GEMV of the format over it; packs as qmv_group_w4g64."""
    import torch
    if outs is None:
        outs = [torch.empty((1, p[3]), dtype=torch.bfloat16, device=x.device) for p in packs]
    if x_norm_ws is None:
        x_norm_ws = torch.empty((1, K), dtype=torch.bfloat16, device=x.device)
    n = len(packs)
    PA = ctypes.c_void_p * n
    wt, st, bt = (PA(*[p[i].data_ptr() for p in packs]) for i in range(3))
    yt = PA(*[o.data_ptr() for o in outs])
    Nt = (ctypes.c_int * n)(*[int(p[3]) for p in packs])
    _check(load().vpq_qmv_qkv_rms_bf16(_stream(), fmt, n, wt, st, bt, _ptr(x), _ptr(norm_w), yt, K, Nt, eps, _ptr(x_norm_ws)),
           "vpq_qmv_qkv_rms_bf16")
    return outs


def qmv_group_w4g64_f16(packs, x, K, M, outs=None):
    """As qmv_group_w4g64 on IEEE binary16 elements."""
    import torch
    if outs is None:
        outs = [torch.empty((M, p[3]), dtype=torch.float16, device=x.device) for p in packs]
    return QmvGroup(packs, x, K, M, outs, f16=True).launch()


def quantize_w4g64(src, K, N, clip=1.0):
    """bf16 [N,K] -> (codes int32 [N,K/8], scales f16 bits int16 [N,K/64], biases f16 bits)."""
    import torch
    w = torch.empty((N, K // 8), dtype=torch.int32, device=src.device)
    s = torch.empty((N, K // 64), dtype=torch.int16, device=src.device)
    b = torch.empty((N, K // 64), dtype=torch.int16, device=src.device)
    _check(load().vpq_quantize_w4g64(_stream(), _ptr(src), _ptr(w), _ptr(s), _ptr(b), K, N, clip),
           "vpq_quantize_w4g64")
    return w, s, b


def f16_to_bf16(t):
    import torch
    out = torch.empty(t.shape, dtype=torch.int16, device=t.device)
    _check(load().vpq_f16_to_bf16(_stream(), _ptr(t), _ptr(out), t.numel()), "vpq_f16_to_bf16")
    return out


def qmm_dense_route_lora(fmt, w, scales, biases, x, K, N, M, w_deq, lora_A, lora_B, r, alpha, expand=True, out=None,
                         t_ws=None):
    """The dequant-once route with the runtime adapter over a pack of format fmt (VPQ_FORMAT_*)."""
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    if t_ws is None:
        t_ws = torch.empty((M, r), dtype=torch.bfloat16, device=w.device)
    _check(load().vpq_qmm_dense_route_lora_bf16(_stream(), fmt, _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N,
                                                M, _ptr(w_deq), 1 if expand else 0, _ptr(lora_A), _ptr(lora_B), r, alpha,
                                                _ptr(t_ws)), "vpq_qmm_dense_route_lora_bf16")
    return out


def dequant_w8_f16(w, scales, biases, K, N, group=64, out=None):
    """8-bit codes, binary16 scales / biases -> binary16 [N, K]."""
    import torch
    if out is None:
        out = torch.empty((N, K), dtype=torch.float16, device=w.device)
    _check(load().vpq_dequant_w8_f16(_stream(), group, _ptr(w), _ptr(scales), _ptr(biases), _ptr(out), K, N),
           "vpq_dequant_w8_f16")
    return out


def qmm_dense_route_w8_f16(w, scales, biases, x, K, N, M, w_deq, group=64, expand=True, out=None):
    import torch
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=w.device)
    _check(load().vpq_qmm_dense_route_w8_f16(_stream(), group, _ptr(w), _ptr(scales), _ptr(biases), _ptr(x), _ptr(out), K, N, M,
                                             _ptr(w_deq), 1 if expand else 0), "vpq_qmm_dense_route_w8_f16")
    return out


def quantize(src, K, N, bits=4, group=64, clip=1.0):
    """The packer at any width and group: src bf16 or float16 [N, K] -> (w int32 [N, K*bits/32], scales, biases float16
    [N, K/group])."""
    import torch
    w = torch.empty((N, K * bits // 32), dtype=torch.int32, device=src.device)
    s = torch.empty((N, K // group), dtype=torch.float16, device=src.device)
    b = torch.empty((N, K // group), dtype=torch.float16, device=src.device)
    _check(load().vpq_quantize(_stream(), bits, group, 1 if src.dtype == torch.float16 else 0, _ptr(src), _ptr(w), _ptr(s),
                               _ptr(b), K, N, clip), "vpq_quantize")
    return w, s, b
