"""ctypes front end of the CPU oracle (oracle/vpq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg -- never by the shipped package.  Arrays are numpy;
bf16/f16 values travel as uint16 bit patterns.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libvpq_oracle.so")
_lib = None

_u16p = ctypes.POINTER(ctypes.c_uint16)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)


def build(force=False):
    """Compile the C restatement with the committed Makefile."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libvpq_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.vpo_f32_to_bf16.restype = ctypes.c_uint16
        L.vpo_f32_to_bf16.argtypes = [ctypes.c_float]
        L.vpo_bf16_to_f32.restype = ctypes.c_float
        L.vpo_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.vpo_f32_to_f16.restype = ctypes.c_uint16
        L.vpo_f32_to_f16.argtypes = [ctypes.c_float]
        L.vpo_f16_to_f32.restype = ctypes.c_float
        L.vpo_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.vpo_weight_bytes.restype = ctypes.c_size_t
        L.vpo_scale_bytes.restype = ctypes.c_size_t
        L.vpo_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


def _c(a, dt):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dt)


def f32_to_bf16(a):
    """Element-wise RNE fp32 -> bf16 bits through the C helper."""
    a = _c(a, np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().vpo_f32_to_bf16_array(_p(a, _f32p), _p(out, _u16p), ctypes.c_size_t(a.size))
    return out


def f32_to_f16(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().vpo_f32_to_f16_array(_p(a, _f32p), _p(out, _u16p), ctypes.c_size_t(a.size))
    return out


def f16_to_f32(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().vpo_f16_to_f32_array(_p(bits, _u16p), _p(out, _f32p), ctypes.c_size_t(bits.size))
    return out


def bf16_to_f32(bits):
    """Exact widening of bf16 bits (numpy; no rounding involved)."""
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f16_to_bf16(bits):
    bits = _c(bits, np.uint16)
    out = np.empty_like(bits)
    lib().vpo_f16_to_bf16_array(_p(bits, _u16p), _p(out, _u16p), ctypes.c_size_t(bits.size))
    return out


def dequant_bf16(w, s, b, K, N):
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((N, K), dtype=np.uint16)
    lib().vpo_dequant_w4g64_bf16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(out, _u16p), K, N)
    return out


def dequant_f32(w, s, b, K, N):
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((N, K), dtype=np.float32)
    lib().vpo_dequant_w4g64_f32(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(out, _f32p), K, N)
    return out


def embed_gather(ids, w, s, b, H, vocab):
    """ids int32 [T] -> bf16 bits [T, H]: dequantized rows of the [vocab, H] table."""
    ids = _c(ids, np.int32)
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((ids.size, H), dtype=np.uint16)
    lib().vpo_embed_gather_w4g64_bf16(ids.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), _p(w, _u32p), _p(s, _u16p),
                                      _p(b, _u16p), _p(out, _u16p), H, ids.size, vocab)
    return out


def argmax(logits):
    """bf16 bits [rows, V] -> int32 [rows]: lowest index of the largest non-NaN logit (0 if there is none)."""
    logits = _c(logits, np.uint16)
    if logits.ndim == 1:
        logits = logits.reshape(1, -1)
    rows, V = logits.shape
    out = np.empty((rows,), dtype=np.int32)
    lib().vpo_argmax_bf16(_p(logits, _u16p), out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), V, rows)
    return out


def sample_exp(x):
    L = lib()
    L.vpo_sample_exp.restype = ctypes.c_float
    L.vpo_sample_exp.argtypes = [ctypes.c_float]
    return np.array([L.vpo_sample_exp(float(v)) for v in np.asarray(x, dtype=np.float32).ravel()], dtype=np.float32)


def sample_log(x):
    L = lib()
    L.vpo_sample_log.restype = ctypes.c_float
    L.vpo_sample_log.argtypes = [ctypes.c_float]
    return np.array([L.vpo_sample_log(float(v)) for v in np.asarray(x, dtype=np.float32).ravel()], dtype=np.float32)


def sample_hash_u01(x):
    L = lib()
    L.vpo_sample_hash_u01.restype = ctypes.c_float
    L.vpo_sample_hash_u01.argtypes = [ctypes.c_uint32]
    return np.array([L.vpo_sample_hash_u01(int(v)) for v in np.asarray(x, dtype=np.uint32).ravel()], dtype=np.float32)


def sample_topp(logits, seen, temp, top_p, seed, n_iter=24, rep=1.0, pres=0.0, top_k=0, min_p=0.0):
    """bf16 bits [V], uint8 [V] -> (token, cached weights bf16 bits [V], seen after the draw)."""
    L = lib()
    L.vpo_sample_topp_bf16.restype = ctypes.c_int32
    L.vpo_sample_topp_bf16.argtypes = [_u16p, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_uint32, _u16p,
                                       ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_float,
                                       ctypes.POINTER(ctypes.c_uint8)]
    logits = _c(logits, np.uint16)
    seen = np.array(seen, dtype=np.uint8, copy=True)
    ws = np.empty(logits.shape, dtype=np.uint16)
    tok = L.vpo_sample_topp_bf16(_p(logits, _u16p), logits.size, temp, top_p, seed, _p(ws, _u16p), n_iter, rep, pres, top_k,
                                 min_p, seen.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)))
    return int(tok), ws, seen


def sample_hist(logits, seen, temp, top_p, seed, n_slabs, rep=1.0, pres=0.0, top_k=0, min_p=0.0):
    """The sampler over n_slabs slabs with histogram thresholds: bf16 bits [V], uint8 [V] ->
    (token, cached weights bf16 bits [V], seen after the draw, weight threshold)."""
    L = lib()
    L.vpo_sample_hist_bf16.restype = ctypes.c_int32
    L.vpo_sample_hist_bf16.argtypes = [_u16p, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_uint32, _u16p,
                                       ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_float,
                                       ctypes.POINTER(ctypes.c_uint8), ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
    logits = _c(logits, np.uint16)
    seen = np.array(seen, dtype=np.uint8, copy=True)
    ws = np.empty(logits.shape, dtype=np.uint16)
    wt = ctypes.c_float(0.0)
    tok = L.vpo_sample_hist_bf16(_p(logits, _u16p), logits.size, temp, top_p, seed, _p(ws, _u16p), rep, pres, top_k, min_p,
                                 seen.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), n_slabs, ctypes.byref(wt))
    return int(tok), ws, seen, float(wt.value)


def qmv(w, s, b, x, K, N, M, residual=None):
    """-> (y64 [M,N] float64, y_bf16 [M,N] uint16); un-rounded-weight semantics."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    residual = _c(residual, np.uint16)
    y64 = np.empty((M, N), dtype=np.float64)
    yb = np.empty((M, N), dtype=np.uint16)
    lib().vpo_qmv_w4g64(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p),
                        _p(y64, _f64p), _p(yb, _u16p), K, N, M, _p(residual, _u16p))
    return y64, yb


def dequant_g32_bf16(w, s, b, K, N):
    """w4g32: scales, biases [N, K/32] -> bf16 bits [N, K]."""
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((N, K), dtype=np.uint16)
    lib().vpo_dequant_w4g32_bf16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(out, _u16p), K, N)
    return out


def qmv_g32(w, s, b, x, K, N, M, residual=None, scale_only=False):
    """w4g32 QMV -> (y64, y_bf16); scale_only: the Q4_0 form, b = -8*s, `b` not read (may be None)."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    residual = _c(residual, np.uint16)
    y64 = np.empty((M, N), dtype=np.float64)
    yb = np.empty((M, N), dtype=np.uint16)
    lib().vpo_qmv_w4g32(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p), _p(y64, _f64p), _p(yb, _u16p),
                        K, N, M, _p(residual, _u16p), 1 if scale_only else 0)
    return y64, yb


def qmv_factored(w, s, b, x, K, N, M):
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    y64 = np.empty((M, N), dtype=np.float64)
    lib().vpo_qmv_w4g64_factored(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p),
                                 _p(y64, _f64p), K, N, M)
    return y64


def lora_t(x, A, M, K, r, alpha):
    x, A = _c(x, np.uint16), _c(A, np.uint16)
    t = np.empty((M, r), dtype=np.uint16)
    lib().vpo_lora_t(_p(x, _u16p), _p(A, _u16p), _p(t, _u16p), M, K, r, ctypes.c_float(alpha))
    return t


def qmm(w, s, b, x, K, N, M, t=None, B=None, r=0):
    """-> (y64, y_bf16); bf16-rounded-weight semantics, optional fused LoRA term."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    t, B = _c(t, np.uint16), _c(B, np.uint16)
    y64 = np.empty((M, N), dtype=np.float64)
    yb = np.empty((M, N), dtype=np.uint16)
    lib().vpo_qmm_w4g64(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p),
                        _p(y64, _f64p), _p(yb, _u16p), K, N, M,
                        _p(t, _u16p), _p(B, _u16p), r)
    return y64, yb


def dequant_f16(w, s, b, K, N):
    """binary16 scales / biases -> binary16 bits [N, K]."""
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((N, K), dtype=np.uint16)
    lib().vpo_dequant_w4g64_f16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(out, _u16p), K, N)
    return out


def matmul_f16(w, s, b, x, K, N, M, rounded, residual=None):
    """binary16 elements -> (y64, y_f16 bits); rounded: the GEMM's binary16-rounded weights."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    residual = _c(residual, np.uint16)
    y64 = np.empty((M, N), dtype=np.float64)
    yh = np.empty((M, N), dtype=np.uint16)
    lib().vpo_matmul_w4g64_f16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p), _p(y64, _f64p), _p(yh, _u16p),
                               K, N, M, _p(residual, _u16p), 1 if rounded else 0)
    return y64, yh


def rmsnorm(x, norm_w, K, M, eps):
    """bf16 bits x [M,K], norm_w [K] -> bf16 bits [M,K]: x * rsqrt(mean(x^2) + eps) * norm_w."""
    x, norm_w = _c(x, np.uint16), _c(norm_w, np.uint16)
    out = np.empty((M, K), dtype=np.uint16)
    lib().vpo_rmsnorm_bf16(_p(x, _u16p), _p(norm_w, _u16p), _p(out, _u16p), K, M, ctypes.c_float(eps))
    return out


def lora_t_f16(x, A, M, K, r, alpha):
    """binary16 x [M,K], A [r,K] -> t [M,r] binary16 bits, two roundings."""
    x, A = _c(x, np.uint16), _c(A, np.uint16)
    t = np.empty((M, r), dtype=np.uint16)
    lib().vpo_lora_t_f16(_p(x, _u16p), _p(A, _u16p), _p(t, _u16p), M, K, r, ctypes.c_float(alpha))
    return t


def qmm_lora_f16(w, s, b, x, K, N, M, t, B, r):
    """binary16 elements, rounded weights, the adapter's t . B^T in the same accumulator -> (y64, y_f16 bits)."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    t, B = _c(t, np.uint16), _c(B, np.uint16)
    y64 = np.empty((M, N), dtype=np.float64)
    yh = np.empty((M, N), dtype=np.uint16)
    lib().vpo_qmm_lora_w4g64_f16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p), _p(y64, _f64p), _p(yh, _u16p),
                                 K, N, M, _p(t, _u16p), _p(B, _u16p), r)
    return y64, yh


_i32p = ctypes.POINTER(ctypes.c_int32)


def moe_sort_pairs(eid, top_k, E, block_rows, max_tiles):
    """-> (tile2e [max_tiles], srow [npad], sdst [npad], blocks in use); pairs of an expert in ascending order."""
    eid = _c(eid, np.int32)
    npad = max_tiles * block_rows
    t2e = np.empty(max_tiles, dtype=np.int32)
    srow = np.empty(npad, dtype=np.int32)
    sdst = np.empty(npad, dtype=np.int32)
    lib().vpo_moe_sort_pairs.restype = ctypes.c_int
    used = lib().vpo_moe_sort_pairs(_p(eid, _i32p), int(eid.size), top_k, E, block_rows, max_tiles,
                                    _p(t2e, _i32p), _p(srow, _i32p), _p(sdst, _i32p))
    return t2e, srow, sdst, used


def qmm_grouped(w, s, b, x, K, N, block_rows, tile2e, srow=None, sdst=None, rows_y=None, bits=4):
    """Grouped expert GEMM over sorted slots -> (y64, y_bf16).  With srow (gate|up) the outputs are
    [npad, N] in slot order; with sdst (down) they are [rows_y, N] in pair order (rows no slot
    writes stay zero)."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    tile2e, srow, sdst = _c(tile2e, np.int32), _c(srow, np.int32), _c(sdst, np.int32)
    npad = int(tile2e.size) * block_rows
    rows = npad if sdst is None else rows_y
    y64 = np.zeros((rows, N), dtype=np.float64)
    yb = np.zeros((rows, N), dtype=np.uint16)
    (lib().vpo_qmm_grouped_w4g64 if bits == 4 else lib().vpo_qmm_grouped_w8g64)(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p), _p(y64, _f64p),
                                _p(yb, _u16p), K, N, npad, block_rows, _p(tile2e, _i32p), _p(srow, _i32p),
                                _p(sdst, _i32p))
    return y64, yb


def interleave(a, b):
    """Rows of a and b (same shape, same dtype) alternating: out[2g] = a[g], out[2g+1] = b[g]."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    assert a.shape == b.shape and a.dtype == b.dtype
    out = np.empty((2 * a.shape[0],) + a.shape[1:], dtype=a.dtype)
    row_bytes = a.strides[0]
    lib().vpo_interleave_rows(a.ctypes.data_as(ctypes.c_void_p), b.ctypes.data_as(ctypes.c_void_p),
                              out.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(row_bytes),
                              ctypes.c_size_t(a.shape[0]))
    return out


def swiglu(y64):
    """[M,N] sums of an interleaved gate|up pack -> (out64 [M,N/2], out_bf16 [M,N/2])."""
    y64 = _c(y64, np.float64)
    M, N = y64.shape
    o64 = np.empty((M, N // 2), dtype=np.float64)
    ob = np.empty((M, N // 2), dtype=np.uint16)
    lib().vpo_swiglu_pairs(_p(y64, _f64p), _p(o64, _f64p), _p(ob, _u16p), M, N)
    return o64, ob


def geglu(y64):
    """[M,N] sums of an interleaved gate|up pack -> (out64 [M,N/2], out_bf16): gelu_tanh(gate) * up."""
    y64 = _c(y64, np.float64)
    M, N = y64.shape
    o64 = np.empty((M, N // 2), dtype=np.float64)
    ob = np.empty((M, N // 2), dtype=np.uint16)
    lib().vpo_geglu_pairs(_p(y64, _f64p), _p(o64, _f64p), _p(ob, _u16p), M, N)
    return o64, ob


def dequant8_bf16(w, s, b, K, N):
    """w8g64: w uint32 [N, K/4] (one byte per value) -> bf16 bits [N, K]."""
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((N, K), dtype=np.uint16)
    lib().vpo_dequant_w8g64_bf16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(out, _u16p), K, N)
    return out


def matmul8(w, s, b, x, K, N, M, rounded, group=64):
    """8-bit codes, y = x . W^T -> (y64, y_bf16); rounded=False: QMV semantics, True: GEMM semantics."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    y64 = np.empty((M, N), dtype=np.float64)
    yb = np.empty((M, N), dtype=np.uint16)
    lib().vpo_matmul_w8(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p), _p(y64, _f64p), _p(yb, _u16p),
                        K, N, M, 1 if rounded else 0, group)
    return y64, yb


def dequant8_g32(w, s, b, K, N):
    """w8g32: w uint32 [N, K/4], scales / biases [N, K/32] -> bf16 bits [N, K]."""
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((N, K), dtype=np.uint16)
    lib().vpo_dequant_w8_bf16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(out, _u16p), K, N, 32)
    return out


def dequant8_f16(w, s, b, K, N, group=64):
    """8-bit codes, binary16 scales / biases [N, K/group] -> binary16 bits [N, K]."""
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    out = np.empty((N, K), dtype=np.uint16)
    lib().vpo_dequant_w8_f16(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(out, _u16p), K, N, group)
    return out


def requant_w8_to_w4(w8, s8, b8, K, N):
    """8-bit group-64 pack -> 4-bit group-64 pack (codes u32 [N, K/8], scales, biases bf16 bits [N, K/64])."""
    w8, s8, b8 = _c(w8, np.uint32), _c(s8, np.uint16), _c(b8, np.uint16)
    w4 = np.empty((N, K // 8), dtype=np.uint32)
    s4 = np.empty((N, K // 64), dtype=np.uint16)
    b4 = np.empty((N, K // 64), dtype=np.uint16)
    lib().vpo_requant_w8_to_w4_g64(_p(w8, _u32p), _p(s8, _u16p), _p(b8, _u16p), _p(w4, _u32p), _p(s4, _u16p),
                                   _p(b4, _u16p), K, N)
    return w4, s4, b4


def quantize(wsrc, K, N, clip=1.0, bits=4, group=64):
    """fp32 [N,K] -> (codes u32 [N, K*bits/32], scales f16 bits [N, K/group], biases f16 bits)."""
    wsrc = _c(wsrc, np.float32)
    codes = np.empty((N, K * bits // 32), dtype=np.uint32)
    s = np.empty((N, K // group), dtype=np.uint16)
    b = np.empty((N, K // group), dtype=np.uint16)
    lib().vpo_quantize(_p(wsrc, _f32p), _p(codes, _u32p), _p(s, _u16p), _p(b, _u16p),
                       K, N, ctypes.c_float(clip), bits, group)
    return codes, s, b


def cpu_dequant_matmul(w, s, b, x, K, N, M, wdeq=None, xf=None):
    """The timed CPU baseline: dequant to fp32 [N,K] + fp32 dot, bf16 out."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    if wdeq is None:
        wdeq = np.empty((N, K), dtype=np.float32)
    if xf is None:
        xf = np.empty((M, K), dtype=np.float32)
    y = np.empty((M, N), dtype=np.uint16)
    lib().vpo_cpu_dequant_matmul(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p),
                                 _p(y, _u16p), _p(wdeq, _f32p), _p(xf, _f32p), K, N, M)
    return y


def cpu_dequant_f32(w, s, b, K, N, wdeq):
    """Stage 1 of the timed baseline alone: the pack expanded to fp32 [N,K]."""
    w, s, b = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16)
    lib().vpo_cpu_dequant_f32(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(wdeq, _f32p), K, N)
    return wdeq


def cpu_matmul_f32(wdeq, x, K, N, M, xf=None):
    """Stage 2 alone: fp32 dot of every row of the expanded matrix with every row of x, bf16 out."""
    x = _c(x, np.uint16)
    if xf is None:
        xf = np.empty((M, K), dtype=np.float32)
    y = np.empty((M, N), dtype=np.uint16)
    lib().vpo_cpu_matmul_f32(_p(wdeq, _f32p), _p(x, _u16p), _p(y, _u16p), _p(xf, _f32p), K, N, M)
    return y


def cpu_fused_qmv(w, s, b, x, K, N, M, xf=None):
    """The fused form: each weight expanded in a register and multiplied at once."""
    w, s, b, x = _c(w, np.uint32), _c(s, np.uint16), _c(b, np.uint16), _c(x, np.uint16)
    if xf is None:
        xf = np.empty((M, K), dtype=np.float32)
    y = np.empty((M, N), dtype=np.uint16)
    lib().vpo_cpu_fused_qmv(_p(w, _u32p), _p(s, _u16p), _p(b, _u16p), _p(x, _u16p), _p(y, _u16p), _p(xf, _f32p),
                            K, N, M)
    return y


def num_threads():
    return int(lib().vpo_num_threads())
