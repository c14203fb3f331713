"""Seeded synthetic inputs for the w4g64 quantized-linear path.

Pure numpy, no GPU and no oracle: the same arrays feed the HIP kernels, the
CPU oracle and the benchmark.  bf16 values travel as uint16 bit patterns.

Distributions (the benchmark configurations' definition):
  q       uniform 0..15, 8 nibbles per uint32 along K, low nibble first
  scale   bf16(U(0.005, 0.02)) per 64-wide group along K
  bias    bf16(-8 * scale * (1 + 0.05 * z)),  z ~ N(0,1)
  x       bf16(N(0,1))
  LoRA    A[r,K], B[N,r] = bf16(N(0, 0.02))
"""
import numpy as np

GROUP = 64


def f32_to_bf16_bits(a):
    """Round-to-nearest-even fp32 -> bf16 bit pattern (uint16), vectorised."""
    x = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (x & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    rounding = np.uint32(0x7FFF) + ((x >> np.uint32(16)) & np.uint32(1))
    out = ((x + rounding) >> np.uint32(16)).astype(np.uint16)
    if nan.any():
        out[nan] = ((x[nan] >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16)
    return out


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def pack_nibbles(q):
    """q uint8 [N,K] in 0..15 -> uint32 [N,K/8], nibble i of word j = q[n, 8j+i]."""
    q = np.asarray(q, dtype=np.uint32)
    N, K = q.shape
    assert K % 8 == 0
    q = q.reshape(N, K // 8, 8)
    shifts = (np.arange(8, dtype=np.uint32) * np.uint32(4))
    return np.bitwise_or.reduce(q << shifts, axis=2).astype(np.uint32)


def unpack_nibbles(w, K):
    """Inverse of pack_nibbles -> uint8 [N,K]."""
    w = np.asarray(w, dtype=np.uint32)
    shifts = (np.arange(8, dtype=np.uint32) * np.uint32(4))
    q = (w[:, :, None] >> shifts) & np.uint32(0xF)
    return q.reshape(w.shape[0], K).astype(np.uint8)


def make_weight(N, K, seed):
    """-> (w uint32 [N,K/8], scales bf16 bits [N,K/64], biases bf16 bits [N,K/64])."""
    assert K % GROUP == 0
    rng = np.random.default_rng(seed)
    w = rng.integers(0, 2**32, size=(N, K // 8), dtype=np.uint32)  # uniform nibbles
    s32 = rng.uniform(0.005, 0.02, size=(N, K // GROUP)).astype(np.float32)
    s = f32_to_bf16_bits(s32)
    z = rng.standard_normal(size=(N, K // GROUP)).astype(np.float32)
    b32 = np.float32(-8.0) * bf16_bits_to_f32(s) * (np.float32(1.0) + np.float32(0.05) * z)
    b = f32_to_bf16_bits(b32)
    return w, s, b


def make_weight8(N, K, seed, group=GROUP):
    """8-bit twin: (w uint32 [N,K/4], one byte per value; scales, biases bf16 bits [N,K/group], group 64 or 32)."""
    assert K % group == 0
    rng = np.random.default_rng(seed)
    w = rng.integers(0, 2**32, size=(N, K // 4), dtype=np.uint32)  # uniform bytes
    s32 = rng.uniform(0.0003, 0.0012, size=(N, K // group)).astype(np.float32)
    s = f32_to_bf16_bits(s32)
    z = rng.standard_normal(size=(N, K // group)).astype(np.float32)
    b32 = np.float32(-128.0) * bf16_bits_to_f32(s) * (np.float32(1.0) + np.float32(0.05) * z)
    return w, s, f32_to_bf16_bits(b32)


def make_weight_g32(N, K, seed, q40=False):
    """group-32 twin: (w uint32 [N,K/8], scales, biases bf16 bits [N,K/32]); q40: biases = bf16(-8*scale) exactly,
    the redundant bias of a Q4_0 pack."""
    assert K % 32 == 0
    rng = np.random.default_rng(seed)
    w = rng.integers(0, 2**32, size=(N, K // 8), dtype=np.uint32)
    s = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(N, K // 32)).astype(np.float32))
    if q40:
        b32 = np.float32(-8.0) * bf16_bits_to_f32(s)        # exact: a power of two times a bf16
    else:
        z = rng.standard_normal(size=(N, K // 32)).astype(np.float32)
        b32 = np.float32(-8.0) * bf16_bits_to_f32(s) * (np.float32(1.0) + np.float32(0.05) * z)
    return w, s, f32_to_bf16_bits(b32)


def make_act(M, K, seed, std=1.0):
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits((rng.standard_normal(size=(M, K)) * std).astype(np.float32))


def make_lora(N, K, r, seed, std=0.02):
    rng = np.random.default_rng(seed)
    A = f32_to_bf16_bits((rng.standard_normal(size=(r, K)) * std).astype(np.float32))
    B = f32_to_bf16_bits((rng.standard_normal(size=(N, r)) * std).astype(np.float32))
    return A, B


def algorithmic_bytes(K, N, M):
    """Packed codes + scales + biases read once, x read once, y written once."""
    return N * K * 9 // 16 + 2 * M * K + 2 * M * N


def algorithmic_flops(K, N, M):
    return 2 * M * N * K
