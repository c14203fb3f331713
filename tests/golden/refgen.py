"""The reference unit tests' own procedural input generators, restated in numpy.

The reference ships no data files for this path: each kernel test fills its
buffers from a small hash or LCG and computes its expectation in the test.
These functions reproduce those INPUTS bit for bit (uint32 wrap-around, fp32
arithmetic), so the same cases can be run here.  Citations are file:line in
the reference tree.

Nothing here imports the reference; it is arithmetic on integers.
"""
import numpy as np

U32 = np.uint32


def _frand(i):
    """tests/unit-tests/metal-lm/quant-gemv.cc:230-232:
    (float)((i * 2654435761u) >> 9 & 0x3ff) / 1023.0f - 0.5f"""
    i = np.asarray(i, dtype=np.uint64)
    h = (i * np.uint64(2654435761)) & np.uint64(0xFFFFFFFF)
    v = ((h >> np.uint64(9)) & np.uint64(0x3FF)).astype(np.float32)
    return v / np.float32(1023.0) - np.float32(0.5)


def knuth_qmv_case(N, K, group=64, extra_rows=1, kpad_to=512):
    """Inputs of metal_lm_smoke.qmv_w4g32_matches_cpu
    (tests/unit-tests/metal-lm/quant-gemv.cc:215-253), at the requested group.

    Returns fp32 scales/biases/x (the test casts them to its element type; the
    caller rounds to bf16), the nibble matrix q [N,K], the packed words
    [(N+extra_rows), K/8] including the test's garbage padding row(s), and x
    padded to a multiple of `kpad_to` with non-zero values."""
    groups = K // group
    o = np.arange(N, dtype=np.uint64)[:, None]
    g = np.arange(groups, dtype=np.uint64)[None, :]
    scales = np.float32(0.03) + np.float32(0.02) * _frand(o * np.uint64(991) + g)
    biases = np.float32(0.1) * _frand(o * np.uint64(131) + g * np.uint64(7) + np.uint64(5))
    oo = np.arange(N + extra_rows, dtype=np.uint64)[:, None]
    kk = np.arange(K, dtype=np.uint64)[None, :]
    idx = (oo * np.uint64(K) + kk) & np.uint64(0xFFFFFFFF)
    h = (idx * np.uint64(2654435761)) & np.uint64(0xFFFFFFFF)
    q_all = ((h >> np.uint64(13)) & np.uint64(0xF)).astype(np.uint32)
    shifts = (np.arange(8, dtype=np.uint32) * np.uint32(4))
    packed = np.bitwise_or.reduce(q_all.reshape(N + extra_rows, K // 8, 8) << shifts, axis=2).astype(np.uint32)
    kpad = ((K + kpad_to - 1) // kpad_to) * kpad_to
    k = np.arange(kpad, dtype=np.uint64)
    x = np.float32(0.5) + _frand(k * np.uint64(7) + np.uint64(3))
    return dict(scales=scales.astype(np.float32), biases=biases.astype(np.float32),
                q=q_all[:N].astype(np.uint8), packed=packed, x=x.astype(np.float32), kpad=kpad)


def _lcg_stream(seed, n):
    """r = r*1664525 + 1013904223 (uint32), n successive values after the seed
    (tests/unit-tests/minimax-h3-blocks.cc:126-129, 147-150)."""
    out = np.empty(n, dtype=np.uint32)
    r = (int(seed) | 1) & 0xFFFFFFFF
    # vectorised jump-free loop in chunks keeps this fast enough for ~1e6 values
    for i in range(n):
        r = (r * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = r
    return out


def lcg_act(n, seed):
    """make_act_ (tests/unit-tests/minimax-h3-blocks.cc:121-132): fp32 values
    ((float)(r >> 16) / 32768.0f - 1.0f) * 0.1f; the test rounds them to bf16 RNE."""
    r = _lcg_stream(seed, n)
    return ((r >> U32(16)).astype(np.float32) / np.float32(32768.0) - np.float32(1.0)) * np.float32(0.1)


def lcg_qweight(N, K, seed):
    """make_qw_ at 4 bits (tests/unit-tests/minimax-h3-blocks.cc:139-158): code
    bytes r >> 24, every scale 0.01, every bias -0.08 (fp32, rounded to bf16 by
    the caller).  -> (packed uint32 [N,K/8], scale, bias)."""
    nbytes = N * K // 2
    r = _lcg_stream(seed, nbytes)
    b = (r >> U32(24)).astype(np.uint8)
    packed = b.view(np.uint32).reshape(N, K // 8) if b.size % 4 == 0 else None
    return packed.copy(), np.float32(0.01), np.float32(-0.08)
