"""Pins for the CPU oracle (oracle/vpq_oracle.c).

The reference holds no golden files for this path and cannot run here, so the
oracle is pinned by (a) library routines it must reduce to (torch / numpy casts,
float64 matmul over an independently unpacked weight), (b) closed forms and
degenerate cases whose answer is fixed by the mathematics, and (c) the reference
tests' own procedural inputs with the tolerances those tests assert.  Each check
is chosen so that a plausible mistake -- wrong nibble order, a dropped bias
term, a transposed operand, a double rounding -- fails it.
"""
import numpy as np
import pytest
import torch

from tests.golden import refgen
from vpipe_amd import synth

G = 64


def np_unpack(w, K):
    """Independent unpack from the second layout statement of the reference
    (affine_qmm_mma.metal:98-99 / metal-compute-gemm-mma.cc:276-280): byte b of a
    row holds k=2b in its low nibble and k=2b+1 in its high nibble."""
    by = np.ascontiguousarray(w).view(np.uint8).reshape(w.shape[0], -1)
    q = np.empty((w.shape[0], K), dtype=np.uint8)
    q[:, 0::2] = by & 0x0F
    q[:, 1::2] = by >> 4
    return q


def np_dequant64(w, s, b, K):
    q = np_unpack(w, K).astype(np.float64)
    sf = synth.bf16_bits_to_f32(s).astype(np.float64)
    bf = synth.bf16_bits_to_f32(b).astype(np.float64)
    return np.repeat(sf, G, axis=1) * q + np.repeat(bf, G, axis=1)


# ---- conversions ------------------------------------------------------------

def test_bf16_rne_matches_torch_everywhere(oracle):
    # every bf16 value, its 2 neighbours' midpoints (ties) and points just off them
    hi = np.arange(0, 1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).ravel()
    f = bits.view(np.float32)
    finite = np.isfinite(f)
    got = oracle.f32_to_bf16(f[finite])
    want = torch.from_numpy(f[finite].copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    # the numpy twin used to generate inputs agrees too
    assert np.array_equal(synth.f32_to_bf16_bits(f[finite]), want)


def test_f16_conversions_match_numpy(oracle):
    all16 = np.arange(0, 1 << 16, dtype=np.uint16)
    want = all16.view(np.float16).astype(np.float32)
    got = oracle.f16_to_f32(all16)
    ok = np.isfinite(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    rng = np.random.default_rng(1)
    f = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 200000),
        want[ok],                                              # exactly representable
        (want[ok] * np.float32(1.0 + 2.0 ** -11)),             # near ties
        np.array([65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 0.0, -0.0], dtype=np.float32),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want16 = f.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16(f), want16)


# ---- layout + dequant -------------------------------------------------------

def test_dequant_matches_independent_numpy(oracle):
    N, K = 24, 256
    w, s, b = synth.make_weight(N, K, 11)
    want = np_dequant64(w, s, b, K)          # exact in float64: s*q has 12 significant bits
    got32 = oracle.dequant_f32(w, s, b, K, N)
    assert np.array_equal(got32, want.astype(np.float32))
    got16 = oracle.dequant_bf16(w, s, b, K, N)
    want16 = torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got16, want16)


def test_dequant_layout_known_answer(oracle):
    # one word 0x76543210 per row: nibble i == i, so W[n, 8j+i] = s*i + b
    N, K = 2, 64
    w = np.full((N, K // 8), 0x76543210, dtype=np.uint32)
    w[1, 3] = 0xFEDCBA98
    s = synth.f32_to_bf16_bits(np.array([[0.5], [0.25]], dtype=np.float32))
    b = synth.f32_to_bf16_bits(np.array([[-1.0], [2.0]], dtype=np.float32))
    d = oracle.dequant_f32(w, s, b, K, N)
    assert np.array_equal(d[0, :8], 0.5 * np.arange(8) - 1.0)
    assert np.array_equal(d[1, 24:32], 0.25 * np.arange(8, 16) + 2.0)
    assert np.array_equal(d[1, :8], 0.25 * np.arange(8) + 2.0)


def test_pack_unpack_roundtrip_and_sizes(oracle):
    rng = np.random.default_rng(5)
    q = rng.integers(0, 16, size=(7, 128), dtype=np.uint8)
    w = synth.pack_nibbles(q)
    assert np.array_equal(synth.unpack_nibbles(w, 128), q)
    assert np.array_equal(np_unpack(w, 128), q)
    # generative-models/quantize/affine-quantizer.h:37-40
    assert oracle.lib().vpo_weight_bytes(96, 256) == 96 * 32 * 4
    assert oracle.lib().vpo_scale_bytes(96, 256) == 96 * 4 * 2


# ---- QMV / QMM: what the mathematics fixes ----------------------------------

@pytest.mark.parametrize("M", [1, 3])
def test_one_hot_activation_reads_back_the_weight(oracle, M):
    # x = e_k  =>  y[n] = W[n,k]; pushes layout and dequant through the full matmul
    N, K = 16, 192
    w, s, b = synth.make_weight(N, K, 21)
    d32 = oracle.dequant_f32(w, s, b, K, N)
    d16 = oracle.dequant_bf16(w, s, b, K, N)
    for k in [0, 1, 7, 8, 63, 64, 130, K - 1]:
        x = np.zeros((M, K), dtype=np.float32)
        x[M - 1, k] = 1.0
        xb = synth.f32_to_bf16_bits(x)
        y64, yb = oracle.qmv(w, s, b, xb, K, N, M)
        assert np.array_equal(y64[M - 1], d32[:, k].astype(np.float64))
        assert np.array_equal(yb[M - 1], synth.f32_to_bf16_bits(d32[:, k]))
        assert not y64[: M - 1].any()
        z64, zb = oracle.qmm(w, s, b, xb, K, N, M)
        assert np.array_equal(zb[M - 1], d16[:, k])          # QMM sees the bf16-rounded weight
        assert np.array_equal(z64[M - 1], synth.bf16_bits_to_f32(d16[:, k]).astype(np.float64))


def test_degenerate_quantizers(oracle):
    N, K, M = 8, 256, 2
    rng = np.random.default_rng(3)
    x = synth.make_act(M, K, 4)
    xf = synth.bf16_bits_to_f32(x).astype(np.float64)
    w, s, b = synth.make_weight(N, K, 5)
    # all codes zero: y = sum_g b_g * sum_{k in g} x_k
    w0 = np.zeros_like(w)
    y64, _ = oracle.qmv(w0, s, b, x, K, N, M)
    want = xf.reshape(M, K // G, G).sum(axis=2) @ synth.bf16_bits_to_f32(b).astype(np.float64).T
    assert np.allclose(y64, want, rtol=1e-12, atol=1e-12)
    # q = 8 everywhere with b = -8 s: every weight is exactly 0
    w8 = np.full_like(w, 0x88888888)
    b8 = synth.f32_to_bf16_bits(-8.0 * synth.bf16_bits_to_f32(s))
    for fn in (oracle.qmv, oracle.qmm):
        y64, yb = fn(w8, s, b8, x, K, N, M)
        assert not y64.any() and not yb.any()
    # scale 0: bias only, whatever the codes
    s0 = np.zeros_like(s)
    y64a, _ = oracle.qmv(w, s0, b, x, K, N, M)
    assert np.allclose(y64a, want, rtol=1e-12, atol=1e-12)
    del rng


@pytest.mark.parametrize("K,N,M", [(64, 5, 1), (512, 33, 4), (4096, 32, 2), (5120, 16, 16)])
def test_matmul_matches_float64_numpy(oracle, K, N, M):
    w, s, b = synth.make_weight(N, K, 100 + K)
    x = synth.make_act(M, K, 200 + K)
    xf = synth.bf16_bits_to_f32(x).astype(np.float64)
    W = np_dequant64(w, s, b, K)                              # un-rounded weight, exact
    W32 = W.astype(np.float32).astype(np.float64)             # the fp32 the QMV path holds
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    assert np.allclose(y64, xf @ W32.T, rtol=1e-11, atol=1e-9)
    # factored form (scale*sum(x q) + bias*sum(x)) is the same number up to fp32(s*q+b) rounding
    yf = oracle.qmv_factored(w, s, b, x, K, N, M)
    assert np.allclose(yf, xf @ W.T, rtol=1e-11, atol=1e-9)
    scale = np.sqrt((y64 ** 2).mean())
    assert np.abs(yf - y64).max() < 2e-6 * scale + 1e-6
    # QMM path: bf16-rounded weight
    Wb = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(W.astype(np.float32))).astype(np.float64)
    z64, zb = oracle.qmm(w, s, b, x, K, N, M)
    assert np.allclose(z64, xf @ Wb.T, rtol=1e-11, atol=1e-9)
    assert np.array_equal(zb, synth.f32_to_bf16_bits(z64.astype(np.float32)))
    assert np.array_equal(yb, synth.f32_to_bf16_bits(y64.astype(np.float32)))


def test_linearity_in_x(oracle):
    K, N = 512, 12
    w, s, b = synth.make_weight(N, K, 31)
    # activations on a coarse grid so x1+x2 is exact in bf16
    rng = np.random.default_rng(32)
    x1 = (rng.integers(-64, 64, size=(1, K)) / 32.0).astype(np.float32)
    x2 = (rng.integers(-64, 64, size=(1, K)) / 32.0).astype(np.float32)
    ya, _ = oracle.qmv(w, s, b, synth.f32_to_bf16_bits(x1), K, N, 1)
    yb_, _ = oracle.qmv(w, s, b, synth.f32_to_bf16_bits(x2), K, N, 1)
    yc, _ = oracle.qmv(w, s, b, synth.f32_to_bf16_bits(x1 + x2), K, N, 1)
    assert np.allclose(ya + yb_, yc, rtol=1e-12, atol=1e-10)


def test_residual_add_rounds_twice(oracle):
    # affine_qmv.metal:264-266: v = (T)result; v += residual  (element-type add)
    K, N = 128, 9
    w, s, b = synth.make_weight(N, K, 41)
    x = synth.make_act(1, K, 42)
    res = synth.make_act(1, N, 43)
    y64, yb = oracle.qmv(w, s, b, x, K, N, 1)
    _, yr = oracle.qmv(w, s, b, x, K, N, 1, residual=res)
    a = torch.from_numpy(yb.view(np.int16)).view(torch.bfloat16)
    r = torch.from_numpy(res.view(np.int16)).view(torch.bfloat16)
    want = (a + r).view(torch.int16).numpy().view(np.uint16)   # torch adds bf16 in fp32 and rounds
    assert np.array_equal(yr, want)


# ---- the reference tests' own inputs and tolerances -------------------------

def test_reference_qmv_case_tail_and_padding(oracle):
    """metal_lm_smoke.qmv_w4g32_matches_cpu (tests/unit-tests/metal-lm/quant-gemv.cc:207-300)
    at group 64: N=16, K=3840 (not a multiple of 512), x padded to 4096 with
    non-zero values, one garbage weight row appended.  The oracle must (a) ignore
    everything past K and past row N and (b) agree with an independent float64
    evaluation within the test's own tolerance 0.03 (it agrees to 1e-6)."""
    N, K = 16, 3840
    c = refgen.knuth_qmv_case(N, K, group=64)
    s = synth.f32_to_bf16_bits(c["scales"])
    b = synth.f32_to_bf16_bits(c["biases"])
    x = synth.f32_to_bf16_bits(c["x"])[None, :]                 # [1, 4096]
    w_all = c["packed"]                                          # [17, K/8]
    assert np.array_equal(np_unpack(w_all[:N], K), c["q"])
    y64, _ = oracle.qmv(w_all[:N], s, b, x[:, :K], K, N, 1)
    # CPU loop of the test: acc(double) += x[k] * (s*q + b)
    W32 = (synth.bf16_bits_to_f32(s).repeat(G, axis=1) * c["q"].astype(np.float32)
           + synth.bf16_bits_to_f32(b).repeat(G, axis=1)).astype(np.float32)
    ref = (synth.bf16_bits_to_f32(x[0, :K]).astype(np.float64)[None, :] * W32.astype(np.float64)).sum(axis=1)
    maxrel = np.abs(y64[0] - ref) / (np.abs(ref) + 1e-2)
    assert maxrel.max() < 1e-9
    # poisoned tail: feeding the padded x with K=4096 against garbage gives a different answer
    assert np.abs(ref).min() > 1.0                              # all-positive x: no cancellation, as the test notes


def test_reference_lcg_weight_case(oracle):
    """make_act_/make_qw_ inputs (tests/unit-tests/minimax-h3-blocks.cc:121-158):
    s = 0.01, b = -0.08 everywhere, LCG code bytes and activations."""
    N, K, M = 32, 256, 5
    packed, s0, b0 = refgen.lcg_qweight(N, K, 0x1234)
    s = np.full((N, K // G), synth.f32_to_bf16_bits(np.float32(s0)), dtype=np.uint16)
    b = np.full((N, K // G), synth.f32_to_bf16_bits(np.float32(b0)), dtype=np.uint16)
    x = synth.f32_to_bf16_bits(refgen.lcg_act(M * K, 21).reshape(M, K))
    q = np_unpack(packed, K).astype(np.float64)
    sf = float(synth.bf16_bits_to_f32(s[0, 0]))
    bf = float(synth.bf16_bits_to_f32(b[0, 0]))
    Wb = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits((sf * q + bf).astype(np.float32))).astype(np.float64)
    want = synth.bf16_bits_to_f32(x).astype(np.float64) @ Wb.T
    z64, zb = oracle.qmm(packed, s, b, x, K, N, M)
    assert np.allclose(z64, want, rtol=1e-12, atol=1e-12)
    rel_l2 = np.sqrt(((synth.bf16_bits_to_f32(zb) - want) ** 2).sum() / (want ** 2).sum())
    assert rel_l2 < 3e-2                                         # metal-compute-gemm-mma.cc:490 bar
    assert rel_l2 < 3e-3                                         # what one bf16 store actually costs


# ---- LoRA --------------------------------------------------------------------

def test_lora_matches_float64_and_reference_tolerance(oracle):
    """minimax_h3_blocks.lora_accumulate_matches_reference
    (tests/unit-tests/minimax-h3-blocks.cc:1162-1296) at a reduced shape: same
    generators (seeds 21/29/31), strength 0.625, rel-L2 < 5e-3 vs float64 and a
    delta that is a real part of the output."""
    M, N, K, R = 24, 48, 512, 64
    scale = 0.625
    x = synth.f32_to_bf16_bits(refgen.lcg_act(M * K, 21).reshape(M, K))
    A = synth.f32_to_bf16_bits(refgen.lcg_act(R * K, 29).reshape(R, K))
    B = synth.f32_to_bf16_bits(refgen.lcg_act(N * R, 31).reshape(N, R))
    w, s, b = synth.make_weight(N, K, 23)
    # shrink the base so the adapter is a visible part of the output, as in the reference case
    s[:] = synth.f32_to_bf16_bits(np.float32(0.0005))
    b[:] = synth.f32_to_bf16_bits(np.float32(-0.004))
    t = oracle.lora_t(x, A, M, K, R, scale)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M, t=t, B=B, r=R)
    xf = synth.bf16_bits_to_f32(x).astype(np.float64)
    Wb = synth.bf16_bits_to_f32(oracle.dequant_bf16(w, s, b, K, N)).astype(np.float64)
    base = xf @ Wb.T
    d = scale * (xf @ synth.bf16_bits_to_f32(A).astype(np.float64).T) @ synth.bf16_bits_to_f32(B).astype(np.float64).T
    want = base + d
    got = synth.bf16_bits_to_f32(yb).astype(np.float64)
    rl2 = np.sqrt(((got - want) ** 2).sum() / (want ** 2).sum())
    assert rl2 < 5e-3
    assert np.sqrt((d ** 2).sum() / (want ** 2).sum()) > 0.05
    # t itself: two roundings, bf16(scale * bf16(x.A^T))
    tt = (xf @ synth.bf16_bits_to_f32(A).astype(np.float64).T).astype(np.float32)
    once = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(tt))
    assert np.array_equal(t, synth.f32_to_bf16_bits(once * np.float32(scale)))
    # an adapter whose t is zero leaves the base untouched, bit for bit
    _, y0 = oracle.qmm(w, s, b, x, K, N, M)
    _, y1 = oracle.qmm(w, s, b, x, K, N, M, t=np.zeros_like(t), B=B, r=R)
    assert np.array_equal(y0, y1)


# ---- the packer ----------------------------------------------------------------

def test_quantize_recovers_on_grid_weights_exactly(oracle):
    # a weight already of the form s*q + b with f16-exact s, b and every group
    # spanning 0..15 must come back with the same codes, scale and bias
    N, K = 6, 256
    rng = np.random.default_rng(7)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    q.reshape(N, K // G, G)[:, :, 0] = 0
    q.reshape(N, K // G, G)[:, :, 1] = 15
    s = (rng.integers(1, 64, size=(N, K // G)) / 1024.0).astype(np.float32)      # f16-exact
    b = (-rng.integers(0, 256, size=(N, K // G)) / 256.0).astype(np.float32)
    W = (np.repeat(s, G, axis=1) * q + np.repeat(b, G, axis=1)).astype(np.float32)
    codes, sf16, bf16_ = oracle.quantize(W, K, N)
    assert np.array_equal(synth.unpack_nibbles(codes, K), q)
    assert np.array_equal(sf16.view(np.float16).astype(np.float32), s)
    assert np.array_equal(bf16_.view(np.float16).astype(np.float32), b)


def test_quantize_roundtrip_bounds_of_the_reference(oracle):
    """model_quantize_roundtrip.affine_writer_reader_dequant
    (tests/unit-tests/model-quantize-roundtrip.cc:84-164): N=96, K=256 ramp+ripple
    source; 4-bit rel-L2 < 0.20; byte sizes."""
    N, K = 96, 256
    n = np.arange(N)[:, None]
    k = np.arange(K)[None, :]
    v = 0.4 * np.sin(0.05 * k + 0.3 * n) + 0.1 * np.cos(0.7 * k) + 0.002 * (k - K / 2)
    src = v.astype(np.float16).astype(np.float32)
    codes, sf16, bf16_ = oracle.quantize(src, K, N)
    assert codes.nbytes == 96 * 32 * 4 and sf16.nbytes == 96 * 4 * 2
    sb = oracle.f16_to_bf16(sf16)
    bb = oracle.f16_to_bf16(bf16_)
    deq = synth.bf16_bits_to_f32(oracle.dequant_bf16(codes, sb, bb, K, N)).astype(np.float64)
    err = np.sqrt(((deq - src) ** 2).sum() / (src.astype(np.float64) ** 2).sum())
    assert err < 0.20
    # numpy re-derivation of the code assignment (round half away from zero)
    g = src.reshape(N, K // G, G)
    mn = g.min(axis=2, keepdims=True)
    mx = g.max(axis=2, keepdims=True)
    sc = ((mx - mn) / np.float32(15.0)).astype(np.float32)
    inv = np.where(sc > 0, np.float32(1.0) / sc, np.float32(0.0)).astype(np.float32)
    t = ((g - mn) * inv).astype(np.float32)
    qn = np.clip(np.floor(t + np.float32(0.5)), 0, 15).astype(np.uint8).reshape(N, K)
    assert np.array_equal(synth.unpack_nibbles(codes, K), qn)
    assert np.array_equal(sf16, sc.astype(np.float16).view(np.uint16).reshape(N, K // G))


@pytest.mark.parametrize("bits,group", [(4, 32), (8, 64), (8, 32)])
def test_quantize_other_widths_and_groups(oracle, bits, group):
    """affine_quant_impl<BITS, GROUP> (gpu-kernels/metal/quant/affine_dequant.metal:243-301) at the other three formats:
    on-grid weights (every group spanning 0..2^bits - 1, f16-exact scale and bias) come back with their codes, scale
    and bias -- which pins the word layout (values per word, words per group and row); a smooth source against a numpy
    re-derivation with the tie rule written out; and the format's expansion of the result stays within half a step."""
    qmax = (1 << bits) - 1
    vpw = 32 // bits
    N, K = 5, 256
    rng = np.random.default_rng(70 + bits + group)
    q = rng.integers(0, qmax + 1, size=(N, K), dtype=np.uint32)
    q.reshape(N, K // group, group)[:, :, 0] = 0
    q.reshape(N, K // group, group)[:, :, 1] = qmax
    s = (rng.integers(1, 16, size=(N, K // group)) / 1024.0).astype(np.float32)
    b = (-rng.integers(0, 256, size=(N, K // group)) / 256.0).astype(np.float32)
    W = (np.repeat(s, group, axis=1) * q + np.repeat(b, group, axis=1)).astype(np.float32)
    codes, sf16, bf16_ = oracle.quantize(W, K, N, bits=bits, group=group)
    assert codes.shape == (N, K // vpw)
    got = ((codes[:, :, None] >> (bits * np.arange(vpw, dtype=np.uint32))) & qmax).reshape(N, K)
    assert np.array_equal(got, q)
    assert np.array_equal(sf16.view(np.float16).astype(np.float32), s)
    assert np.array_equal(bf16_.view(np.float16).astype(np.float32), b)
    # smooth source, numpy re-derivation
    N, K = 24, 256
    n = np.arange(N)[:, None]
    k = np.arange(K)[None, :]
    src = (0.4 * np.sin(0.05 * k + 0.3 * n) + 0.1 * np.cos(0.7 * k) + 0.002 * (k - K / 2)).astype(np.float16).astype(np.float32)
    codes, sf16, bf16_ = oracle.quantize(src, K, N, bits=bits, group=group)
    g = src.reshape(N, K // group, group)
    mn, mx = g.min(axis=2, keepdims=True), g.max(axis=2, keepdims=True)
    sc = ((mx - mn) / np.float32(qmax)).astype(np.float32)
    inv = np.where(sc > 0, np.float32(1.0) / sc, np.float32(0.0)).astype(np.float32)
    t = ((g - mn) * inv).astype(np.float32)
    fl = np.floor(t)
    qn = np.clip(np.where(t - fl >= np.float32(0.5), fl + 1, fl), 0, qmax).astype(np.uint32).reshape(N, K)
    got = ((codes[:, :, None] >> (bits * np.arange(vpw, dtype=np.uint32))) & qmax).reshape(N, K)
    assert np.array_equal(got, qn)
    assert np.array_equal(sf16, sc.astype(np.float16).view(np.uint16).reshape(N, K // group))
    assert np.array_equal(bf16_, mn.astype(np.float16).view(np.uint16).reshape(N, K // group))
    recon = mn + sc * qn.reshape(N, K // group, group)
    assert (np.abs(recon - g) <= 0.5 * sc * (1 + 1e-5) + 1e-7).all()


def test_cpu_baseline_is_the_same_algorithm(oracle):
    K, N, M = 512, 40, 3
    w, s, b = synth.make_weight(N, K, 51)
    x = synth.make_act(M, K, 52)
    y = oracle.cpu_dequant_matmul(w, s, b, x, K, N, M)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    got = synth.bf16_bits_to_f32(y).astype(np.float64)
    assert np.abs(got - y64).max() <= 2.0 ** -7 * np.abs(y64).max()
    assert (y != yb).mean() < 0.05


# ---- fused gate|up + SwiGLU -------------------------------------------------------

def test_swiglu_expression_against_scipy_and_identities(oracle):
    from scipy.special import expit
    rng = np.random.default_rng(5)
    y = rng.normal(size=(4, 64)) * 4.0
    y[0, :8] = [0.0, 3.0, 50.0, 2.0, -50.0, 2.0, 1.0, 0.0]     # gate 0, +large, -large; up 0
    o64, ob = oracle.swiglu(y)
    gate, up = y[:, 0::2], y[:, 1::2]
    assert np.allclose(o64, gate * expit(gate) * up, rtol=1e-14, atol=1e-300)
    # silu(0) = 0; silu(v) -> v for large v; silu(-large) -> 0; up = 0 -> 0
    assert o64[0, 0] == 0.0 and abs(o64[0, 1] - 100.0) < 1e-12 and abs(o64[0, 2]) < 1e-18 and o64[0, 3] == 0.0
    # silu(v) - silu(-v) == v: pairs (v, 1) and (-v, 1)
    v = rng.normal(size=32) * 3
    pair = np.stack([np.stack([v, np.ones_like(v)], 1).ravel(), np.stack([-v, np.ones_like(v)], 1).ravel()])
    o2, _ = oracle.swiglu(pair)
    assert np.allclose(o2[0] - o2[1], v, rtol=0, atol=1e-15)
    # gate and up are not interchangeable: the even column is the gate
    swapped = y.reshape(4, 32, 2)[:, :, ::-1].reshape(4, 64)
    assert not np.allclose(oracle.swiglu(swapped)[0], o64)
    assert np.array_equal(ob, oracle.f32_to_bf16(o64.astype(np.float32)))


def test_interleave_is_row_alternation(oracle):
    rng = np.random.default_rng(6)
    for dt, cols in ((np.uint32, 24), (np.uint16, 3), (np.uint16, 1)):
        a = rng.integers(0, 60000, size=(7, cols)).astype(dt)
        b = rng.integers(0, 60000, size=(7, cols)).astype(dt)
        out = oracle.interleave(a, b)
        assert np.array_equal(out, np.stack([a, b], axis=1).reshape(14, cols))
        assert np.array_equal(out[0::2], a) and np.array_equal(out[1::2], b)


def test_fused_pack_equals_two_separate_packs(oracle):
    # the interleave is a permutation, not a different computation
    # (tests/unit-tests/minimax-h3-blocks.cc:807-846): the fused pack's sums are the two packs' sums
    K, F, M = 512, 24, 3
    gw, gs, gb = synth.make_weight(F, K, 41)
    uw, us, ub = synth.make_weight(F, K, 42)
    x = synth.make_act(M, K, 43)
    w, s, b = oracle.interleave(gw, uw), oracle.interleave(gs, us), oracle.interleave(gb, ub)
    for fn in (oracle.qmv, oracle.qmm):
        y, _ = fn(w, s, b, x, K, 2 * F, M)
        g, _ = fn(gw, gs, gb, x, K, F, M)
        u, _ = fn(uw, us, ub, x, K, F, M)
        assert np.array_equal(y[:, 0::2], g) and np.array_equal(y[:, 1::2], u)
        o64, _ = oracle.swiglu(y)
        assert np.allclose(o64, g / (1.0 + np.exp(-g)) * u, rtol=1e-14)


def test_embed_gather_is_row_selection_of_the_dense_table(oracle):
    vocab, H = 37, 192
    w, s, b = synth.make_weight(vocab, H, 90)
    dense = oracle.dequant_bf16(w, s, b, H, vocab)
    ids = np.array([0, 36, 5, 5, 17, -1, 37, 2], dtype=np.int32)
    got = oracle.embed_gather(ids, w, s, b, H, vocab)
    ok = (ids >= 0) & (ids < vocab)
    assert np.array_equal(got[ok], dense[ids[ok]])
    assert not got[~ok].any()


def test_geglu_expression_against_torch_gelu_tanh(oracle):
    rng = np.random.default_rng(8)
    y = rng.normal(size=(3, 40)) * 3.0
    y[0, :6] = [0.0, 2.0, 30.0, 2.0, -30.0, 2.0]
    o64, ob = oracle.geglu(y)
    gate, up = torch.from_numpy(y[:, 0::2].copy()), torch.from_numpy(y[:, 1::2].copy())
    want = (torch.nn.functional.gelu(gate, approximate="tanh") * up).numpy()
    assert np.allclose(o64, want, rtol=1e-12, atol=1e-300)
    assert o64[0, 0] == 0.0 and abs(o64[0, 1] - 60.0) < 1e-9 and abs(o64[0, 2]) < 1e-12
    # not the sigmoid gate: the two activations differ by a few percent at |g| ~ 1
    assert not np.allclose(o64, oracle.swiglu(y)[0], rtol=1e-2)
    assert np.array_equal(ob, oracle.f32_to_bf16(o64.astype(np.float32)))


# ---- 8-bit twin (w8g64) ---------------------------------------------------------------

def test_w8_oracle_against_numpy_from_the_byte_view(oracle):
    # one byte per value, little-endian within the word (affine_dequant.metal:60-67): the byte view
    # of the words IS the code matrix
    N, K, M = 9, 192, 3
    w, s, b = synth.make_weight8(N, K, 70)
    q = w.view(np.uint8).reshape(N, K).astype(np.float64)
    sf = synth.bf16_bits_to_f32(s).astype(np.float64).repeat(64, axis=1)
    bf = synth.bf16_bits_to_f32(b).astype(np.float64).repeat(64, axis=1)
    W = sf * q + bf                                    # exact in float64
    got = oracle.dequant8_bf16(w, s, b, K, N)
    assert np.array_equal(got, synth.f32_to_bf16_bits(W.astype(np.float32)))
    x = synth.make_act(M, K, 71)
    xf = synth.bf16_bits_to_f32(x).astype(np.float64)
    y_qmv, _ = oracle.matmul8(w, s, b, x, K, N, M, rounded=False)
    Wf32 = (sf.astype(np.float32) * q.astype(np.float32) + bf.astype(np.float32)).astype(np.float64)
    assert np.allclose(y_qmv, xf @ Wf32.T, rtol=1e-12, atol=1e-12)
    y_qmm, _ = oracle.matmul8(w, s, b, x, K, N, M, rounded=True)
    Wb = synth.bf16_bits_to_f32(got).astype(np.float64)
    assert np.allclose(y_qmm, xf @ Wb.T, rtol=1e-12, atol=1e-12)
    # one-hot activation reads back one (rounded / unrounded) weight column
    e = np.zeros((1, K), dtype=np.float32); e[0, 77] = 1.0
    y1, _ = oracle.matmul8(w, s, b, synth.f32_to_bf16_bits(e), K, N, 1, rounded=True)
    assert np.array_equal(y1[0], Wb[:, 77])
    # byte order: code 0x04030201 is q = 1, 2, 3, 4
    w1 = np.full((1, 16), 0x04030201, dtype=np.uint32)
    one = synth.f32_to_bf16_bits(np.ones((1, 1), dtype=np.float32))
    zero = np.zeros((1, 1), dtype=np.uint16)
    assert list(synth.bf16_bits_to_f32(oracle.dequant8_bf16(w1, one, zero, 64, 1))[0, :4]) == [1.0, 2.0, 3.0, 4.0]



def test_argmax_is_the_first_maximum(oracle):
    # pinned against numpy's argmax (first occurrence of the maximum) on NaN-free rows with many
    # ties, and against a plain left-to-right scan written out here for rows with NaN and -inf
    rng = np.random.default_rng(77)
    vals = rng.integers(-40, 40, size=(6, 5000)).astype(np.float32) / 4.0      # bf16-exact, heavy ties
    bits = synth.f32_to_bf16_bits(vals)
    assert np.array_equal(oracle.argmax(bits), np.argmax(synth.bf16_bits_to_f32(bits), axis=1).astype(np.int32))
    nan, ninf, pinf = 0x7FC0, 0xFF80, 0x7F80
    one, two = 0x3F80, 0x4000
    cases = [([nan, one, two, two], 2), ([ninf, ninf, ninf], 0), ([nan, ninf, ninf], 1), ([nan, nan], 0),
             ([two, nan, pinf, pinf], 2), ([one], 0), ([nan, 0x8000, 0x0000], 1)]      # -0.0 == +0.0: the first
    for row, want in cases:
        best, bi = -np.inf, -1
        for i, h in enumerate(row):
            v = float(synth.bf16_bits_to_f32(np.array([h], dtype=np.uint16))[0])
            if v > best or (bi < 0 and v == best):
                best, bi = v, i
        assert max(bi, 0) == want
        assert int(oracle.argmax(np.array(row, dtype=np.uint16))[0]) == want


def test_group32_twins_against_closed_forms_and_the_group64_oracle(oracle):
    # (1) a group-64 pack rewritten with every scale and bias repeated twice is a group-32 pack of
    # the same weight: both oracles must give the same bits; (2) the dense expansion against the
    # closed form in numpy; (3) the QMV against a float64 matmul of that expansion; (4) the Q4_0
    # form (bias never read) equals the affine form whose stored bias is -8*scale.
    N, K, M = 24, 256, 3
    w, s64, b64 = synth.make_weight(N, K, 910)
    x = synth.make_act(M, K, 911)
    s32, b32 = np.repeat(s64, 2, axis=1), np.repeat(b64, 2, axis=1)
    assert np.array_equal(oracle.dequant_g32_bf16(w, s32, b32, K, N), oracle.dequant_bf16(w, s64, b64, K, N))
    y64a, yba = oracle.qmv_g32(w, s32, b32, x, K, N, M)
    y64b, ybb = oracle.qmv(w, s64, b64, x, K, N, M)
    assert np.array_equal(y64a, y64b) and np.array_equal(yba, ybb)

    w, s, b = synth.make_weight_g32(N, K, 912)
    q = synth.unpack_nibbles(w, K).astype(np.float32)
    sf = np.repeat(synth.bf16_bits_to_f32(s), 32, axis=1)
    bf = np.repeat(synth.bf16_bits_to_f32(b), 32, axis=1)
    dense32 = (sf * q).astype(np.float32) + bf            # s*q exact in fp32, one rounding in the add
    assert np.array_equal(oracle.dequant_g32_bf16(w, s, b, K, N), synth.f32_to_bf16_bits(dense32))
    y64, _ = oracle.qmv_g32(w, s, b, x, K, N, M)
    want = synth.bf16_bits_to_f32(x).astype(np.float64) @ dense32.astype(np.float64).T
    assert np.allclose(y64, want, rtol=1e-12, atol=1e-9)

    w, s, b = synth.make_weight_g32(N, K, 913, q40=True)
    ya, yb_a = oracle.qmv_g32(w, s, b, x, K, N, M)
    yq, yb_q = oracle.qmv_g32(w, s, None, x, K, N, M, scale_only=True)
    assert np.array_equal(ya, yq) and np.array_equal(yb_a, yb_q)
    res = synth.make_act(M, N, 914)
    _, with_res = oracle.qmv_g32(w, s, None, x, K, N, M, residual=res, scale_only=True)
    assert np.array_equal(with_res, synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(yb_q) + synth.bf16_bits_to_f32(res)))


def test_moe_sort_and_grouped_gemm_reduce_to_the_per_pair_statement(oracle):
    """The expert sort against numpy's stable argsort (an independent statement of a counting sort) and
    its invariants; the grouped GEMMs against the plain oracle GEMM of every pair on its expert's
    slab (the reference's claim for them: "token-exact with the per-pair paths",
    gpu-kernels/metal/quant/affine_qmm_steel.metal:1027-1031)."""
    E, top_k, T, B = 5, 2, 9, 4
    rng = np.random.default_rng(31)
    eid = rng.integers(0, E, size=T * top_k, dtype=np.int32)
    eid[3] = 4
    eid[eid == 2] = 1                                   # expert 2 gets nothing
    npair = eid.size
    max_tiles = (npair + B - 1) // B + E
    t2e, srow, sdst, used = oracle.moe_sort_pairs(eid, top_k, E, B, max_tiles)
    hist = np.bincount(eid, minlength=E)
    blocks = (hist + B - 1) // B
    assert used == blocks.sum()
    assert np.array_equal(t2e[:used], np.repeat(np.arange(E), blocks)) and (t2e[used:] == -1).all()
    order = np.argsort(eid, kind="stable")              # pairs by expert, ascending inside an expert
    first = np.concatenate([[0], np.cumsum(blocks)[:-1]]) * B
    want_sdst = np.full(max_tiles * B, -1, dtype=np.int32)
    pos = 0
    for e in range(E):
        want_sdst[first[e]:first[e] + hist[e]] = order[pos:pos + hist[e]]
        pos += hist[e]
    assert np.array_equal(sdst, want_sdst)
    assert np.array_equal(srow, np.where(want_sdst >= 0, want_sdst // top_k, -1))
    assert sorted(sdst[sdst >= 0].tolist()) == list(range(npair))

    K, inner, H = 128, 6, 10
    gu = [synth.make_weight(2 * inner, K, 700 + e) for e in range(E)]
    dn = [synth.make_weight(H, K, 800 + e) for e in range(E)]
    guw, gus, gub = (np.stack([p[i] for p in gu]) for i in range(3))
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(T, K, 900)
    y64, yb = oracle.qmm_grouped(guw, gus, gub, x, K, 2 * inner, B, t2e, srow=srow)
    for slot in range(max_tiles * B):
        if t2e[slot // B] < 0:
            continue
        if srow[slot] < 0:
            assert not y64[slot].any()                  # zero row in, zero sums out
            continue
        e = t2e[slot // B]
        assert e == eid[sdst[slot]]
        p64, pb = oracle.qmm(guw[e], gus[e], gub[e], x[srow[slot]:srow[slot] + 1], K, 2 * inner, 1)
        assert np.array_equal(y64[slot], p64[0]) and np.array_equal(yb[slot], pb[0])
    xs = synth.make_act(max_tiles * B, K, 901)
    d64, dbits = oracle.qmm_grouped(dw, ds, db, xs, K, H, B, t2e, sdst=sdst, rows_y=npair)
    for slot in range(max_tiles * B):
        p = sdst[slot]
        if p < 0:
            continue
        p64, pb = oracle.qmm(dw[eid[p]], ds[eid[p]], db[eid[p]], xs[slot:slot + 1], K, H, 1)
        assert np.array_equal(d64[p], p64[0]) and np.array_equal(dbits[p], pb[0])
    # ids outside [0, E) get no slot
    bad = np.array([1, -1, E, 0], dtype=np.int32)
    t2, sr, sd, u = oracle.moe_sort_pairs(bad, 1, E, B, 6)
    assert sorted(sd[sd >= 0].tolist()) == [0, 3] and u == 2


def f16_pack(N, K, seed):
    """A 4-bit pack whose scales and biases are IEEE binary16 (the reference's VPIPE_ELT = half build)."""
    rng = np.random.default_rng(seed)
    w = rng.integers(0, 2**32, size=(N, K // 8), dtype=np.uint32)
    s = rng.uniform(0.005, 0.02, size=(N, K // 64)).astype(np.float16)
    b = (np.float32(-8.0) * s.astype(np.float32) * (1 + 0.05 * rng.standard_normal(s.shape))).astype(np.float16)
    return w, s.view(np.uint16), b.view(np.uint16)


def test_f16_element_twins_against_numpy_float16(oracle):
    """binary16 twins: the dense expansion against numpy's own float16 arithmetic written from the layout
    (shifts on the packed words, a float32 multiply-add, numpy's round-to-nearest-even cast), the two
    contractions against a float64 matmul of that expansion, the residual add in binary16."""
    N, K, M = 19, 256, 3
    w, s, b = f16_pack(N, K, 41)
    q = ((w[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF).reshape(N, K).astype(np.float32)
    sf = np.repeat(s.view(np.float16).astype(np.float32), 64, axis=1)
    bf = np.repeat(b.view(np.float16).astype(np.float32), 64, axis=1)
    dense32 = sf * q + bf                                   # s*q is exact in fp32: no contraction issue
    want = dense32.astype(np.float16)
    assert np.array_equal(oracle.dequant_f16(w, s, b, K, N), want.view(np.uint16))
    x = np.random.default_rng(42).standard_normal((M, K)).astype(np.float16)
    xb = x.view(np.uint16)
    y64, yh = oracle.matmul_f16(w, s, b, xb, K, N, M, rounded=False)
    ref = x.astype(np.float64) @ dense32.astype(np.float64).T
    assert np.allclose(y64, ref, rtol=0, atol=1e-12 * np.abs(ref).max() + 1e-12)
    assert np.array_equal(yh, ref.astype(np.float32).astype(np.float16).view(np.uint16))
    r64, _ = oracle.matmul_f16(w, s, b, xb, K, N, M, rounded=True)
    refr = x.astype(np.float64) @ want.astype(np.float64).T
    assert np.allclose(r64, refr, rtol=0, atol=1e-12 * np.abs(refr).max() + 1e-12)
    assert not np.array_equal(r64, y64)                     # the rounding of the weights is visible
    res = np.random.default_rng(43).standard_normal((M, N)).astype(np.float16)
    _, ya = oracle.matmul_f16(w, s, b, xb, K, N, M, rounded=False, residual=res.view(np.uint16))
    want_add = (yh.view(np.float16).astype(np.float32) + res.astype(np.float32)).astype(np.float16)
    assert np.array_equal(ya, want_add.view(np.uint16))


def test_w8_expansion_on_binary16_elements_against_numpy_float16(oracle):
    """The half build's 8-bit expansion (groups of 64 and of 32): numpy's float16 arithmetic from the byte view of the
    words -- a float32 multiply-add whose product is exact, numpy's round-to-nearest-even cast."""
    rng = np.random.default_rng(44)
    for group in (64, 32):
        N, K = 13, 256
        w = rng.integers(0, 2**32, size=(N, K // 4), dtype=np.uint32)
        s = rng.uniform(0.0003, 0.0012, size=(N, K // group)).astype(np.float16)
        b = (-128.0 * s.astype(np.float32) * rng.uniform(0.9, 1.1, size=s.shape)).astype(np.float16)
        q = w.view(np.uint8).reshape(N, K).astype(np.float32)          # little-endian bytes = values in k order
        dense32 = np.repeat(s.astype(np.float32), group, axis=1) * q + np.repeat(b.astype(np.float32), group, axis=1)
        got = oracle.dequant8_f16(w, s.view(np.uint16), b.view(np.uint16), K, N, group=group)
        assert np.array_equal(got, dense32.astype(np.float16).view(np.uint16))
        assert np.abs(dense32).max() > 0


def test_f16_adapter_against_numpy_float16(oracle):
    """The adapter on binary16 elements, written independently in numpy: t = f16(alpha * f16(x . A^T)) with the
    contraction in float64 and numpy's own float16 casts, then y = f16(x . f16(W)^T + t . B^T); an adapter whose t is
    zero leaves the base GEMM's bits; the delta is a visible part of the output."""
    N, K, M, R = 21, 256, 5, 48
    alpha = 0.625
    w, s, b = f16_pack(N, K, 61)
    rng = np.random.default_rng(62)
    x = rng.standard_normal((M, K)).astype(np.float16)
    A = (0.05 * rng.standard_normal((R, K))).astype(np.float16)
    B = (0.05 * rng.standard_normal((N, R))).astype(np.float16)
    t = oracle.lora_t_f16(x.view(np.uint16), A.view(np.uint16), M, K, R, alpha)
    tt = (x.astype(np.float64) @ A.astype(np.float64).T).astype(np.float32).astype(np.float16)
    want_t = (tt.astype(np.float32) * np.float32(alpha)).astype(np.float16)
    assert np.array_equal(t, want_t.view(np.uint16))
    y64, yh = oracle.qmm_lora_f16(w, s, b, x.view(np.uint16), K, N, M, t, B.view(np.uint16), R)
    Wh = oracle.dequant_f16(w, s, b, K, N).view(np.float16).astype(np.float64)      # pinned above against numpy
    base = x.astype(np.float64) @ Wh.T
    delta = want_t.astype(np.float64) @ B.astype(np.float64).T
    ref = base + delta
    assert np.allclose(y64, ref, rtol=0, atol=1e-12 * np.abs(ref).max() + 1e-12)
    assert np.array_equal(yh, ref.astype(np.float32).astype(np.float16).view(np.uint16))
    assert np.sqrt((delta ** 2).sum() / (ref ** 2).sum()) > 0.01
    b64, bh = oracle.matmul_f16(w, s, b, x.view(np.uint16), K, N, M, rounded=True)
    z64, zh = oracle.qmm_lora_f16(w, s, b, x.view(np.uint16), K, N, M, np.zeros_like(t), B.view(np.uint16), R)
    assert np.array_equal(z64, b64) and np.array_equal(zh, bh)


def test_rmsnorm_against_torch_and_closed_forms(oracle):
    """The RMSNorm ahead of the fused-QKV GEMV: against torch.nn.functional.rms_norm in float64 (an independent
    routine) to one bf16 step with almost every element equal; a row of ones gives norm_w / sqrt(1 + eps); a row of
    +-c with eps = 0 gives +-norm_w exactly, whatever c (scale invariance); rows are independent."""
    import torch
    K, M, eps = 1536, 3, 1e-6
    x = synth.make_act(M, K, 71)
    nw = synth.f32_to_bf16_bits((1.0 + 0.1 * np.random.default_rng(72).standard_normal(K)).astype(np.float32))
    got = oracle.rmsnorm(x, nw, K, M, eps)
    xt = torch.from_numpy(synth.bf16_bits_to_f32(x).astype(np.float64))
    wt = torch.from_numpy(synth.bf16_bits_to_f32(nw).astype(np.float64))
    ref = torch.nn.functional.rms_norm(xt, (K,), weight=wt, eps=eps).numpy()
    want = synth.f32_to_bf16_bits(ref.astype(np.float32))
    assert (got != want).mean() < 0.01 and parity_ulp(got, want) <= 1
    assert np.array_equal(oracle.rmsnorm(x[1:2], nw, K, 1, eps), got[1:2])
    ones = synth.f32_to_bf16_bits(np.ones((1, K), dtype=np.float32))
    w1 = synth.bf16_bits_to_f32(nw).astype(np.float64) / np.sqrt(1.0 + 0.25)
    g1 = oracle.rmsnorm(ones, nw, K, 1, 0.25)
    assert parity_ulp(g1[0], synth.f32_to_bf16_bits(w1.astype(np.float32))) <= 1
    sign = np.where(np.arange(K) % 3 == 0, -1.0, 1.0).astype(np.float32)
    for c in (0.5, 8.0, 96.0):
        gc = oracle.rmsnorm(synth.f32_to_bf16_bits((c * sign)[None, :]), nw, K, 1, 0.0)
        assert np.array_equal(gc[0], synth.f32_to_bf16_bits(sign * synth.bf16_bits_to_f32(nw)))


def parity_ulp(a, b):
    from tests import parity
    return int(parity.bf16_ulp_distance(a, b).max())


def test_w8g32_twins_against_numpy_and_the_group64_oracle(oracle):
    """8-bit codes in groups of 32: the dense expansion against numpy written from the byte view of the words, both
    contractions against a float64 matmul of it, and a group-64 pack whose scales and biases are each stored twice
    gives the group-64 oracle's bits."""
    N, K, M = 11, 192, 3
    w, s, b = synth.make_weight8(N, K, 81, group=32)
    q = w.view(np.uint8).reshape(N, K).astype(np.float32)          # little-endian bytes = values in k order
    sf = np.repeat(synth.bf16_bits_to_f32(s), 32, axis=1)
    bf = np.repeat(synth.bf16_bits_to_f32(b), 32, axis=1)
    dense32 = sf * q + bf                                          # s*q exact in fp32 (8 x 8 bit significands)
    assert np.array_equal(oracle.dequant8_g32(w, s, b, K, N), synth.f32_to_bf16_bits(dense32))
    x = synth.make_act(M, K, 82)
    xf = synth.bf16_bits_to_f32(x).astype(np.float64)
    y64, yb = oracle.matmul8(w, s, b, x, K, N, M, rounded=False, group=32)
    ref = xf @ dense32.astype(np.float64).T
    assert np.allclose(y64, ref, rtol=0, atol=1e-12 * np.abs(ref).max() + 1e-12)
    assert np.array_equal(yb, synth.f32_to_bf16_bits(ref.astype(np.float32)))
    r64, _ = oracle.matmul8(w, s, b, x, K, N, M, rounded=True, group=32)
    refr = xf @ synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(dense32)).astype(np.float64).T
    assert np.allclose(r64, refr, rtol=0, atol=1e-12 * np.abs(refr).max() + 1e-12)
    w6, s6, b6 = synth.make_weight8(N, K, 83)
    s2, b2 = np.repeat(s6, 2, axis=1), np.repeat(b6, 2, axis=1)
    assert np.array_equal(oracle.dequant8_g32(w6, s2, b2, K, N), oracle.dequant8_bf16(w6, s6, b6, K, N))
    a64, ab = oracle.matmul8(w6, s2, b2, x, K, N, M, rounded=False, group=32)
    c64, cb = oracle.matmul8(w6, s6, b6, x, K, N, M, rounded=False)
    assert np.array_equal(a64, c64) and np.array_equal(ab, cb)


def test_requantizer_known_answers_invariants_and_numpy(oracle):
    """affine_requant_w8_to_w4_g64 (gpu-kernels/metal/quant/affine_dequant.metal:134-186).  (a) A pack whose bytes are
    17 c (c a nibble, 0 and 15 both present in every group) with power-of-two scale requantizes to exactly the nibbles
    c in k order, scale 17 s and the same bias: pins the byte -> nibble order and the word layout.  (b) A constant
    group: scale 0, codes 0, bias = the value.  (c) On a random pack: every group uses code 0 and code 15, the
    reconstruction with the unrounded scale is within half a step, and the whole agrees with a vectorized numpy
    statement written from the layout."""
    rng = np.random.default_rng(91)
    N, K = 5, 256
    c = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    c.reshape(N, K // 64, 64)[:, :, 3] = 0
    c.reshape(N, K // 64, 64)[:, :, 40] = 15
    w8 = (c * 17).astype(np.uint8).view(np.uint32).reshape(N, K // 4)
    s8 = synth.f32_to_bf16_bits(np.full((N, K // 64), 2.0 ** -6, np.float32))
    b8 = synth.f32_to_bf16_bits(np.full((N, K // 64), -1.0, np.float32))
    w4, s4, b4 = oracle.requant_w8_to_w4(w8, s8, b8, K, N)
    nib = ((w4[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF).reshape(N, K).astype(np.uint8)
    assert np.array_equal(nib, c)
    assert np.array_equal(s4, synth.f32_to_bf16_bits(np.full((N, K // 64), 17.0 * 2.0 ** -6, np.float32)))
    assert np.array_equal(b4, b8)
    # (b)
    w8c = np.full((1, 16), 0x5A5A5A5A, np.uint32)
    s1 = synth.f32_to_bf16_bits(np.array([[0.25]], np.float32))
    b1 = synth.f32_to_bf16_bits(np.array([[-3.0]], np.float32))
    w4c, s4c, b4c = oracle.requant_w8_to_w4(w8c, s1, b1, 64, 1)
    assert not w4c.any() and s4c[0, 0] == 0
    assert b4c[0, 0] == synth.f32_to_bf16_bits(np.array([0.25 * 0x5A - 3.0], np.float32))[0]
    # (c)
    N, K = 13, 320
    w8, s8, b8 = synth.make_weight8(N, K, 92)
    w4, s4, b4 = oracle.requant_w8_to_w4(w8, s8, b8, K, N)
    q8 = w8.view(np.uint8).reshape(N, K // 64, 64).astype(np.float32)
    v = synth.bf16_bits_to_f32(s8)[:, :, None] * q8 + synth.bf16_bits_to_f32(b8)[:, :, None]
    assert v.dtype == np.float32
    mn, mx = v.min(axis=2, keepdims=True), v.max(axis=2, keepdims=True)
    scale = (mx - mn) / np.float32(15.0)
    inv = np.float32(1.0) / scale
    t = (v - mn) * inv
    fl = np.floor(t)
    q4 = np.clip(np.where(t - fl >= np.float32(0.5), fl + 1, fl), 0, 15).astype(np.uint32)   # halves away from zero (t >= 0); t - fl is exact
    assert (t - fl == np.float32(0.5)).any()                       # exact halves occur, so the tie rule is exercised
    nib = ((w4[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF).reshape(N, K // 64, 64)
    assert np.array_equal(nib, q4)
    assert np.array_equal(s4, synth.f32_to_bf16_bits(scale[:, :, 0]))
    assert np.array_equal(b4, synth.f32_to_bf16_bits(mn[:, :, 0]))
    assert (nib.min(axis=2) == 0).all() and (nib.max(axis=2) == 15).all()
    recon = mn.astype(np.float64) + scale.astype(np.float64) * nib
    assert (np.abs(recon - v) <= 0.5 * scale * (1 + 1e-5)).all()


def test_grouped_gemm_oracle_with_byte_codes_reduces_to_the_plain_8bit_gemm(oracle):
    """The 8-bit form of the grouped restatement: every live slot equals the plain 8-bit GEMM oracle
    (bf16-rounded weights) of its row on its expert's slab."""
    E, top_k, T, B, K, N = 3, 2, 7, 4, 128, 9
    eid = np.random.default_rng(51).integers(0, E, size=T * top_k, dtype=np.int32)
    t2e, srow, sdst, _ = oracle.moe_sort_pairs(eid, top_k, E, B, (eid.size + B - 1) // B + E)
    packs = [synth.make_weight8(N, K, 600 + e) for e in range(E)]
    w, s, b = (np.stack([p[i] for p in packs]) for i in range(3))
    x = synth.make_act(T, K, 52)
    y64, yb = oracle.qmm_grouped(w, s, b, x, K, N, B, t2e, srow=srow, bits=8)
    seen = 0
    for slot in range(srow.size):
        if t2e[slot // B] < 0 or srow[slot] < 0:
            continue
        e = t2e[slot // B]
        p64, pb = oracle.matmul8(w[e], s[e], b[e], x[srow[slot]:srow[slot] + 1], K, N, 1, rounded=True)
        assert np.array_equal(y64[slot], p64[0]) and np.array_equal(yb[slot], pb[0])
        seen += 1
    assert seen == eid.size


def test_cpu_baseline_stages_agree_with_the_oracle(oracle):
    # the timed baseline's pieces (expansion, fp32 dot, fused form) against the float64 oracle and each other
    K, N, M = 1024, 33, 3
    w, s, b = synth.make_weight(N, K, 1)
    x = synth.make_act(M, K, 2)
    wdeq = np.empty((N, K), dtype=np.float32)
    oracle.cpu_dequant_f32(w, s, b, K, N, wdeq)
    assert np.array_equal(wdeq, oracle.dequant_f32(w, s, b, K, N))
    staged = oracle.cpu_matmul_f32(wdeq, x, K, N, M)
    whole = oracle.cpu_dequant_matmul(w, s, b, x, K, N, M)
    fused = oracle.cpu_fused_qmv(w, s, b, x, K, N, M)
    assert np.array_equal(staged, whole)
    y64, _ = oracle.qmv(w, s, b, x, K, N, M)
    for got in (staged, fused):
        g = synth.bf16_bits_to_f32(got).astype(np.float64)
        rms = np.sqrt((y64 ** 2).mean())
        assert (np.abs(g - y64) / np.maximum(np.abs(y64), 1e-2 * rms)).max() < 1e-2


# ---- the sampler tail (llm_elementwise.metal:3063-3298) ---------------------------------------------

def _sampler_kept_set_f64(logits_f, seen, temp, top_p, rep, pres, top_k, min_p):
    """The host sampler's pipeline in float64 with a sort (no bisection): the set of tokens that survive, and their
    probabilities.  Independent of the oracle's thresholds; equal to them wherever no weight sits at a threshold."""
    v = logits_f.astype(np.float64)
    pen = np.where(v >= 0, v / rep, v * rep) - pres
    eff = np.where(seen != 0, pen, v)
    w = np.exp((eff - eff.max()) / max(temp, 1e-6))
    keep = np.ones(w.shape, dtype=bool)
    if 0 < top_k < w.size:
        keep &= w >= np.sort(w)[::-1][top_k - 1]
    keep &= w >= max(min_p, 0.0)
    order = np.argsort(-w * keep, kind="stable")
    csum = np.cumsum((w * keep)[order])
    n_nucleus = int(np.searchsorted(csum, top_p * w.sum(), side="left")) + 1
    nucleus = np.zeros_like(keep)
    nucleus[order[:n_nucleus]] = True
    keep &= nucleus
    p = w * keep
    return keep, p / p.sum(), eff


def test_sampler_exp_log_and_hash_are_what_they_say(oracle):
    x = np.concatenate([np.linspace(-87, 0, 4001), -np.geomspace(1e-8, 80, 500)]).astype(np.float32)
    e = oracle.sample_exp(x).astype(np.float64)
    assert np.max(np.abs(e - np.exp(x.astype(np.float64))) / np.exp(x.astype(np.float64))) < 2e-7
    assert oracle.sample_exp([-88.0, -1e9, -np.inf])[0] == 0 and not oracle.sample_exp([-1e9, -np.inf, np.nan]).any()
    assert oracle.sample_exp([0.0])[0] == 1.0
    u = np.concatenate([np.geomspace(1e-20, 1, 3000), np.linspace(0.5, 2, 701), [46.0, 3.4e38]]).astype(np.float32)
    l = oracle.sample_log(u).astype(np.float64)
    ref = np.log(u.astype(np.float64))
    assert np.max(np.abs(l - ref) / np.maximum(np.abs(ref), 1e-3)) < 2e-7
    assert oracle.sample_log([1.0])[0] == 0.0
    # the hash, re-stated with Python integers (llm_elementwise.metal:3096-3104)
    def h(x):
        x ^= x >> 16; x = (x * 0x7feb352d) & 0xffffffff
        x ^= x >> 15; x = (x * 0x846ca68b) & 0xffffffff
        x ^= x >> 16
        return np.float32((np.float32(x) + np.float32(0.5)) * np.float32(1.0 / 4294967296.0))
    xs = [0, 1, 2, 12345, 0x80000000, 0xffffffff, 2654435761]
    assert np.array_equal(oracle.sample_hash_u01(xs), np.array([h(v) for v in xs], dtype=np.float32))
    us = oracle.sample_hash_u01(np.arange(200000, dtype=np.uint32))
    assert 0 < us.min() and us.max() <= 1.0 and abs(us.mean() - 0.5) < 5e-3


def test_sampler_degenerate_settings_reduce_to_argmax(oracle):
    rng = np.random.default_rng(31)
    V = 5000
    bits = synth.f32_to_bf16_bits((rng.standard_normal(V) * 4).astype(np.float32))
    seen = np.zeros(V, dtype=np.uint8)
    top = int(oracle.argmax(bits)[0])
    for seed in range(5):
        assert oracle.sample_topp(bits, seen, 1.0, 1.0, seed, top_k=1)[0] == top          # only the best survives
        assert oracle.sample_topp(bits, seen, 1.0, 1e-6, seed)[0] == top                  # a nucleus of one
        assert oracle.sample_topp(bits, seen, 1.0, 1.0, seed, min_p=1.0)[0] == top        # floor at the largest weight
        assert oracle.sample_topp(bits, seen, 1e-4, 1.0, seed)[0] == top                  # temperature -> 0
    tok, ws, seen_after = oracle.sample_topp(bits, seen, 0.8, 0.9, 7)
    assert seen_after[tok] == 1 and seen_after.sum() == 1 and not seen.any()
    assert synth.bf16_bits_to_f32(ws).max() == 1.0                                        # the largest weight is exactly 1
    # a repetition penalty that pushes the favourite below the runner-up changes the greedy answer
    vals = np.full(V, -5.0, dtype=np.float32); vals[10] = 4.0; vals[20] = 3.5
    bits2 = synth.f32_to_bf16_bits(vals)
    seen2 = np.zeros(V, dtype=np.uint8); seen2[10] = 1
    assert oracle.sample_topp(bits2, seen2, 1.0, 1.0, 0, top_k=1)[0] == 10                # 4.0 / 1.0 still first
    assert oracle.sample_topp(bits2, seen2, 1.0, 1.0, 0, top_k=1, rep=1.5)[0] == 20       # 4 / 1.5 < 3.5
    assert oracle.sample_topp(bits2, seen2, 1.0, 1.0, 0, top_k=1, pres=1.0)[0] == 20      # 4 - 1 < 3.5
    vals[10] = -1.0; vals[20] = -1.2                                                      # negative logits are multiplied
    assert oracle.sample_topp(synth.f32_to_bf16_bits(vals), seen2, 1.0, 1.0, 0, top_k=1, rep=1.5)[0] == 20


@pytest.mark.parametrize("temp,top_p,top_k,min_p,rep,pres", [(1.0, 1.0, 0, 0.0, 1.0, 0.0), (0.7, 0.9, 0, 0.0, 1.0, 0.0),
                                                            (1.3, 1.0, 12, 0.0, 1.0, 0.0), (1.0, 0.95, 40, 0.02, 1.2, 0.3)])
def test_sampler_draws_from_the_filtered_distribution(oracle, temp, top_p, top_k, min_p, rep, pres):
    """Over many seeds the drawn tokens lie in the kept set of an independent float64 restatement of the pipeline
    (sorted, no bisection) and follow its renormalised probabilities (chi-square)."""
    rng = np.random.default_rng(41)
    V = 300
    vals = (rng.standard_normal(V) * 2.0).astype(np.float32)
    bits = synth.f32_to_bf16_bits(vals)
    seen = (rng.random(V) < 0.2).astype(np.uint8)
    keep, prob, _ = _sampler_kept_set_f64(synth.bf16_bits_to_f32(bits), seen, temp, top_p, rep, pres, top_k, min_p)
    draws = 6000
    counts = np.zeros(V)
    for seed in range(draws):
        tok, ws, _ = oracle.sample_topp(bits, seen, temp, top_p, seed * 2654435761 % (1 << 32), n_iter=30, rep=rep, pres=pres,
                                        top_k=top_k, min_p=min_p)
        counts[tok] += 1
    # thresholds sit between weights (bf16-cached), so the kept set may differ from the float64 one by tokens whose
    # weight is within bf16 rounding of a threshold: allow those, nothing else
    w = synth.bf16_bits_to_f32(ws).astype(np.float64)
    outside = np.nonzero((counts > 0) & ~keep)[0]
    edge = w[keep].min() if keep.any() else 0.0
    assert all(abs(w[i] - edge) <= edge * 2.0 ** -7 for i in outside), outside
    big = keep & (prob * draws >= 8)
    chi2 = (((counts[big] - prob[big] * draws) ** 2) / (prob[big] * draws)).sum()
    dof = int(big.sum())
    assert chi2 < dof + 6 * np.sqrt(2 * dof) + 10, (chi2, dof)


def test_histogram_sampler_with_the_filters_off_is_the_exact_sampler(oracle):
    """No top-k, no top-p: nothing depends on the histogram, so the token (and the cached weights) are those of the
    one-workgroup sampler, which is pinned above; with min-p alone the threshold is min_p itself in both."""
    rng = np.random.default_rng(51)
    for V, n_slabs in ((1, 1), (300, 1), (300, 7), (5000, 3), (5000, 64)):
        bits = synth.f32_to_bf16_bits((rng.standard_normal(V) * 3).astype(np.float32))
        seen = (rng.random(V) < 0.15).astype(np.uint8)
        for seed in range(12):
            for min_p in (0.0, 0.03):
                a = oracle.sample_topp(bits, seen, 0.9, 1.0, seed, rep=1.3, pres=0.2, min_p=min_p)
                b = oracle.sample_hist(bits, seen, 0.9, 1.0, seed, n_slabs, rep=1.3, pres=0.2, min_p=min_p)
                assert a[0] == b[0] and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])
                w = synth.bf16_bits_to_f32(b[1])
                assert np.array_equal(w >= b[3], w >= np.float32(min_p))      # the threshold keeps what min_p keeps


@pytest.mark.parametrize("temp,top_p,top_k,min_p", [(1.0, 0.9, 0, 0.0), (0.7, 1.0, 25, 0.0), (1.2, 0.8, 60, 0.0),
                                                    (1.0, 0.95, 40, 0.01), (1.0, 0.5, 3, 0.0)])
def test_histogram_sampler_threshold_is_the_low_edge_of_the_boundary_bin(oracle, temp, top_p, top_k, min_p):
    """The threshold against a float64 sort: for top-k it is the low edge of the bin holding the k-th largest weight,
    for top-p that of the bin holding the last weight of the smallest nucleus -- at most the exact threshold, and
    more than it divided by one bin's width (two where the truncated fixed-point masses may push the nucleus one bin
    on); the three thresholds combine by their maximum."""
    rng = np.random.default_rng(61)
    binw = 40.0 / 1024.0
    for V, n_slabs in ((400, 1), (6000, 5), (6000, 64)):
        vals = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits((rng.standard_normal(V) * 2.5).astype(np.float32)))
        bits = synth.f32_to_bf16_bits(vals)
        seen = np.zeros(V, dtype=np.uint8)
        _, _, _, wt = oracle.sample_hist(bits, seen, temp, top_p, 3, n_slabs, top_k=top_k, min_p=min_p)
        w = np.exp((vals.astype(np.float64) - vals.max()) / temp)
        sw = np.sort(w)[::-1]
        lo, hi = [], []
        if 0 < top_k < V:
            lo.append(sw[top_k - 1] * np.exp(-binw)); hi.append(sw[top_k - 1])
        n = int(np.searchsorted(np.cumsum(sw), top_p * w.sum(), side="left"))
        if n < V:
            lo.append(sw[n] * np.exp(-2 * binw)); hi.append(sw[n])
        lo.append(min_p); hi.append(min_p)
        assert max(lo) * (1 - 1e-5) < wt <= max(hi) * (1 + 1e-5), (V, n_slabs, wt, lo, hi)
        # and it is a bin edge (or min_p): -log(wt) / binw is an integer
        if wt > min_p:
            r = -np.log(float(wt)) / binw
            assert abs(r - round(r)) < 1e-3 and round(r) >= 1


def test_histogram_sampler_draws_from_the_kept_set(oracle):
    """Draws over many seeds stay inside {w >= threshold} and follow the renormalised float64 probabilities of that
    set (chi-square); the drawn token is marked seen."""
    rng = np.random.default_rng(71)
    V, n_slabs, temp, top_p, top_k = 300, 4, 0.9, 0.92, 35
    bits = synth.f32_to_bf16_bits((rng.standard_normal(V) * 2.0).astype(np.float32))
    seen = (rng.random(V) < 0.2).astype(np.uint8)
    rep, pres = 1.2, 0.3
    _, _, eff = _sampler_kept_set_f64(synth.bf16_bits_to_f32(bits), seen, temp, 1.0, rep, pres, 0, 0.0)
    draws = 6000
    counts = np.zeros(V)
    for seed in range(draws):
        tok, ws, seen_after, wt = oracle.sample_hist(bits, seen, temp, top_p, seed * 2654435761 % (1 << 32), n_slabs, rep=rep,
                                                     pres=pres, top_k=top_k)
        counts[tok] += 1
        assert seen_after[tok] == 1
    w = synth.bf16_bits_to_f32(ws).astype(np.float64)
    keep = w >= wt
    assert not counts[~keep].any()
    assert top_k <= keep.sum() < V // 2                       # looser than top-k by at most a bin, far from everything
    p64 = np.exp((eff - eff.max()) / temp) * keep
    p64 /= p64.sum()
    big = keep & (p64 * draws >= 8)
    chi2 = (((counts[big] - p64[big] * draws) ** 2) / (p64[big] * draws)).sum()
    dof = int(big.sum())
    assert chi2 < dof + 6 * np.sqrt(2 * dof) + 10, (chi2, dof)
