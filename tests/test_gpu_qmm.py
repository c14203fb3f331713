"""GPU parity: QMM (bf16-rounded weight tile, MFMA, fp32 accumulate) and the fused
runtime LoRA against the CPU oracle, through the C ABI.  Shapes follow the
reference's qmm tests (tests/unit-tests/metal-compute-gemm-mma.cc:312-498) and
LoRA test (tests/unit-tests/minimax-h3-blocks.cc:1162-1296), then the
benchmark's prefill and video-DiT shapes with the oracle on a row/column sample."""
import numpy as np
import pytest
import torch

from tests import parity
from tests.golden import refgen
from vpipe_amd import synth

pytestmark = pytest.mark.gpu


def stage(D, dev, w, s, b, x):
    return D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)


REFERENCE_SHAPES = [
    # M, N, K  -- qmm_mma.correctness and qmm_mma.ragged_n_matches_reference
    (64, 64, 64), (96, 128, 128), (130, 320, 256), (512, 256, 2560),
    (33, 33, 128), (64, 95, 192), (96, 161, 256),
    (17, 16, 64), (1, 8, 64), (257, 129, 512),
]


@pytest.mark.parametrize("M,N,K", REFERENCE_SHAPES)
def test_qmm_reference_shapes(vpq, oracle, dev, D, M, N, K):
    w, s, b = synth.make_weight(N, K, 999 + N + K)
    x = synth.make_act(M, K, 555 + M + N + K)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    got = D.bits(out.view)
    parity.check_bf16(got, y64, yb)
    out.assert_intact()
    # the reference's own bar (rel-L2 < 3e-2 against an fp32 CPU loop over the UN-rounded weight)
    W = oracle.dequant_f32(w, s, b, K, N).astype(np.float64)
    ref = synth.bf16_bits_to_f32(x).astype(np.float64) @ W.T
    assert parity.rel_l2(synth.bf16_bits_to_f32(got), ref) < 3e-2


def test_qmm_one_hot_reads_back_the_rounded_weight(vpq, oracle, dev, D):
    # x = e_k  =>  y[m,n] = bf16(fp32(s*q+b)) exactly: the tile's dequant is the a1 arithmetic
    K, N, M = 256, 144, 20
    w, s, b = synth.make_weight(N, K, 17)
    d16 = oracle.dequant_bf16(w, s, b, K, N)
    x = np.zeros((M, K), dtype=np.float32)
    ks = [(m * 37 + 5) % K for m in range(M)]
    for m, k in enumerate(ks):
        x[m, k] = 1.0
    wd, sd, bd, xd = stage(D, dev, w, s, b, synth.f32_to_bf16_bits(x))
    got = D.bits(vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M))
    for m, k in enumerate(ks):
        assert np.array_equal(got[m], d16[:, k]), m


def test_qmm_reference_lcg_inputs(vpq, oracle, dev, D):
    """make_act_/make_qw_ inputs of tests/unit-tests/minimax-h3-blocks.cc:121-158
    (s = 0.01, b = -0.08, LCG bytes); agreement bar of mma_matches_steel: rel-L2 < 3e-2."""
    M, N, K = 128, 96, 512
    packed, s0, b0 = refgen.lcg_qweight(N, K, 0xBEEF)
    s = np.full((N, K // 64), synth.f32_to_bf16_bits(np.float32(s0)), dtype=np.uint16)
    b = np.full((N, K // 64), synth.f32_to_bf16_bits(np.float32(b0)), dtype=np.uint16)
    x = synth.f32_to_bf16_bits(refgen.lcg_act(M * K, 21).reshape(M, K))
    y64, yb = oracle.qmm(packed, s, b, x, K, N, M)
    got = D.bits(vpq.qmm_w4g64(*stage(D, dev, packed, s, b, x), K, N, M))
    parity.check_bf16(got, y64, yb)


@pytest.mark.parametrize("r,alpha", [(8, 1.0), (16, 1.5), (24, 0.5), (32, 1.0), (40, 1.25), (48, 0.75), (64, 0.625), (72, 1.0), (128, 2.0),
                                     (256, 0.5), (384, 0.25)])
def test_qmm_lora_fused(vpq, oracle, dev, D, r, alpha):
    M, N, K = 96, 160, 512
    w, s, b = synth.make_weight(N, K, 23)
    s[:] = synth.f32_to_bf16_bits(np.float32(0.0005))      # small base: the delta is a visible part of y
    b[:] = synth.f32_to_bf16_bits(np.float32(-0.004))
    x = synth.f32_to_bf16_bits(refgen.lcg_act(M * K, 21).reshape(M, K))
    A = synth.f32_to_bf16_bits(refgen.lcg_act(r * K, 29).reshape(r, K))
    B = synth.f32_to_bf16_bits(refgen.lcg_act(N * r, 31).reshape(N, r))
    t_ref = oracle.lora_t(x, A, M, K, r, alpha)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    Ad, Bd = D.bf16(A, dev), D.bf16(B, dev)
    t = vpq.lora_a(xd, Ad, M, K, r, alpha)
    t_bits = D.bits(t)
    assert parity.bf16_ulp_distance(t_bits, t_ref).max() <= 1
    # the fused tile consumes the t the library produced: oracle on that same t
    y64, yb = oracle.qmm(w, s, b, x, K, N, M, t=t_bits, B=B, r=r)
    t_ws = torch.empty((M, r), dtype=torch.bfloat16, device=dev)
    got = D.bits(vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, lora_A=Ad, lora_B=Bd, r=r, alpha=alpha, t_ws=t_ws))
    assert np.array_equal(D.bits(t_ws), t_bits)
    parity.check_bf16(got, y64, yb)
    # float64 end to end: the reference's bar (rel-L2 < 5e-3, delta > 5% of the output)
    xf = synth.bf16_bits_to_f32(x).astype(np.float64)
    Wb = synth.bf16_bits_to_f32(oracle.dequant_bf16(w, s, b, K, N)).astype(np.float64)
    d = alpha * (xf @ synth.bf16_bits_to_f32(A).astype(np.float64).T) @ synth.bf16_bits_to_f32(B).astype(np.float64).T
    want = xf @ Wb.T + d
    assert parity.rel_l2(synth.bf16_bits_to_f32(got), want) < 5e-3
    assert np.sqrt((d ** 2).sum() / (want ** 2).sum()) > 0.05


@pytest.mark.parametrize("M,K,r", [(1, 64, 16), (33, 192, 32), (257, 4096, 16), (1000, 5120, 32), (31, 1024, 48), (600, 2048, 128),
                                   (50, 512, 8), (100, 1024, 24), (64, 2048, 40)])
def test_lora_pre_pass_alone(vpq, oracle, dev, D, M, K, r):
    """t = bf16(alpha * bf16(x . A^T)) (lora_gemm_a_, minimax-h3/metal-minimax-h3-transformer.cc:1030-1067) on ragged
    M, a K of one chunk, K with fewer chunks than wavefronts, and both kernels (ranks up to 32 / above), against the
    oracle within one ulp of the inner rounding bf16(x . A^T) (fp32 sums in another order than the oracle's double);
    alpha = 2 scales that exactly, alpha = 0.875 can carry the one ulp across a binade (two ulps of the smaller one);
    the scratch's guard bands stay intact."""
    alpha = 2.0 if (M + r) % 3 else 0.875
    x = synth.make_act(M, K, 8800 + M)
    A, _ = synth.make_lora(8, K, r, 8801 + r, std=0.05)
    t_ref = oracle.lora_t(x, A, M, K, r, alpha)
    out = parity.Guarded((M, r), torch.bfloat16, dev)
    vpq.lora_a(D.bf16(x, dev), D.bf16(A, dev), M, K, r, alpha, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    got = synth.bf16_bits_to_f32(D.bits(out.view)).astype(np.float64)
    ref = synth.bf16_bits_to_f32(t_ref).astype(np.float64)
    # one ulp of the inner rounding (2^-7 relative; 2^-6 of the result where alpha carries it across a binade), and
    # where the sum cancels, the fp32 accumulation's own error against the oracle's double
    mag = np.abs(synth.bf16_bits_to_f32(x).astype(np.float64)) @ np.abs(synth.bf16_bits_to_f32(A).astype(np.float64)).T
    allowed = (2.0 ** -7 if alpha == 2.0 else 2.0 ** -6) * np.abs(ref) + alpha * 64 * 2.0 ** -24 * mag
    assert (np.abs(got - ref) <= allowed).all()
    assert (D.bits(out.view) != t_ref).mean() < 0.02
    assert np.abs(synth.bf16_bits_to_f32(t_ref)).max() > 0


def test_qmm_lora_scale_zero_is_exactly_off(vpq, dev, D):
    # minimax_h3_lora: strength 0 == no adapter, bit for bit (metal-minimax-h3-transformer.cc:2211-2219)
    M, N, K, r = 70, 130, 256, 32
    w, s, b = synth.make_weight(N, K, 3)
    x = synth.make_act(M, K, 4)
    A, B = synth.make_lora(N, K, r, 5)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    base = D.bits(vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M))
    off = D.bits(vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, lora_A=D.bf16(A, dev), lora_B=D.bf16(B, dev),
                               r=r, alpha=0.0))
    assert np.array_equal(base, off)


def _sampled_check(vpq, oracle, dev, D, M, N, K, seed, lora_r=0, alpha=1.0, dense_route_too=False):
    """Full-size launch; oracle on a sample of rows of x and rows of W (tile edges included).  dense_route_too: the
    dequant-once route with the same adapter gives the same bits over the whole output."""
    w, s, b = synth.make_weight(N, K, seed)
    x = synth.make_act(M, K, seed + 1)
    rng = np.random.default_rng(seed + 2)
    ms = np.unique(np.concatenate([np.arange(4), np.arange(M - 4, M), rng.integers(0, M, 40)]))
    ns = np.unique(np.concatenate([np.arange(4), np.arange(N - 4, N), rng.integers(0, N, 56)]))
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    kw = {}
    t_bits = B = None
    if lora_r:
        A, B = synth.make_lora(N, K, lora_r, seed + 3)
        kw = dict(lora_A=D.bf16(A, dev), lora_B=D.bf16(B, dev), r=lora_r, alpha=alpha,
                  t_ws=torch.empty((M, lora_r), dtype=torch.bfloat16, device=dev))
    y = vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, **kw)
    torch.cuda.synchronize()
    got = D.bits(y[torch.from_numpy(ms).to(dev)][:, torch.from_numpy(ns).to(dev)])
    if lora_r:
        t_all = D.bits(kw["t_ws"])
        t_ref = oracle.lora_t(x[ms], A, len(ms), K, lora_r, alpha)
        assert parity.bf16_ulp_distance(t_all[ms], t_ref).max() <= 1
        t_bits, B = t_all[ms], B[ns]
    y64, yb = oracle.qmm(w[ns], s[ns], b[ns], x[ms], K, len(ns), len(ms), t=t_bits, B=B, r=lora_r)
    parity.check_bf16(got, y64, yb)
    if dense_route_too:
        w_deq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
        y2 = vpq.qmm_dense_route_w4g64(wd, sd, bd, xd, K, N, M, w_deq, **kw)
        torch.cuda.synchronize()
        assert torch.equal(y2, y)
    return y


@pytest.mark.parametrize("K,N", [(4096, 12288), (12288, 4096), (4096, 4096)])
def test_qmm_prefill_shapes(vpq, oracle, dev, D, K, N):
    _sampled_check(vpq, oracle, dev, D, 2048, N, K, 0x5EED0004 + N)


@pytest.mark.parametrize("K,N", [(5120, 5120), (5120, 20480), (20480, 5120)])
def test_qmm_video_dit_shapes_with_lora(vpq, oracle, dev, D, K, N):
    # M = 16320 = 127*128 + 64: an M tail; y of 5120->20480 is 668 MB: 64-bit addressing
    _sampled_check(vpq, oracle, dev, D, 16320, N, K, 0x5EED0005 + N, lora_r=32, alpha=1.0, dense_route_too=True)


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (130, 320, 256), (33, 33, 128), (257, 129, 512), (1, 8, 64)])
def test_qmm_dense_route_matches_oracle(vpq, oracle, dev, D, M, N, K):
    # the dequant-once route (expansion + the library's dense GEMM): same arithmetic as the fused kernel
    w, s, b = synth.make_weight(N, K, 4200 + N + K)
    x = synth.make_act(M, K, 4300 + M)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    w_deq = torch.zeros((N, K), dtype=torch.bfloat16, device=dev)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_dense_route_w4g64(wd, sd, bd, xd, K, N, M, w_deq, expand=True, out=out.view)
    torch.cuda.synchronize()
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    assert np.array_equal(D.bits(w_deq), oracle.dequant_bf16(w, s, b, K, N))
    # with the kept expansion: no expansion pass, same bits
    again = vpq.qmm_dense_route_w4g64(wd, sd, bd, xd, K, N, M, w_deq, expand=False)
    assert torch.equal(again, out.view)
    # and the bits of the fused large-tile kernel: the dense GEMM is that kernel with the weight tile loaded
    if K % 512 == 0:
        assert torch.equal(vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, tile_n=256), out.view)


@pytest.mark.parametrize("M,N,K,splits", [(100, 256, 2048, 0), (65, 128, 1024, 2), (300, 640, 4096, 0), (257, 129, 1536, 3),
                                          (128, 4096, 4096, 0), (40, 96, 1088, 16)])
def test_qmm_split_k(vpq, oracle, dev, D, M, N, K, splits):
    # few output tiles over a long K: shares of K into fp32 planes, folded in order, rounded once
    # (the reference's deep-K split, generative-models/shared/mma-splitk.h:30-52)
    w, s, b = synth.make_weight(N, K, 3000 + N)
    x = synth.make_act(M, K, 3100 + M)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_splitk_w4g64(wd, sd, bd, xd, K, N, M, splits=splits, out=out.view)
    torch.cuda.synchronize()
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    again = vpq.qmm_splitk_w4g64(wd, sd, bd, xd, K, N, M, splits=splits)
    assert torch.equal(again, out.view)                       # bit-reproducible
    if splits > 1:
        with pytest.raises(vpq.VpqError):
            vpq.qmm_splitk_w4g64(wd, sd, bd, xd, K, N, M, splits=splits, ws=torch.empty(256, dtype=torch.uint8, device=dev))


def test_linear_entrance_splits_k_when_given_the_room(vpq, oracle, dev, D):
    M, N, K = 128, 512, 4096
    w, s, b = synth.make_weight(N, K, 3200)
    x = synth.make_act(M, K, 3201)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    need = vpq.load().vpq_qmm_workspace_bytes(K, N, M)
    assert need >= 2 * M * N * 4
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    split = vpq.linear_w4g64(wd, sd, bd, xd, K, N, M, ws=ws)
    plain = vpq.linear_w4g64(wd, sd, bd, xd, K, N, M)
    torch.cuda.synchronize()
    parity.check_bf16(D.bits(split), y64, yb)
    parity.check_bf16(D.bits(plain), y64, yb)
    assert vpq.load().vpq_qmm_workspace_bytes(4096, 12288, 2048) == 0      # enough tiles: no split


@pytest.mark.parametrize("M", [33, 48, 64])
def test_linear_entrance_at_three_or_four_slabs(vpq, oracle, dev, D, M):
    # with the room to split K the GEMM (bf16-rounded weights), without it slabs of QMV (un-rounded
    # weights): each within the tolerance of its own oracle, and not the same bits
    N, K = 384, 4096
    w, s, b = synth.make_weight(N, K, 3300 + M)
    x = synth.make_act(M, K, 3301 + M)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    need = vpq.load().vpq_linear_workspace_bytes(K, N, M)
    assert need >= 2 * M * N * 4
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    split = vpq.linear_w4g64(wd, sd, bd, xd, K, N, M, ws=ws)
    direct = vpq.qmm_splitk_w4g64(wd, sd, bd, xd, K, N, M, splits=0, ws=ws.clone())
    slabs = vpq.linear_w4g64(wd, sd, bd, xd, K, N, M)
    torch.cuda.synchronize()
    assert torch.equal(split, direct)
    assert not torch.equal(split, slabs)
    parity.check_bf16(D.bits(split), y64, yb)
    v64, vb = oracle.qmv(w, s, b, x, K, N, M)                 # the slabs' arithmetic: un-rounded weights
    parity.check_bf16(D.bits(slabs), v64, vb)
    # 32 rows and fewer stay slabs whatever the workspace
    x32 = xd[:32].contiguous()
    assert torch.equal(vpq.linear_w4g64(wd, sd, bd, x32, K, N, 32, ws=ws), vpq.linear_w4g64(wd, sd, bd, x32, K, N, 32))


# M, N, K: the minimal K (one block of 8 steps), ragged M and N in both tile widths, more than one
# band of 8 rows of tiles (M > 2048), a single row
BIG_TILE_SHAPES = [(300, 520, 512), (257, 193, 1024), (2300, 200, 512), (1, 8, 512), (640, 384, 1536)]


@pytest.mark.parametrize("tile_n", [-128, 192, 256])
@pytest.mark.parametrize("M,N,K", BIG_TILE_SHAPES)
def test_qmm_large_tile_kernel(vpq, oracle, dev, D, M, N, K, tile_n):
    # against the oracle, and bit for bit against the 256x128 tile kernel: same MFMA, same K order
    w, s, b = synth.make_weight(N, K, 7100 + N + K)
    x = synth.make_act(M, K, 7200 + M + K)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, tile_n=tile_n)
    small = vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, tile_n=128)
    torch.cuda.synchronize()
    out.assert_intact()
    assert torch.equal(out.view, small)
    rng = np.random.default_rng(M + N)
    ms = np.unique(np.concatenate([np.arange(min(4, M)), np.arange(max(M - 4, 0), M), rng.integers(0, M, 24)]))
    y64, yb = oracle.qmm(w, s, b, x[ms], K, N, len(ms))
    parity.check_bf16(D.bits(out.view)[ms], y64, yb)


@pytest.mark.parametrize("tile_n", [-128, 192, 256])
@pytest.mark.parametrize("r", [8, 16, 24, 32, 48, 64, 88, 96, 256, 384])
def test_qmm_large_tile_kernel_with_lora(vpq, oracle, dev, D, r, tile_n):
    M, N, K, alpha = 300, 450, 1024, 0.75
    w, s, b = synth.make_weight(N, K, 7300 + r)
    s[:] = synth.f32_to_bf16_bits(np.float32(0.0005))      # small base: the delta is a visible part of y
    b[:] = synth.f32_to_bf16_bits(np.float32(-0.004))
    x = synth.make_act(M, K, 7301)
    A, B = synth.make_lora(N, K, r, 7302, std=0.05)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    Ad, Bd = D.bf16(A, dev), D.bf16(B, dev)
    t_ws = torch.empty((M, r), dtype=torch.bfloat16, device=dev)
    got = vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, lora_A=Ad, lora_B=Bd, r=r, alpha=alpha, t_ws=t_ws, tile_n=tile_n)
    small = vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, lora_A=Ad, lora_B=Bd, r=r, alpha=alpha, tile_n=128)
    assert torch.equal(got, small)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M, t=D.bits(t_ws), B=B, r=r)
    parity.check_bf16(D.bits(got), y64, yb)
    base = vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, tile_n=tile_n)
    assert not torch.equal(base, got)


@pytest.mark.parametrize("M,N,K,r", [(300, 450, 1024, 32), (64, 40, 192, 16), (2304, 4096, 512, 48), (130, 328, 1536, 384),
                                     (200, 264, 512, 8), (90, 136, 640, 24)])
def test_dense_route_with_lora_is_the_fused_gemm(vpq, oracle, dev, D, M, N, K, r):
    """The dequant-once route with the runtime adapter: the bits of the fused GEMM with the same adapter (whose
    parity test_qmm_lora_fused holds) where the fused kernel runs the same tiles, the oracle's tolerance everywhere,
    the kept expansion the same bits, the scratch the adapter's t, guard bands intact."""
    alpha = 0.75
    w, s, b = synth.make_weight(N, K, 7600 + r)
    s[:] = synth.f32_to_bf16_bits(np.float32(0.0005))
    b[:] = synth.f32_to_bf16_bits(np.float32(-0.004))
    x = synth.make_act(M, K, 7601)
    A, B = synth.make_lora(N, K, r, 7602, std=0.05)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    Ad, Bd = D.bf16(A, dev), D.bf16(B, dev)
    w_deq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    t_ws = parity.Guarded((M, r), torch.bfloat16, dev)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_dense_route_w4g64(wd, sd, bd, xd, K, N, M, w_deq, out=out.view, lora_A=Ad, lora_B=Bd, r=r, alpha=alpha, t_ws=t_ws.view)
    torch.cuda.synchronize()
    out.assert_intact()
    t_ws.assert_intact()
    assert torch.equal(t_ws.view, vpq.lora_a(xd, Ad, M, K, r, alpha))
    rows = np.arange(M) if M * N * K < 2e9 else np.r_[0:40, 1000:1024, M - 40:M]
    y64, yb = oracle.qmm(w, s, b, x[rows], K, N, len(rows), t=D.bits(t_ws.view)[rows], B=B, r=r)
    parity.check_bf16(D.bits(out.view)[rows], y64, yb)
    if K % 512 == 0:
        assert torch.equal(out.view, vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, lora_A=Ad, lora_B=Bd, r=r, alpha=alpha))
    kept = vpq.qmm_dense_route_w4g64(wd, sd, bd, xd, K, N, M, w_deq, expand=False, lora_A=Ad, lora_B=Bd, r=r, alpha=alpha)
    assert torch.equal(kept, out.view)
    assert not torch.equal(out.view, vpq.qmm_dense_route_w4g64(wd, sd, bd, xd, K, N, M, w_deq))
    L = vpq.load()
    p = out.view.data_ptr()
    assert L.vpq_qmm_dense_route_lora_w4g64_bf16(None, p, p, p, p, p, K, N, M, p, 1, p, p, 36, 1.0, p) == -2
    assert L.vpq_qmm_dense_route_lora_w4g64_bf16(None, p, p, p, p, p, K, N, M, p, 1, p, p, r, 1.0, None) == -4


def test_qmm_large_tile_kernel_refuses_what_it_cannot_take(vpq, dev, D):
    M, N, K = 64, 64, 576                                   # K not a multiple of 512
    w, s, b = synth.make_weight(N, K, 1)
    x = synth.make_act(M, K, 2)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    with pytest.raises(vpq.VpqError):
        vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, tile_n=256)
    with pytest.raises(vpq.VpqError):
        vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, tile_n=64)
    vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, tile_n=128)


def test_linear_entrance_takes_the_dequant_once_route_when_given_the_room(vpq, oracle, dev, D):
    M, N, K = 8200, 384, 512
    w, s, b = synth.make_weight(N, K, 7400)
    x = synth.make_act(M, K, 7401)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    need = vpq.load().vpq_linear_workspace_bytes(K, N, M)
    assert need >= N * K * 2
    assert vpq.load().vpq_linear_workspace_bytes(K, N, 512) == vpq.load().vpq_qmm_workspace_bytes(K, N, 512)
    ws = torch.zeros((need,), dtype=torch.uint8, device=dev)
    y = vpq.linear_w4g64(wd, sd, bd, xd, K, N, M, ws=ws)
    torch.cuda.synchronize()
    # the workspace now holds the expanded weight, bit-exact, and y is the dense route's result
    dense = ws[:N * K * 2].view(torch.bfloat16).view(N, K)
    assert np.array_equal(D.bits(dense), oracle.dequant_bf16(w, s, b, K, N))
    wdeq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    assert torch.equal(y, vpq.qmm_dense_route_w4g64(wd, sd, bd, xd, K, N, M, wdeq))
    rng = np.random.default_rng(5)
    ms = np.unique(rng.integers(0, M, 48))
    y64, yb = oracle.qmm(w, s, b, x[ms], K, N, len(ms))
    parity.check_bf16(D.bits(y)[ms], y64, yb)
    # too little room: the fused kernel -- the same arithmetic in the same order, so the same bits
    small = vpq.linear_w4g64(wd, sd, bd, xd, K, N, M, ws=ws[:4096])
    parity.check_bf16(D.bits(small)[ms], y64, yb)
    assert torch.equal(small, y)
