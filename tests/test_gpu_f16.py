"""GPU parity of the IEEE binary16 element type (the reference's VPIPE_ELT = half build) for the 4-bit
group-64 pack: dense expansion bit-exact, QMV (plain, residual, gated) and the dequant-once GEMM route
against the CPU oracle's binary16 twins, through the C ABI."""
import numpy as np
import pytest
import torch

from tests import parity
from tests.test_oracle_pins import f16_pack

pytestmark = pytest.mark.gpu

F16_TOL = 2e-3


def dev16(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(dev).view(torch.float16)


def bits16(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def check_f16(got_bits, ref64):
    """|got - ref| <= 2e-3 * max(|ref|, 1e-2 rms) + one binary16 step at |ref| (one rounding)."""
    got = got_bits.view(np.float16).astype(np.float64)
    rms = np.sqrt((ref64 ** 2).mean())
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref64), 2.0 ** -14))) - 10)
    allowed = F16_TOL * np.maximum(np.abs(ref64), 1e-2 * rms) + ulp
    worst = (np.abs(got - ref64) / allowed).max()
    assert worst <= 1.0, "binary16 output off by %.2f x the allowed error" % worst
    assert parity.rel_l2(got, ref64) <= 2e-3 + 3e-4


@pytest.mark.parametrize("N,K", [(1, 64), (33, 192), (257, 3840), (1024, 4096)])
def test_dequant_f16_bit_exact(vpq, oracle, dev, D, N, K):
    w, s, b = f16_pack(N, K, 100 + N)
    out = vpq.dequant_w4g64_f16(D.u32(w, dev), dev16(s, dev), dev16(b, dev), K, N)
    assert np.array_equal(bits16(out), oracle.dequant_f16(w, s, b, K, N))


@pytest.mark.parametrize("K,N,M", [(64, 5, 1), (192, 33, 3), (3840, 16, 1), (4096, 95, 8), (2560, 64, 16), (4096, 4096, 1)])
def test_qmv_f16(vpq, oracle, dev, D, K, N, M):
    w, s, b = f16_pack(N, K, 200 + K + N)
    x = np.random.default_rng(300 + K + M).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    y64, _ = oracle.matmul_f16(w, s, b, x, K, N, M, rounded=False)
    wd, sd, bd, xd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev)
    f = vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, f32out=True)
    out = parity.Guarded((M, N), torch.float16, dev)
    vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_f32(f.cpu().numpy(), y64)
    check_f16(bits16(out.view), y64)
    # the bf16 build of the same kernel on the same pack read as bf16 differs: the element type is live
    assert not torch.equal(out.view.view(torch.int16), vpq.qmv_w4g64(wd, sd.view(torch.bfloat16), bd.view(torch.bfloat16),
                                                                     xd.view(torch.bfloat16), K, N, M, variant=1).view(torch.int16))


@pytest.mark.parametrize("K,N,M", [(512, 16, 2), (1024, 37, 4), (5120, 530, 3), (5120, 1029, 5), (4608, 250, 8),
                                   (2560, 64, 12), (8192, 100, 16), (512, 16 * 1300, 2), (17408, 66, 9)])
def test_qmv_f16_several_rows_ring_kernel(vpq, oracle, dev, D, K, N, M):
    """2..16 rows of x on K % 512 == 0 run on the ring kernel's binary16 mode: x through LDS (up to 4 rows) and in
    registers, one and several slices per wavefront, ragged last tile, the two-register form at 2 rows."""
    w, s, b = f16_pack(N, K, 900 + K + N)
    x = np.random.default_rng(950 + K + M).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    y64, _ = oracle.matmul_f16(w, s, b, x, K, N, M, rounded=False)
    wd, sd, bd, xd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev)
    f = vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, f32out=True)
    out = parity.Guarded((M, N), torch.float16, dev)
    vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_f32(f.cpu().numpy(), y64)
    check_f16(bits16(out.view), y64)
    assert torch.equal(f, vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, f32out=True))     # bit-reproducible


@pytest.mark.parametrize("M", [2, 3, 4])
def test_qmv_f16_lm_head_rows_streaming_kernel(vpq, oracle, dev, D, M):
    """2..4 rows over an lm_head-sized pack (>= 150 MB of codes) run on the streaming MFMA kernel's binary16 mode.
    Full-size launch; the oracle evaluates a sample of output rows (first and last tiles included)."""
    K, N = 5120, 151936
    w, s, b = f16_pack(N, K, 1200 + M)
    x = np.random.default_rng(1250 + M).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    rng = np.random.default_rng(N + M)
    rows = np.unique(np.concatenate([np.arange(16), np.arange(N - 16, N), rng.integers(0, N, 224)]))
    y64, _ = oracle.matmul_f16(w[rows], s[rows], b[rows], x, K, len(rows), M, rounded=False)
    wd, sd, bd, xd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev)
    f = vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, f32out=True).cpu().numpy()
    y = bits16(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M))
    parity.check_f32(f[:, rows], y64)
    check_f16(y[:, rows], y64)
    z = vpq.qmv_w4g64_f16(wd, sd, bd, torch.zeros_like(xd), K, N, M, f32out=True)
    assert not z.any().item()                                  # all rows: zero activations give exactly zero


def test_qmv_f16_residual_and_gated(vpq, oracle, dev, D):
    K, ffn, M = 1024, 40, 2
    N = 2 * ffn
    w, s, b = f16_pack(N, K, 401)
    x = np.random.default_rng(402).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    res = np.random.default_rng(403).standard_normal((M, N)).astype(np.float16).view(np.uint16)
    y64, _ = oracle.matmul_f16(w, s, b, x, K, N, M, rounded=False)
    _, want_add = oracle.matmul_f16(w, s, b, x, K, N, M, rounded=False, residual=res)
    wd, sd, bd, xd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev)
    got_add = bits16(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, residual=dev16(res, dev)))
    plain = bits16(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M))
    redo = (plain.view(np.float16).astype(np.float32) + res.view(np.float16).astype(np.float32)).astype(np.float16)
    assert np.array_equal(got_add, redo.view(np.uint16))          # rounded, then added in binary16
    assert (np.abs(got_add.view(np.float16).astype(np.float64) - want_add.view(np.float16).astype(np.float64)) <=
            2e-3 * np.abs(y64) + 4e-3).all()
    for activation, fn in ((1, oracle.swiglu), (2, oracle.geglu)):
        g64, _ = fn(y64)
        got = bits16(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, activation=activation))
        check_f16(got, g64)


@pytest.mark.parametrize("K,N", [(2048, 38), (2560, 250), (5120, 1030), (17408, 66)])
def test_qmv_f16_one_row_streaming_kernel(vpq, oracle, dev, D, K, N):
    """One row of x on K % 512 == 0 takes the streaming decode kernel on binary16 arithmetic: plain, fp32 out,
    residual and both gated forms, ragged N, guard bands intact."""
    M = 1
    w, s, b = f16_pack(N, K, 600 + K + N)
    x = np.random.default_rng(601 + K).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    res = np.random.default_rng(602 + K).standard_normal((M, N)).astype(np.float16).view(np.uint16)
    y64, _ = oracle.matmul_f16(w, s, b, x, K, N, M, rounded=False)
    wd, sd, bd, xd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev)
    parity.check_f32(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, f32out=True).cpu().numpy(), y64)
    out = parity.Guarded((M, N), torch.float16, dev)
    vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    plain = bits16(out.view)
    check_f16(plain, y64)
    got_add = bits16(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, residual=dev16(res, dev)))
    redo = (plain.view(np.float16).astype(np.float32) + res.view(np.float16).astype(np.float32)).astype(np.float16)
    assert np.array_equal(got_add, redo.view(np.uint16))
    for activation, fn in ((1, oracle.swiglu), (2, oracle.geglu)):
        g64, _ = fn(y64)
        check_f16(bits16(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, M, activation=activation)), g64)
    # a pack whose scales sit off 16 bytes takes the general kernel: same values to the tolerance
    so = torch.empty(sd.numel() + 1, dtype=torch.float16, device=dev)[1:].view(sd.shape).copy_(sd)
    check_f16(bits16(vpq.qmv_w4g64_f16(wd, so, bd, xd, K, N, M)), y64)


@pytest.mark.parametrize("K,rows,M", [(2048, (64, 16, 16), 1), (4096, (520, 136), 1), (4096, (96, 40, 40, 8), 1), (1024, (48, 16, 16), 1),
                                      (2048, (64, 16), 3)])
def test_qmv_f16_grouped_launch(vpq, oracle, dev, D, K, rows, M):
    """Several packs sharing x (q|k|v, gate|up) on binary16 elements: each output has the bits of its own
    vpq_qmv_w4g64_f16 call (one launch where the streaming kernel takes the shape, separate calls otherwise)."""
    x = np.random.default_rng(801 + K).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    xd = dev16(x, dev)
    packs, singles = [], []
    for i, n in enumerate(rows):
        w, s, b = f16_pack(n, K, 810 + 7 * i + K)
        wd, sd, bd = D.u32(w, dev), dev16(s, dev), dev16(b, dev)
        packs.append((wd, sd, bd, n))
        singles.append(vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, n, M))
        y64, _ = oracle.matmul_f16(w, s, b, x, K, n, M, rounded=False)
        check_f16(bits16(singles[-1]), y64)
    outs = [parity.Guarded((M, n), torch.float16, dev) for n in rows]
    vpq.qmv_group_w4g64_f16(packs, xd, K, M, outs=[o.view for o in outs])
    torch.cuda.synchronize()
    for o, single in zip(outs, singles):
        o.assert_intact()
        assert torch.equal(o.view, single)


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (130, 320, 256), (257, 129, 512)])
def test_qmm_f16_dense_route(vpq, oracle, dev, D, M, N, K):
    w, s, b = f16_pack(N, K, 500 + M)
    x = np.random.default_rng(501 + M).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    y64, _ = oracle.matmul_f16(w, s, b, x, K, N, M, rounded=True)
    wd, sd, bd, xd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev)
    w_deq = torch.empty((N, K), dtype=torch.float16, device=dev)
    got = vpq.qmm_dense_route_w4g64_f16(wd, sd, bd, xd, K, N, M, w_deq)
    torch.cuda.synchronize()
    assert np.array_equal(bits16(w_deq), oracle.dequant_f16(w, s, b, K, N))
    check_f16(bits16(got), y64)
    kept = vpq.qmm_dense_route_w4g64_f16(wd, sd, bd, xd, K, N, M, w_deq, expand=False)
    assert torch.equal(kept, got)


@pytest.mark.parametrize("M,N,K", [(64, 64, 512), (130, 328, 1024), (257, 136, 512), (300, 520, 1536), (33, 200, 448),
                                   (513, 130, 1088), (2304, 8192, 512)])
def test_qmm_f16_fused(vpq, oracle, dev, D, M, N, K):
    """The fused GEMM on binary16 elements (weight tile = f16(s q + b), f16 MFMA, fp32 accumulation): against
    the oracle's rounded-weight twin, bit for bit against the dequant-once route (same tiles, same order of
    accumulation), gated stores against the oracle's activations, guard bands intact."""
    w, s, b = f16_pack(N, K, 700 + M)
    x = np.random.default_rng(701 + M).standard_normal((M, K)).astype(np.float16).view(np.uint16)
    # rows are independent: the shape with enough tiles for the large-tile kernel is checked on a sample of them
    rows = np.arange(M) if M * N * K < 2e9 else np.r_[0:40, 1000:1024, M - 40:M]
    y64, _ = oracle.matmul_f16(w, s, b, x[rows], K, N, len(rows), rounded=True)
    wd, sd, bd, xd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev)
    out = parity.Guarded((M, N), torch.float16, dev)
    vpq.qmm_w4g64_f16(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    check_f16(bits16(out.view)[rows], y64)
    w_deq = torch.empty((N, K), dtype=torch.float16, device=dev)
    assert torch.equal(out.view, vpq.qmm_dense_route_w4g64_f16(wd, sd, bd, xd, K, N, M, w_deq))
    # the element type is live: the bf16 kernel on the same bits gives something else
    assert not torch.equal(out.view.view(torch.int16),
                           vpq.qmm_w4g64(wd, sd.view(torch.bfloat16), bd.view(torch.bfloat16), xd.view(torch.bfloat16),
                                         K, N, M).view(torch.int16))
    for activation, fn in ((1, oracle.swiglu), (2, oracle.geglu)):
        g64, _ = fn(y64)
        og = parity.Guarded((M, N // 2), torch.float16, dev)
        vpq.qmm_w4g64_f16(wd, sd, bd, xd, K, N, M, activation=activation, out=og.view)
        torch.cuda.synchronize()
        og.assert_intact()
        check_f16(bits16(og.view)[rows], g64)


@pytest.mark.parametrize("M,N,K,r", [(64, 64, 512, 16), (130, 328, 1024, 32), (300, 520, 1536, 48), (257, 136, 512, 128),
                                     (96, 200, 1024, 384), (70, 264, 320, 32), (2304, 8192, 512, 32), (100, 136, 512, 8), (66, 72, 320, 24)])
def test_qmm_f16_fused_with_adapter(vpq, oracle, dev, D, M, N, K, r):
    """The adapter on binary16 elements: t bit for bit against the oracle where the fp32 sum is not at a rounding
    boundary (at most a handful of elements one step off), the fused GEMM against the oracle's twin, alpha = 0 the
    plain GEMM's bits, guard bands intact."""
    w, s, b = f16_pack(N, K, 800 + M)
    rng = np.random.default_rng(801 + M)
    x = rng.standard_normal((M, K)).astype(np.float16).view(np.uint16)
    A = (0.05 * rng.standard_normal((r, K))).astype(np.float16).view(np.uint16)
    B = (0.05 * rng.standard_normal((N, r))).astype(np.float16).view(np.uint16)
    alpha = 0.75
    wd, sd, bd, xd, Ad, Bd = D.u32(w, dev), dev16(s, dev), dev16(b, dev), dev16(x, dev), dev16(A, dev), dev16(B, dev)
    rows = np.arange(M) if M * N * K < 2e9 else np.r_[0:40, 1000:1024, M - 40:M]
    t_want = oracle.lora_t_f16(x[rows], A, len(rows), K, r, alpha)
    t_got = parity.Guarded((M, r), torch.float16, dev)
    vpq.lora_a_f16(xd, Ad, M, K, r, alpha, out=t_got.view)
    torch.cuda.synchronize()
    t_got.assert_intact()
    tg = bits16(t_got.view)[rows]
    off = tg != t_want
    assert off.mean() <= 0.01
    assert np.abs(tg.view(np.float16).astype(np.float64) - t_want.view(np.float16).astype(np.float64)).max() <= \
        2.0 ** -10 * np.abs(t_want.view(np.float16).astype(np.float64)).max()
    # the GEMM against the oracle fed with the t the device produced (its own rounding-boundary cases included)
    y64, _ = oracle.qmm_lora_f16(w, s, b, x[rows], K, N, len(rows), tg, B, r)
    out = parity.Guarded((M, N), torch.float16, dev)
    t_ws = parity.Guarded((M, r), torch.float16, dev)
    vpq.qmm_lora_w4g64_f16(wd, sd, bd, xd, K, N, M, Ad, Bd, r, alpha, out=out.view, t_ws=t_ws.view)
    torch.cuda.synchronize()
    out.assert_intact()
    t_ws.assert_intact()
    assert torch.equal(t_ws.view, t_got.view)
    check_f16(bits16(out.view)[rows], y64)
    base64, _ = oracle.matmul_f16(w, s, b, x[rows], K, N, len(rows), rounded=True)
    assert np.sqrt(((y64 - base64) ** 2).sum() / (y64 ** 2).sum()) > 1e-3          # the adapter is live
    plain = vpq.qmm_w4g64_f16(wd, sd, bd, xd, K, N, M)
    assert torch.equal(vpq.qmm_lora_w4g64_f16(wd, sd, bd, xd, K, N, M, Ad, Bd, r, 0.0), plain)
    L = vpq.load()
    p = out.view.data_ptr()
    assert L.vpq_qmm_lora_w4g64_f16(None, p, p, p, p, p, K, N, M, p, p, 36, 1.0, p) == -2
    assert L.vpq_qmm_lora_w4g64_f16(None, p, p, p, p, p, K, N, M, p, p, r, 1.0, None) == -4
    assert L.vpq_lora_a_f16(None, p, p, p, M, K, 528, 1.0) == -2


def test_qmm_f16_fused_rejects(vpq, dev):
    L = vpq.load()
    p = torch.zeros(1 << 16, dtype=torch.int32, device=dev).data_ptr()
    assert L.vpq_qmm_w4g64_f16(None, p, p, p, p, p, 440, 8, 4, 0) == -2         # K % 64 != 0
    assert L.vpq_qmm_w4g64_f16(None, p, p, p, p, p, 512, 7, 4, 1) == -2         # gated needs an even N
    assert L.vpq_qmm_w4g64_f16(None, p, p, p, p, p, 512, 8, 4, 3) == -2
    assert L.vpq_qmm_w4g64_f16(None, p, p, p, None, p, 512, 8, 4, 0) == -1


def test_f16_entries_reject_bad_arguments(vpq, dev):
    L = vpq.load()
    p = torch.zeros(4096, dtype=torch.int32, device=dev).data_ptr()
    assert L.vpq_dequant_w4g64_f16(None, p, p, p, None, 64, 8) == -1
    assert L.vpq_qmv_w4g64_f16(None, p, p, p, p, p, 60, 8, 1, None) == -2
    assert L.vpq_qmv_w4g64_f16(None, p, p, p, p, p, 64, 8, 17, None) == -2
    assert L.vpq_qmv_gated_w4g64_f16(None, p, p, p, p, p, 64, 7, 1, 1) == -2
    assert L.vpq_qmm_dense_route_w4g64_f16(None, p, p, p, p, p, 64, 8, 4, None, 1) == -4


@pytest.mark.parametrize("group", [64, 32])
@pytest.mark.parametrize("M,N,K", [(1, 8, 64), (70, 136, 320), (300, 264, 1024)])
def test_w8_on_binary16_elements_expansion_and_dense_route(vpq, oracle, dev, D, group, M, N, K):
    """The half build's affine_dequant_w8g64 / _w8g32 and affine_qmm_steel_w8g64 / _w8g32 (what the reference's codec
    runs, moss/metal-moss-codec.cc:181-183, 579-581): the expansion bit for bit against the oracle, the GEMM by the
    dequant-once route against float64 of x . W^T with W that expansion, the kept expansion the same bits."""
    rng = np.random.default_rng(9300 + M + group)
    w = rng.integers(0, 2**32, size=(N, K // 4), dtype=np.uint32)
    s = rng.uniform(0.0003, 0.0012, size=(N, K // group)).astype(np.float16)
    b = (-128.0 * s.astype(np.float32) * rng.uniform(0.9, 1.1, size=s.shape)).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dense = oracle.dequant8_f16(w, s.view(np.uint16), b.view(np.uint16), K, N, group=group)
    wd = torch.from_numpy(w.view(np.int32)).to(dev)
    sd, bd, xd = torch.from_numpy(s).to(dev), torch.from_numpy(b).to(dev), torch.from_numpy(x).to(dev)
    got = vpq.dequant_w8_f16(wd, sd, bd, K, N, group=group)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint16), dense)
    w_deq = torch.empty((N, K), dtype=torch.float16, device=dev)
    out = parity.Guarded((M, N), torch.float16, dev)
    vpq.qmm_dense_route_w8_f16(wd, sd, bd, xd, K, N, M, w_deq, group=group, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    assert np.array_equal(w_deq.cpu().numpy().view(np.uint16), dense)
    want = x.astype(np.float64) @ dense.view(np.float16).astype(np.float64).T
    y = out.view.cpu().numpy().astype(np.float64)
    # one binary16 rounding of an fp32 sum: 2^-11 relative, plus the sum's own error where it cancels
    mag = np.abs(x.astype(np.float64)) @ np.abs(dense.view(np.float16).astype(np.float64)).T
    assert (np.abs(y - want) <= 2.0 ** -11 * np.abs(want) + 64 * 2.0 ** -24 * mag + 2.0 ** -24).all()
    kept = vpq.qmm_dense_route_w8_f16(wd, sd, bd, xd, K, N, M, w_deq, group=group, expand=False)
    assert torch.equal(kept, out.view)
    L = vpq.load()
    p = out.view.data_ptr()
    assert L.vpq_dequant_w8_f16(None, 48, p, p, p, p, K, N) == -2
    assert L.vpq_qmm_dense_route_w8_f16(None, group, p, p, p, p, p, K, N, M, None, 1) == -4
    assert L.vpq_qmm_dense_route_w8_f16(None, group, p, p, p, p, p, K + 8, N, M, p, 1) == -2
