"""GPU parity: dense expansion (bit-exact) and QMV (every kernel variant) against
the CPU oracle, through the C ABI.  Cases follow the reference's own tests
(tests/unit-tests/metal-lm/quant-gemv.cc): K tails, padded/garbage rows, batched
rows, residual add, and the benchmark's full shapes."""
import numpy as np
import pytest
import torch

from tests import parity
from tests.golden import refgen
from vpipe_amd import capi, synth

pytestmark = pytest.mark.gpu

SIMPLE, MFMA, AUTO = capi.VPQ_QMV_SIMPLE, capi.VPQ_QMV_MFMA, capi.VPQ_QMV_AUTO
FLOW = capi.VPQ_QMV_FLOW


def stage(D, dev, w, s, b, x=None):
    out = [D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev)]
    if x is not None:
        out.append(D.bf16(x, dev))
    return out


# ---- a1: dequant is bit-exact -------------------------------------------------

@pytest.mark.parametrize("N,K", [(1, 64), (33, 192), (257, 3840), (4096, 4096)])
def test_dequant_bit_exact(vpq, oracle, dev, D, N, K):
    w, s, b = synth.make_weight(N, K, 7 + N)
    wd, sd, bd = stage(D, dev, w, s, b)
    out = parity.Guarded((N, K), torch.bfloat16, dev)
    vpq.dequant_w4g64(wd, sd, bd, K, N, out=out.view)
    torch.cuda.synchronize()
    got = D.bits(out.view)
    assert np.array_equal(got, oracle.dequant_bf16(w, s, b, K, N))
    out.assert_intact()


def test_dequant_every_code_against_every_scale(vpq, oracle, dev, D):
    # all 16 codes x a sweep of 2^16 (scale, bias) bit patterns: the bf16 rounding
    # of fp32(s*q+b) must agree everywhere, including ties and cancellation.
    K = 64
    N = 1 << 16
    rng = np.random.default_rng(99)
    w = np.tile(np.array([0x76543210, 0xFEDCBA98], dtype=np.uint32), (N, K // 16))
    s = np.arange(N, dtype=np.uint32).astype(np.uint16)[:, None]          # every bf16 pattern once
    s = np.where((s & 0x7F80) == 0x7F80, np.uint16(0x3C00), s)            # drop inf/nan patterns
    bvals = synth.f32_to_bf16_bits((-8.0 * synth.bf16_bits_to_f32(s) *
                                    (1 + 0.05 * rng.standard_normal(s.shape))).astype(np.float32))
    bvals = np.where((bvals & 0x7F80) == 0x7F80, np.uint16(0), bvals)
    wd, sd, bd = stage(D, dev, w, s, bvals)
    got = D.bits(vpq.dequant_w4g64(wd, sd, bd, K, N))
    want = oracle.dequant_bf16(w, s, bvals, K, N)
    finite = np.isfinite(synth.bf16_bits_to_f32(want))
    assert np.array_equal(got[finite], want[finite])


@pytest.mark.parametrize("vocab,H,T", [(37, 192, 8), (1000, 4096, 1), (151936, 1024, 300)])
def test_embed_gather_rows_are_bit_exact(vpq, oracle, dev, D, vocab, H, T):
    # dequant_embed_gather (gpu-kernels/metal/ops/llm_elementwise.metal:1676-1701): a gathered row
    # is that row of the dense table, bit for bit; ids outside the table give zero rows
    w, s, b = synth.make_weight(vocab, H, 400 + H)
    rng = np.random.default_rng(T)
    ids = rng.integers(0, vocab, size=T).astype(np.int32)
    ids[0], ids[-1] = vocab - 1, 0
    if T >= 8:
        ids[3], ids[4] = -1, vocab
    wd, sd, bd = stage(D, dev, w, s, b)
    out = parity.Guarded((T, H), torch.bfloat16, dev)
    vpq.embed_gather_w4g64(torch.from_numpy(ids).to(dev), wd, sd, bd, H, vocab, out=out.view)
    torch.cuda.synchronize()
    assert np.array_equal(D.bits(out.view), oracle.embed_gather(ids, w, s, b, H, vocab))
    out.assert_intact()


# ---- a2/a3/a4: QMV --------------------------------------------------------------

SMALL = [
    # K, N, M
    (512, 16, 1), (512, 16, 4), (1024, 48, 2), (1024, 40, 3), (2048, 160, 5),
    (1536, 33, 7), (512, 95, 8), (2560, 64, 16), (4096, 16, 13),
]


@pytest.mark.parametrize("variant", [SIMPLE, MFMA, AUTO])
@pytest.mark.parametrize("K,N,M", SMALL)
def test_qmv_small_shapes(vpq, oracle, dev, D, K, N, M, variant):
    w, s, b = synth.make_weight(N, K, 1000 + K + N)
    x = synth.make_act(M, K, 2000 + K + M)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    ws = vpq.qmv_workspace(K, N, M)
    f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, ws=ws, variant=variant, f32out=True)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, ws=ws, variant=variant)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), y64)
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    assert not ws[:256].any().item()                # arrival counters are left zeroed


ROWS_SHAPES = [
    # K, N, M: K below, at and above one pass of 2048, not a multiple of it; N not a multiple of the rows per wavefront
    (64, 5, 1), (512, 16, 2), (1024, 33, 1), (2048, 95, 2), (3840, 16, 1), (4096, 16 * 50 + 3, 1), (5120, 64, 2),
    (12288, 160, 1), (17408, 33, 2),
]


@pytest.mark.parametrize("K,N,M", ROWS_SHAPES)
def test_qmv_row_streaming_kernel(vpq, oracle, dev, D, K, N, M):
    w, s, b = synth.make_weight(N, K, 8000 + K + N)
    x = synth.make_act(M, K, 8100 + K + M)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=capi.VPQ_QMV_ROWS, f32out=True)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, variant=capi.VPQ_QMV_ROWS)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), y64)
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    res = synth.make_act(M, N, 8200 + N)
    got = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, residual=D.bf16(res, dev), variant=capi.VPQ_QMV_ROWS))
    want = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(D.bits(out.view)) + synth.bf16_bits_to_f32(res))
    assert np.array_equal(got, want)


def _packer_case(kind, N, K, seed):
    """bf16-representable fp32 weights that exercise one corner of affine_quant_w4_g64
    (gpu-kernels/metal/quant/affine_dequant.metal:243-285)."""
    rng = np.random.default_rng(seed)
    if kind == "gauss":
        v = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    elif kind == "ties":
        # mn = 0, mx = 15 in every group, so scale = 1 exactly and values at j + 0.5 sit on rounding ties:
        # Metal's round() takes them away from zero
        v = rng.integers(0, 31, size=(N, K)).astype(np.float32) * 0.5
        v[:, 0::64] = 0.0
        v[:, 1::64] = 15.0
    elif kind == "constant":
        # constant groups: scale 0, inv 0, every code 0; every other group is ordinary
        v = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
        for g in range(0, K // 64, 2):
            v[:, g * 64:(g + 1) * 64] = rng.standard_normal((N, 1)).astype(np.float32)
    elif kind == "outliers":
        v = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
        v[rng.random((N, K)) < 0.01] *= 40.0
    else:
        raise ValueError(kind)
    return synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(v))


@pytest.mark.parametrize("kind,N,K,clip", [
    ("gauss", 96, 1024, 1.0), ("gauss", 4096, 4096, 1.0), ("gauss", 33, 320, 0.9), ("outliers", 257, 2048, 0.75),
    ("ties", 64, 512, 1.0), ("constant", 48, 1024, 1.0), ("constant", 48, 1024, 0.8), ("gauss", 1, 64, 1.0),
])
def test_packer_matches_the_oracle_bit_for_bit(vpq, oracle, dev, D, kind, N, K, clip):
    # codes, F16 scales and F16 zero points of the device packer == the CPU restatement, for clipped ranges,
    # exact rounding ties, constant groups (scale 0) and a layer-sized matrix
    v = _packer_case(kind, N, K, 600 + N + K)
    codes, s16, b16 = oracle.quantize(v, K, N, clip=clip)
    wd, sd, bd = vpq.quantize_w4g64(D.bf16(synth.f32_to_bf16_bits(v), dev), K, N, clip=clip)
    torch.cuda.synchronize()
    assert np.array_equal(wd.cpu().numpy().view(np.uint32), codes)
    assert np.array_equal(sd.cpu().numpy().view(np.uint16), s16)
    assert np.array_equal(bd.cpu().numpy().view(np.uint16), b16)
    if kind == "ties":
        # the known answer itself: scale 1, zero point 0, code = round-half-away(v)
        q = (codes[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15
        assert np.array_equal(q.reshape(N, K), np.minimum(np.floor(v + 0.5), 15).astype(np.uint32))
    if kind == "constant":
        q = (codes[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15
        assert not q.reshape(N, K // 64, 64)[:, 0::2].any()
        assert not s16.reshape(N, K // 64)[:, 0::2].any()


@pytest.mark.parametrize("bits,group", [(4, 64), (4, 32), (8, 64), (8, 32)])
@pytest.mark.parametrize("kind,N,K,clip,f16", [("gauss", 96, 1024, 1.0, False), ("gauss", 33, 320, 0.9, True),
                                               ("outliers", 257, 2048, 0.75, False), ("constant", 48, 1024, 1.0, True)])
def test_packer_at_every_width_and_group(vpq, oracle, dev, D, bits, group, kind, N, K, clip, f16):
    # affine_quant_w4_g64 / _w4_g32 / _w8_g64 / _w8_g32 (gpu-kernels/metal/quant/affine_dequant.metal:243-301) over a
    # bf16 or a binary16 source: codes, F16 scales and F16 zero points bit for bit against the oracle
    v = _packer_case(kind, N, K, 700 + N + K + bits + group)
    if f16:
        v = v.astype(np.float16).astype(np.float32)
        src = torch.from_numpy(v.astype(np.float16)).to(dev)
    else:
        src = D.bf16(synth.f32_to_bf16_bits(v), dev)
    codes, s16, b16 = oracle.quantize(v, K, N, clip=clip, bits=bits, group=group)
    wd, sd, bd = vpq.quantize(src, K, N, bits=bits, group=group, clip=clip)
    torch.cuda.synchronize()
    assert np.array_equal(wd.cpu().numpy().view(np.uint32), codes)
    assert np.array_equal(sd.cpu().numpy().view(np.uint16), s16)
    assert np.array_equal(bd.cpu().numpy().view(np.uint16), b16)
    assert codes.any() or kind == "constant"
    L = vpq.load()
    p = src.data_ptr()
    assert L.vpq_quantize(None, 5, group, 0, p, p, p, p, K, N, 1.0) == -2
    assert L.vpq_quantize(None, bits, 48, 0, p, p, p, p, K, N, 1.0) == -2
    assert L.vpq_quantize(None, bits, group, 0, p, p, p, p, K + 8, N, 1.0) == -2


FLOW_SHAPES = [
    # K, N: one to nine slices of 2048, K not a multiple of 2048 (idle lanes in the last slice), every plan of
    # slices per wavefront x K parts (2560: 2x1, 4096: 2x1, 5120: 3x1, 8192: 4x1, 12288: 3x2, 14336: 4x2, 17408: 3x3),
    # N not a multiple of the rows per wavefront / workgroup
    (2048, 5), (2560, 33), (4096, 16 * 50 + 3), (5120, 64), (8192, 95), (12288, 161), (14336, 18), (17408, 33),
    (24576, 7), (4096, 1),
]


@pytest.mark.parametrize("K,N", FLOW_SHAPES)
def test_qmv_flow_kernel(vpq, oracle, dev, D, K, N):
    M = 1
    w, s, b = synth.make_weight(N, K, 8300 + K + N)
    x = synth.make_act(M, K, 8400 + K)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=FLOW, f32out=True)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, variant=FLOW)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), y64)
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    # AUTO takes this kernel at M = 1 below lm_head-sized packs: same bits
    assert np.array_equal(D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=AUTO)), D.bits(out.view))
    res = synth.make_act(M, N, 8500 + N)
    got = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, residual=D.bf16(res, dev), variant=FLOW))
    want = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(D.bits(out.view)) + synth.bf16_bits_to_f32(res))
    assert np.array_equal(got, want)


def test_qmv_flow_kernel_refuses_what_it_does_not_take(vpq, dev, D):
    w, s, b = synth.make_weight(16, 1024, 1)
    wd, sd, bd = stage(D, dev, w, s, b)
    x = D.bf16(synth.make_act(2, 1024, 2), dev)
    with pytest.raises(capi.VpqError):
        vpq.qmv_w4g64(wd, sd, bd, x[:1].contiguous(), 1024, 16, 1, variant=FLOW)      # K below one slice
    w, s, b = synth.make_weight(16, 2048, 1)
    wd, sd, bd = stage(D, dev, w, s, b)
    x = D.bf16(synth.make_act(2, 2048, 2), dev)
    with pytest.raises(capi.VpqError):
        vpq.qmv_w4g64(wd, sd, bd, x, 2048, 16, 2, variant=FLOW)                        # two rows of x


def test_qmv_flow_one_hot_reads_back_weights_exactly(vpq, oracle, dev, D):
    # x = e_k: y[n] must be fp32(s*q+b) exactly (layout, nibble order, K parts, un-rounded weights)
    K, N = 12288, 10
    w, s, b = synth.make_weight(N, K, 6)
    d32 = oracle.dequant_f32(w, s, b, K, N)
    wd, sd, bd = stage(D, dev, w, s, b)
    for k in [0, 1, 4, 7, 8, 31, 32, 63, 64, 2047, 2048, 6143, 6144, 6145, 9999, K - 1]:
        x = np.zeros((1, K), dtype=np.float32)
        x[0, k] = 1.0
        y = vpq.qmv_w4g64(wd, sd, bd, D.bf16(synth.f32_to_bf16_bits(x), dev), K, N, 1, variant=FLOW, f32out=True)
        assert np.array_equal(y.cpu().numpy()[0], d32[:, k]), k


STREAM_SHAPES = [
    # K, N, M: one and several slices per wavefront, ragged last tile, more tiles than
    # workgroups (each workgroup walks several tiles), every M the kernel takes
    (512, 16, 1), (1024, 33, 2), (4096, 95, 3), (4096, 16 * 800 + 5, 1), (8192, 48, 4),
    (12288, 160, 1), (12288, 16 * 300, 2), (17408, 64, 1), (17408, 33, 2), (24576, 17, 1),
]


RING_SHAPES = STREAM_SHAPES + [
    # every M (1, 2 and 4 accumulator registers), ragged N, several tiles per workgroup,
    # one to five slices per wavefront
    (512, 16, 16), (1024, 40, 5), (2048, 33, 8), (4096, 16 * 1030 + 7, 4), (5120, 16 * 600, 9), (20480, 72, 16),
    (4096, 16 * 2100 + 3, 1), (12288, 16 * 700 + 9, 3),
    # many tiles per workgroup with x in registers: 12 at 6 rows, the cap of 8 at 12 rows
    (1024, 16 * 3000, 6), (512, 16 * 2100 + 5, 12),
    # 3 and 4 rows over a wide matrix take the two-register form
    (1024, 16 * 1400 + 2, 3), (512, 16 * 1300, 4),
    # ... and so do 2 rows where that saves a generation of workgroups (1300 tiles: 6 per workgroup, one generation)
    (512, 16 * 1300, 2), (1536, 16 * 1088 + 7, 2),
]


@pytest.mark.parametrize("K,N,M", RING_SHAPES)
def test_qmv_ring_kernel(vpq, oracle, dev, D, K, N, M):
    w, s, b = synth.make_weight(N, K, 6000 + K + N)
    x = synth.make_act(M, K, 7000 + K + M)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=capi.VPQ_QMV_RING, f32out=True)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, variant=capi.VPQ_QMV_RING)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), y64)
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    # bit-reproducible: a second launch gives the same bits
    f2 = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=capi.VPQ_QMV_RING, f32out=True)
    assert torch.equal(f, f2)


@pytest.mark.parametrize("K,N,M", STREAM_SHAPES)
def test_qmv_streaming_kernel(vpq, oracle, dev, D, K, N, M):
    w, s, b = synth.make_weight(N, K, 4000 + K + N)
    x = synth.make_act(M, K, 5000 + K + M)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=capi.VPQ_QMV_STREAM, f32out=True)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, variant=capi.VPQ_QMV_STREAM)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), y64)
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    # same inputs through the one-item-per-wavefront kernel: same arithmetic, so the fp32
    # results agree to accumulation-order noise
    f2 = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=MFMA, f32out=True)
    rms = float(np.sqrt((y64 ** 2).mean()))
    assert (f - f2).abs().max().item() <= 1e-5 * rms + 1e-6


@pytest.mark.parametrize("K,N,M", [(1024, 33, 16), (4096, 64, 5), (8192, 48, 2), (17408, 200, 16), (2560, 16, 9)])
def test_qmv_ring_split_k_matches_oracle_and_is_deterministic(vpq, oracle, dev, D, K, N, M):
    """The ring kernel with K split across workgroups (fp32 planes + fold launch): oracle parity with and without a
    residual, the fp32 result before the store, the same bits run to run, and the planes' guard bytes intact."""
    w, s, b = synth.make_weight(N, K, 41 + K)
    x = synth.make_act(M, K, 42 + K)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    ws = parity.Guarded((vpq.load().vpq_qmv_workspace_bytes(K, N, M) // 4,), torch.float32, dev)
    ws.view.fill_(float("nan"))                     # the planes need no initial content
    runs = []
    for _ in range(3):
        out = parity.Guarded((M, N), torch.bfloat16, dev)
        vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, ws=ws.view, variant=capi.VPQ_QMV_RING_SPLITK)
        torch.cuda.synchronize()
        out.assert_intact()
        ws.assert_intact()
        runs.append(D.bits(out.view).copy())
    parity.check_bf16(runs[0], y64, yb)
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, ws=ws.view, variant=capi.VPQ_QMV_RING_SPLITK, f32out=True)
    parity.check_f32(f.cpu().numpy(), y64)
    # the unsplit kernel agrees to accumulation-order noise
    f1 = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=capi.VPQ_QMV_RING, f32out=True)
    rms = float(np.sqrt((y64 ** 2).mean()))
    assert (f - f1).abs().max().item() <= 1e-5 * rms + 1e-6
    # residual: added to the rounded product, rounded again (affine_qmv.metal:347-363)
    res = synth.make_act(M, N, 43 + K)
    got = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, residual=D.bf16(res, dev), ws=ws.view, variant=capi.VPQ_QMV_RING_SPLITK)
    want = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(runs[0]) + synth.bf16_bits_to_f32(res))
    assert np.array_equal(D.bits(got), want)
    # a workspace too small for the planes is refused
    with pytest.raises(capi.VpqError) as e:
        vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, ws=ws.view[: M * N], variant=capi.VPQ_QMV_RING_SPLITK)
    assert e.value.status == capi.VPQ_ERR_WORKSPACE


def test_qmv_one_hot_reads_back_weights_exactly(vpq, oracle, dev, D):
    # x = e_k: y[n] must be bf16(fp32(s*q+b)) EXACTLY for every kernel -- layout,
    # nibble order and the un-rounded-weight arithmetic in one known answer.
    K, N = 1024, 32
    w, s, b = synth.make_weight(N, K, 5)
    d32 = oracle.dequant_f32(w, s, b, K, N)
    wd, sd, bd = stage(D, dev, w, s, b)
    for variant in (SIMPLE, MFMA, capi.VPQ_QMV_STREAM):
        for k in [0, 1, 4, 7, 8, 15, 16, 63, 64, 511, 512, 777, K - 1]:
            x = np.zeros((1, K), dtype=np.float32)
            x[0, k] = 1.0
            y = vpq.qmv_w4g64(wd, sd, bd, D.bf16(synth.f32_to_bf16_bits(x), dev), K, N, 1,
                              variant=variant, f32out=True)
            got = y.cpu().numpy()[0]
            # the MFMA kernel forms s*(128+q) - 128 s ... in fp32: exact for one-hot x
            assert np.array_equal(got, d32[:, k]), (variant, k)


def test_qmv_reference_tail_case(vpq, oracle, dev, D):
    """metal_lm_smoke.qmv_w4g32_matches_cpu inputs (quant-gemv.cc:215-253) at g64:
    K = 3840 is not a multiple of 512, x is padded with non-zero values to 4096 and
    a garbage weight row follows row N-1.  Bar of the reference: max
    |d|/(|ref|+1e-2) < 0.03."""
    N, K = 16, 3840
    c = refgen.knuth_qmv_case(N, K, group=64)
    s = synth.f32_to_bf16_bits(c["scales"])
    b = synth.f32_to_bf16_bits(c["biases"])
    x = synth.f32_to_bf16_bits(c["x"])[None, :]              # 4096 values, only K are used
    y64, yb = oracle.qmv(c["packed"][:N], s, b, x[:, :K], K, N, 1)
    wd = D.u32(c["packed"], dev)                             # N+1 rows on the device
    y = vpq.qmv_w4g64(wd, D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev), K, N, 1)
    got = synth.bf16_bits_to_f32(D.bits(y))[0].astype(np.float64)
    assert (np.abs(got - y64[0]) / (np.abs(y64[0]) + 1e-2)).max() < 0.03
    parity.check_bf16(D.bits(y), y64, yb)


def test_qmv_batched_rows_are_independent(vpq, oracle, dev, D):
    # the batched tiles of the reference are bit-identical per row to the M=1 kernel
    # (affine_qmv.metal:1563-1564); here: row m of an M-row call == the M=1 call on row m.
    K, N, M = 2048, 64, 7
    w, s, b = synth.make_weight(N, K, 77)
    x = synth.make_act(M, K, 78)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    for variant in (SIMPLE, MFMA):
        full = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=variant))
        for m in range(M):
            one = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd[m:m + 1].contiguous(), K, N, 1, variant=variant))
            assert np.array_equal(full[m], one[0]), (variant, m)


def test_qmv_ring_rows_are_independent(vpq, oracle, dev, D):
    # the same contract for the ring kernel, within each of its register forms (2..4, 5..8, 9..16 rows of x):
    # a row's result depends on that row of x only -- not on its position, not on its neighbours
    K, N = 2048, 80
    w, s, b = synth.make_weight(N, K, 79)
    wd, sd, bd = stage(D, dev, w, s, b)
    for M in (3, 7, 12):
        x = synth.make_act(M, K, 80 + M)
        xd = D.bf16(x, dev)
        full = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=capi.VPQ_QMV_RING))
        perm = np.random.default_rng(M).permutation(M)
        shuffled = D.bits(vpq.qmv_w4g64(wd, sd, bd, D.bf16(x[perm], dev), K, N, M, variant=capi.VPQ_QMV_RING))
        assert np.array_equal(shuffled, full[perm]), M
        fewer = D.bits(vpq.qmv_w4g64(wd, sd, bd, D.bf16(x[:M - 1], dev), K, N, M - 1, variant=capi.VPQ_QMV_RING))
        assert np.array_equal(fewer, full[:M - 1]), M
        other = x.copy()
        other[1:] = synth.make_act(M - 1, K, 99 + M)
        mixed = D.bits(vpq.qmv_w4g64(wd, sd, bd, D.bf16(other, dev), K, N, M, variant=capi.VPQ_QMV_RING))
        assert np.array_equal(mixed[0], full[0]), M


def test_qmv_residual_add(vpq, oracle, dev, D):
    K, N, M = 1024, 48, 2
    w, s, b = synth.make_weight(N, K, 61)
    x = synth.make_act(M, K, 62)
    res = synth.make_act(M, N, 63)
    _, yr = oracle.qmv(w, s, b, x, K, N, M, residual=res)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    for variant in (SIMPLE, MFMA):
        y = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, residual=D.bf16(res, dev), variant=variant)
        assert parity.bf16_ulp_distance(D.bits(y), yr).max() <= 1


DECODE_LAYER = [(4096, 4096), (4096, 1024), (4096, 12288), (12288, 4096)]


@pytest.mark.parametrize("K,N", DECODE_LAYER)
def test_qmv_decode_layer_shapes_full(vpq, oracle, dev, D, K, N):
    w, s, b = synth.make_weight(N, K, 0x5EED0002 + N)
    x = synth.make_act(1, K, 0x5EED0102 + K)
    y64, yb = oracle.qmv(w, s, b, x, K, N, 1)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    ws = vpq.qmv_workspace(K, N, 1)
    for variant in (AUTO, SIMPLE):
        f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, 1, ws=ws, variant=variant, f32out=True)
        y = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, 1, ws=ws, variant=variant)
        parity.check_f32(f.cpu().numpy(), y64)
        parity.check_bf16(D.bits(y), y64, yb)


@pytest.mark.parametrize("K,N", [(5120, 5120), (5120, 17408), (17408, 5120), (5120, 151936)])
@pytest.mark.parametrize("M", [1, 2, 4, 8, 16])
def test_qmv_small_batch_shapes_row_sample(vpq, oracle, dev, D, K, N, M):
    # full-size launch; the oracle evaluates a sample of output rows (first and last
    # tiles included), since every output row depends on its own weight row only.
    w, s, b = synth.make_weight(N, K, 0x5EED0003 + N)
    x = synth.make_act(M, K, 0x5EED0103 + K + M)
    rng = np.random.default_rng(N + M)
    rows = np.unique(np.concatenate([np.arange(16), np.arange(N - 16, N), rng.integers(0, N, 224)]))
    y64, yb = oracle.qmv(w[rows], s[rows], b[rows], x, K, len(rows), M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    ws = vpq.qmv_workspace(K, N, M)
    f = vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, ws=ws, f32out=True).cpu().numpy()
    y = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, ws=ws))
    parity.check_f32(f[:, rows], y64)
    parity.check_bf16(y[:, rows], y64, yb)
    # size-independent property over ALL rows: zero activations give exactly zero
    z = vpq.qmv_w4g64(wd, sd, bd, torch.zeros_like(xd), K, N, M, ws=ws, f32out=True)
    assert not z.any().item()


def test_linear_entrance_routes_by_rows(vpq, oracle, dev, D):
    # qmm_auto_ and its ladder (metal-qwen-model.cc:3839-4033): GEMV arithmetic for few rows -- one
    # launch up to 16, slabs of 16 rows up to 64 -- and the GEMM above
    K, N = 1024, 80
    w, s, b = synth.make_weight(N, K, 91)
    wd, sd, bd = stage(D, dev, w, s, b)
    for M, fn in ((16, oracle.qmv), (17, oracle.qmv), (41, oracle.qmv), (64, oracle.qmv), (65, oracle.qmm)):
        x = synth.make_act(M, K, 92 + M)
        y64, yb = fn(w, s, b, x, K, N, M)
        out = parity.Guarded((M, N), torch.bfloat16, dev)
        vpq.linear_w4g64(wd, sd, bd, D.bf16(x, dev), K, N, M, out=out.view)
        torch.cuda.synchronize()
        parity.check_bf16(D.bits(out.view), y64, yb)
        out.assert_intact()
        if fn is oracle.qmv:
            # a slab is the plain QMV call on its rows: same bits
            ref = torch.cat([vpq.qmv_w4g64(wd, sd, bd, D.bf16(x[m0:m0 + 16], dev), K, N, min(16, M - m0))
                             for m0 in range(0, M, 16)])
            assert torch.equal(out.view, ref)


@pytest.mark.parametrize("K,Ns,M", [(4096, (4096, 1024, 1024), 1), (4096, (12288, 12288), 1), (1024, (48, 33, 16, 95), 3),
                                    (2048, (64,), 2), (12288, (160, 4096), 16), (3840, (64, 32), 1), (3840, (64, 160, 410), 2),
                                    (1984, (240, 80), 5)])
def test_qmv_grouped_launch_equals_separate_launches(vpq, oracle, dev, D, K, Ns, M):
    # q|k|v and gate|up in one launch (the reference's fused QKV GEMV, affine_qmv.metal:405-516):
    # bit-identical to separate launches, and within tolerance of the oracle
    packs, refs = [], []
    x = synth.make_act(M, K, 9000 + K + M)
    xd = D.bf16(x, dev)
    for i, N in enumerate(Ns):
        w, s, b = synth.make_weight(N, K, 8000 + 7 * i + N)
        packs.append((D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), N))
        refs.append(oracle.qmv(w, s, b, x, K, N, M))
    outs = [parity.Guarded((M, N), torch.bfloat16, dev) for N in Ns]
    vpq.qmv_group_w4g64(packs, xd, K, M, outs=[o.view for o in outs])
    torch.cuda.synchronize()
    # the kernel a grouped launch shares its arithmetic with: the streaming one at M = 1, the tile one otherwise
    variant = (FLOW if M == 1 and K >= 2048 else MFMA) if K % 512 == 0 else AUTO
    for (wd, sd, bd, N), (y64, yb), out in zip(packs, refs, outs):
        got = D.bits(out.view)
        parity.check_bf16(got, y64, yb)
        out.assert_intact()
        single = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=variant))
        assert np.array_equal(got, single)


def test_qmv_grouped_row_concatenated_qkv(vpq, oracle, dev, D):
    # the reference's layout: one row-concatenated q|k|v pack, three outputs
    K, rows, M = 2048, (256, 64, 64), 1
    N = sum(rows)
    w, s, b = synth.make_weight(N, K, 31)
    x = synth.make_act(M, K, 32)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    packs, r0 = [], 0
    for r in rows:
        packs.append((wd[r0:r0 + r], sd[r0:r0 + r], bd[r0:r0 + r], r))
        r0 += r
    outs = vpq.qmv_group_w4g64(packs, xd, K, M)
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    got = np.concatenate([D.bits(o) for o in outs], axis=1)
    parity.check_bf16(got, y64, yb)


@pytest.mark.parametrize("K,M", [(64, 1), (1536, 3), (4096, 1), (5120, 40)])
def test_rmsnorm_rows(vpq, oracle, dev, D, K, M):
    """vpq_rmsnorm_bf16 (gpu-kernels/metal/quant/affine_qmv.metal:601-616): against the oracle to one bf16 step (fp32
    against float64 sums move a few elements across a rounding boundary), the same bits run to run, guard bands."""
    x = synth.make_act(M, K, 7100 + K)
    nw = synth.f32_to_bf16_bits((1.0 + 0.1 * np.random.default_rng(7200 + K).standard_normal(K)).astype(np.float32))
    want = oracle.rmsnorm(x, nw, K, M, 1e-6)
    out = parity.Guarded((M, K), torch.bfloat16, dev)
    vpq.rmsnorm_bf16(D.bf16(x, dev), D.bf16(nw, dev), K, M, 1e-6, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    got = D.bits(out.view)
    assert (got != want).mean() <= 0.02
    assert parity.bf16_ulp_distance(got, want).max() <= 1
    assert torch.equal(out.view, vpq.rmsnorm_bf16(D.bf16(x, dev), D.bf16(nw, dev), K, M, 1e-6))


@pytest.mark.parametrize("fmt", [0, 1, 2])
@pytest.mark.parametrize("K,rows", [(4096, (256, 64, 64)), (1536, (96, 32))])
def test_qmv_qkv_rms(vpq, oracle, dev, D, fmt, K, rows):
    """affine_qmv_qkv_rms_w4g64 / _w4g32 / _w8g64 (affine_qmv.metal:561-740): the normalized row lands in the scratch
    with the bits of vpq_rmsnorm_bf16, the outputs have the bits of the format's grouped GEMV over that row, and the
    whole agrees with the oracle's GEMV over the oracle's normalized row."""
    N = sum(rows)
    make = (synth.make_weight, synth.make_weight_g32, synth.make_weight8)[fmt]
    w, s, b = make(N, K, 7300 + K + fmt)
    x = synth.make_act(1, K, 7400 + K)
    nw = synth.f32_to_bf16_bits((1.0 + 0.1 * np.random.default_rng(7500 + K).standard_normal(K)).astype(np.float32))
    wd, sd, bd, xd, nwd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev), D.bf16(nw, dev)
    packs, r0 = [], 0
    for n in rows:
        packs.append((wd[r0:r0 + n], sd[r0:r0 + n], bd[r0:r0 + n], n))
        r0 += n
    ws = parity.Guarded((1, K), torch.bfloat16, dev)
    outs = [parity.Guarded((1, n), torch.bfloat16, dev) for n in rows]
    vpq.qmv_qkv_rms(fmt, packs, xd, nwd, K, 1e-6, outs=[o.view for o in outs], x_norm_ws=ws.view)
    torch.cuda.synchronize()
    ws.assert_intact()
    xn = vpq.rmsnorm_bf16(xd, nwd, K, 1, 1e-6)
    assert torch.equal(ws.view, xn)
    group = (vpq.qmv_group_w4g64, vpq.qmv_group_w4g32, vpq.qmv_group_w8g64)[fmt]
    for o, ref in zip(outs, group(packs, xn, K, 1)):
        o.assert_intact()
        assert torch.equal(o.view, ref)
    xo = oracle.rmsnorm(x, nw, K, 1, 1e-6)
    y64 = (oracle.qmv(w, s, b, xo, K, N, 1)[0], oracle.qmv_g32(w, s, b, xo, K, N, 1)[0],
           oracle.matmul8(w, s, b, xo, K, N, 1, rounded=False)[0])[fmt]
    got = synth.bf16_bits_to_f32(np.concatenate([D.bits(o.view) for o in outs], axis=1)).astype(np.float64)
    assert parity.rel_l2(got, y64) <= 4e-3
    L = vpq.load()
    p = ws.view.data_ptr()
    assert L.vpq_qmv_qkv_rms_bf16(None, 3, 1, None, None, None, p, p, None, K, None, 1e-6, p) == -2
    assert L.vpq_qmv_qkv_rms_bf16(None, 0, 1, None, None, None, p, p, None, K, None, 1e-6, None) == -4
