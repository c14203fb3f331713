"""GPU parity of the 4-bit group-32 twins (GGUF Q4_0 repacked to affine): dense expansion bit-exact,
QMV with and without the scale-only shortcut, the gated stores, the dequant-once GEMM route --
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from tests import parity
from vpipe_amd import capi, synth

pytestmark = pytest.mark.gpu


def stage(D, dev, w, s, b, x=None):
    out = [D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev)]
    if x is not None:
        out.append(D.bf16(x, dev))
    return out


@pytest.mark.parametrize("N,K", [(1, 32), (33, 96), (257, 3840), (2048, 4096)])
def test_dequant_g32_bit_exact(vpq, oracle, dev, D, N, K):
    w, s, b = synth.make_weight_g32(N, K, 21 + N)
    wd, sd, bd = stage(D, dev, w, s, b)
    out = parity.Guarded((N, K), torch.bfloat16, dev)
    vpq.dequant_w4g32(wd, sd, bd, K, N, out=out.view)
    torch.cuda.synchronize()
    assert np.array_equal(D.bits(out.view), oracle.dequant_g32_bf16(w, s, b, K, N))
    out.assert_intact()


# both kernels (up to two rows of x: row-streaming; more: one wavefront per row), K below / at / above a
# 2048-wide pass and not a multiple of 64, ragged N
QMV_SHAPES = [(32, 5, 1), (96, 33, 2), (1024, 48, 3), (2080, 130, 1), (3872, 64, 2), (4096, 95, 8), (2560, 64, 16),
              (5120, 4096, 1)]


@pytest.mark.parametrize("K,N,M", QMV_SHAPES)
def test_qmv_g32(vpq, oracle, dev, D, K, N, M):
    w, s, b = synth.make_weight_g32(N, K, 6000 + K + N)
    x = synth.make_act(M, K, 6100 + K + M)
    y64, yb = oracle.qmv_g32(w, s, b, x, K, N, M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    f = vpq.qmv_w4g32(wd, sd, bd, xd, K, N, M, f32out=True)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w4g32(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), y64)
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()
    res = synth.make_act(M, N, 6200 + N)
    got = D.bits(vpq.qmv_w4g32(wd, sd, bd, xd, K, N, M, residual=D.bf16(res, dev)))
    want = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(D.bits(out.view)) + synth.bf16_bits_to_f32(res))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("K,N,M", [(96, 33, 2), (2080, 130, 1), (4096, 95, 8), (5120, 1024, 1)])
def test_qmv_g32_scale_only_is_the_affine_form_on_a_q40_pack(vpq, oracle, dev, D, K, N, M):
    # affine_qmv.metal:322-326: "bit-identical output" with the bias buffer never read
    w, s, b = synth.make_weight_g32(N, K, 6300 + K + N, q40=True)
    x = synth.make_act(M, K, 6400 + K + M)
    y64, yb = oracle.qmv_g32(w, s, None, x, K, N, M, scale_only=True)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    affine = vpq.qmv_w4g32(wd, sd, bd, xd, K, N, M)
    only = vpq.qmv_w4g32(wd, sd, None, xd, K, N, M, scale_only=True)
    assert torch.equal(affine, only)
    parity.check_bf16(D.bits(only), y64, yb)
    parity.check_f32(vpq.qmv_w4g32(wd, sd, None, xd, K, N, M, f32out=True, scale_only=True).cpu().numpy(), y64)


@pytest.mark.parametrize("scale_only", [False, True])
@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
@pytest.mark.parametrize("K,F,M", [(96, 17, 1), (2048, 64, 2), (2592, 40, 5), (4096, 128, 16)])
def test_qmv_g32_gated(vpq, oracle, dev, D, K, F, M, activation, scale_only):
    N = 2 * F
    w, s, b = synth.make_weight_g32(N, K, 6500 + K + F, q40=scale_only)
    x = synth.make_act(M, K, 6600 + K + M)
    y64, _ = oracle.qmv_g32(w, s, b, x, K, N, M, scale_only=scale_only)
    o64, ob = (oracle.swiglu if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu)(y64)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.qmv_w4g32(wd, sd, None if scale_only else bd, xd, K, N, M, out=out.view, activation=activation, scale_only=scale_only)
    torch.cuda.synchronize()
    parity.check_bf16(D.bits(out.view), o64, ob, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)
    out.assert_intact()


@pytest.mark.parametrize("M,N,K", [(64, 64, 32), (130, 320, 288), (257, 129, 512)])
def test_qmm_g32_dense_route(vpq, oracle, dev, D, M, N, K):
    w, s, b = synth.make_weight_g32(N, K, 6700 + N)
    x = synth.make_act(M, K, 6800 + M)
    dense = oracle.dequant_g32_bf16(w, s, b, K, N)
    y64 = synth.bf16_bits_to_f32(x).astype(np.float64) @ synth.bf16_bits_to_f32(dense).astype(np.float64).T
    yb = synth.f32_to_bf16_bits(y64.astype(np.float32))
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    wdeq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    y = vpq.qmm_dense_route_w4g32(wd, sd, bd, xd, K, N, M, wdeq)
    torch.cuda.synchronize()
    assert np.array_equal(D.bits(wdeq), dense)
    parity.check_bf16(D.bits(y), y64, yb)
    assert torch.equal(y, vpq.qmm_dense_route_w4g32(wd, sd, bd, xd, K, N, M, wdeq, expand=False))


def test_g32_rejects_bad_arguments(vpq, dev):
    L = vpq.load()
    t = torch.zeros(4096, dtype=torch.int32, device=dev)
    p = t.data_ptr()
    assert L.vpq_qmv_w4g32_bf16(None, p, p, None, p, p, 32, 8, 1, None, 0) == -1      # affine form needs the biases
    assert L.vpq_qmv_w4g32_bf16(None, p, p, None, p, p, 32, 8, 1, None, 1) == 0
    assert L.vpq_qmv_w4g32_bf16(None, p, p, p, p, p, 48, 8, 1, None, 0) == -2         # K % 32
    assert L.vpq_qmv_w4g32_bf16(None, p, p, p, p, p, 32, 8, 17, None, 0) == -2
    assert L.vpq_qmv_gated_w4g32_bf16(None, p, p, p, p, p, 32, 7, 1, capi.VPQ_GATE_SWIGLU, 0) == -2
    assert L.vpq_dequant_w4g32_bf16(None, p, p, p, None, 32, 8) == -1
    torch.cuda.synchronize()


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (300, 200, 128), (257, 129, 512), (520, 260, 1536)])
def test_qmm_g32_fused_tile_kernel(vpq, oracle, dev, D, M, N, K):
    # the fused kernel with a scale and a bias per 32 values: the GEMM on the oracle's bit-exact expansion
    w, s, b = synth.make_weight_g32(N, K, 6900 + N)
    x = synth.make_act(M, K, 6901 + M)
    dense = oracle.dequant_g32_bf16(w, s, b, K, N)
    y64 = synth.bf16_bits_to_f32(x).astype(np.float64) @ synth.bf16_bits_to_f32(dense).astype(np.float64).T
    yb = synth.f32_to_bf16_bits(y64.astype(np.float32))
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_w4g32(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_bf16(D.bits(out.view), y64, yb)
    # a group-64 pack with every scale and bias written twice is the same matrix: the group-64 kernel's bits
    w64, s64, b64 = synth.make_weight(N, K, 6902 + N)
    s2, b2 = np.repeat(s64, 2, axis=1), np.repeat(b64, 2, axis=1)
    got32 = vpq.qmm_w4g32(D.u32(w64, dev), D.bf16(s2, dev), D.bf16(b2, dev), xd, K, N, M)
    got64 = vpq.qmm_w4g64(D.u32(w64, dev), D.bf16(s64, dev), D.bf16(b64, dev), xd, K, N, M, tile_n=128)
    assert torch.equal(got32, got64)


@pytest.mark.parametrize("tile_n", [256, -128])
@pytest.mark.parametrize("M,N,K", [(64, 64, 512), (300, 200, 1024), (257, 136, 512), (520, 392, 1536)])
def test_qmm_g32_large_tile_kernel(vpq, oracle, dev, D, M, N, K, tile_n):
    """Groups of 32 through the large-tile kernel at its two tile widths for this format (256, 128): the GEMM on the oracle's bit-exact
    expansion, the bits of the 256 x 128 tile kernel, the gated stores, and on a group-64 pack with doubled scales
    the bits of the group-64 large-tile kernel."""
    w, s, b = synth.make_weight_g32(N, K, 7100 + N)
    x = synth.make_act(M, K, 7101 + M)
    dense = oracle.dequant_g32_bf16(w, s, b, K, N)
    y64 = synth.bf16_bits_to_f32(x).astype(np.float64) @ synth.bf16_bits_to_f32(dense).astype(np.float64).T
    yb = synth.f32_to_bf16_bits(y64.astype(np.float32))
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_w4g32(wd, sd, bd, xd, K, N, M, out=out.view, tile_n=tile_n)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_bf16(D.bits(out.view), y64, yb)
    assert torch.equal(out.view, vpq.qmm_w4g32(wd, sd, bd, xd, K, N, M, tile_n=128))
    for activation, fn in ((capi.VPQ_GATE_SWIGLU, oracle.swiglu), (capi.VPQ_GATE_GEGLU, oracle.geglu)):
        want64, wantb = fn(y64)
        og = parity.Guarded((M, N // 2), torch.bfloat16, dev)
        vpq.qmm_w4g32(wd, sd, bd, xd, K, N, M, out=og.view, activation=activation, tile_n=tile_n)
        torch.cuda.synchronize()
        og.assert_intact()
        parity.check_bf16(D.bits(og.view), want64, wantb, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)
    w64, s64, b64 = synth.make_weight(N, K, 7102 + N)
    s2, b2 = np.repeat(s64, 2, axis=1), np.repeat(b64, 2, axis=1)
    got32 = vpq.qmm_w4g32(D.u32(w64, dev), D.bf16(s2, dev), D.bf16(b2, dev), xd, K, N, M, tile_n=tile_n)
    got64 = vpq.qmm_w4g64(D.u32(w64, dev), D.bf16(s64, dev), D.bf16(b64, dev), xd, K, N, M, tile_n=tile_n)
    assert torch.equal(got32, got64)


@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
def test_qmm_g32_gated_store(vpq, oracle, dev, D, activation):
    K, F, M = 512, 70, 130
    w, s, b = synth.make_weight_g32(2 * F, K, 6950)
    x = synth.make_act(M, K, 6951)
    dense = oracle.dequant_g32_bf16(w, s, b, K, 2 * F)
    y64 = synth.bf16_bits_to_f32(x).astype(np.float64) @ synth.bf16_bits_to_f32(dense).astype(np.float64).T
    want64, wantb = (oracle.swiglu if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu)(y64)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    got = vpq.qmm_w4g32(wd, sd, bd, xd, K, 2 * F, M, activation=activation)
    parity.check_bf16(D.bits(got), want64, wantb, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)
    assert vpq.load().vpq_qmm_w4g32_bf16(None, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), xd.data_ptr(), got.data_ptr(),
                                         96, 8, 4) == -2            # K % 64


@pytest.mark.parametrize("K,M,rows", [(4096, 1, (256, 64, 64)), (96, 2, (33, 7)), (2560, 5, (48, 16, 16)), (1024, 1, (40,))])
def test_qmv_group_g32_is_the_separate_calls(vpq, dev, D, K, M, rows):
    """affine_qmv_qkv_w4g32 (gpu-kernels/metal/quant/affine_qmv.metal:518-538): the row-concatenated q|k|v pack as one
    call; every output has the bits of its own vpq_qmv_w4g32_bf16 call (whose parity test_qmv_g32 holds), guard bands
    intact.  M <= 2 is one launch of the row-streaming kernel, more rows are separate launches."""
    N = sum(rows)
    w, s, b = synth.make_weight_g32(N, K, 6800 + K + N)
    x = synth.make_act(M, K, 6900 + K + M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    packs, r0 = [], 0
    for n in rows:
        packs.append((wd[r0:r0 + n], sd[r0:r0 + n], bd[r0:r0 + n], n))
        r0 += n
    outs = [parity.Guarded((M, n), torch.bfloat16, dev) for n in rows]
    vpq.qmv_group_w4g32(packs, xd, K, M, outs=[o.view for o in outs])
    torch.cuda.synchronize()
    for o, p in zip(outs, packs):
        o.assert_intact()
        assert torch.equal(o.view, vpq.qmv_w4g32(p[0], p[1], p[2], xd, K, p[3], M))
    L = vpq.load()
    assert L.vpq_qmv_group_w4g32_bf16(None, 5, None, None, None, None, None, K, None, M, 0) == -1
