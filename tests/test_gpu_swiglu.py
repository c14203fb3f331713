"""GPU parity of the fused gate|up projection + SwiGLU (QMV and QMM arithmetic) and of the
load-time row interleave, against the CPU oracle, through the C ABI.  The agreement test of
the reference (tests/unit-tests/minimax-h3-blocks.cc:807-846: fused store against GEMM + a
separate activation pass, rel-L2 < 3e-2) is carried over with its tolerance."""
import numpy as np
import pytest
import torch

from tests import parity
from vpipe_amd import capi, synth

pytestmark = pytest.mark.gpu

SIMPLE, MFMA, SPLITK, RING, AUTO = (capi.VPQ_QMV_SIMPLE, capi.VPQ_QMV_MFMA, capi.VPQ_QMV_RING_SPLITK,
                                    capi.VPQ_QMV_RING, capi.VPQ_QMV_AUTO)


def fused_pack(oracle, F, K, seed):
    """Two independent packs [F,K] (gate, up) and their interleaved pack [2F,K]."""
    gate = synth.make_weight(F, K, seed)
    up = synth.make_weight(F, K, seed + 1)
    return gate, up, tuple(oracle.interleave(a, b) for a, b in zip(gate, up))


def stage(D, dev, pack, x):
    w, s, b = pack
    return D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)


@pytest.mark.parametrize("K,F", [(64, 5), (128, 33), (512, 16), (4096, 96)])
def test_interleave_rows_on_the_device(vpq, oracle, dev, D, K, F):
    gate, up, want = fused_pack(oracle, F, K, 300 + K)
    g = (D.u32(gate[0], dev), D.bf16(gate[1], dev), D.bf16(gate[2], dev))
    u = (D.u32(up[0], dev), D.bf16(up[1], dev), D.bf16(up[2], dev))
    w, s, b = vpq.interleave_gate_up(g, u)
    torch.cuda.synchronize()
    assert np.array_equal(D.words(w), want[0])
    assert np.array_equal(D.bits(s), want[1])
    assert np.array_equal(D.bits(b), want[2])


QMV_SHAPES = [
    # K, F (features; the pack has 2F rows), M
    (512, 8, 1), (512, 17, 4), (1024, 24, 2), (1024, 20, 3), (2048, 80, 5), (1536, 33, 7),
    (4096, 47, 8), (2560, 32, 16), (4096, 8, 13), (8192, 264, 1),
]


@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
@pytest.mark.parametrize("K,F,M", [(64, 5, 1), (1984, 17, 2), (2048, 24, 1), (3840, 33, 2), (5120, 80, 1)])
def test_qmv_gated_row_streaming_kernel(vpq, oracle, dev, D, K, F, M, activation):
    # the row-streaming kernel's register-local (gate, up) pairs; K not a multiple of 512 is also what
    # the automatic choice sends there
    _, _, pack = fused_pack(oracle, F, K, 520 + K + F)
    x = synth.make_act(M, K, 620 + K + M)
    y64, _ = oracle.qmv(*pack, x, K, 2 * F, M)
    o64, ob = (oracle.swiglu if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu)(y64)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    f = vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, variant=capi.VPQ_QMV_ROWS, f32out=True, activation=activation)
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, out=out.view, variant=capi.VPQ_QMV_ROWS, activation=activation)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), o64)
    parity.check_bf16(D.bits(out.view), o64, ob, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)
    out.assert_intact()
    if K % 512 != 0:
        auto = vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, variant=AUTO, activation=activation)
        assert torch.equal(auto, out.view)


@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
@pytest.mark.parametrize("K,F", [(2048, 3), (4096, 101), (12288, 37), (17408, 9)])
def test_qmv_gated_flow_kernel(vpq, oracle, dev, D, K, F, activation):
    # the streaming M = 1 kernel's register-local gated store (a gate/up pair of rows is one wavefront's)
    _, _, pack = fused_pack(oracle, F, K, 520 + K + F)
    x = synth.make_act(1, K, 620 + K)
    y64, _ = oracle.qmv(*pack, x, K, 2 * F, 1)
    o64, ob = oracle.swiglu(y64) if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu(y64)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    f = vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, 1, variant=capi.VPQ_QMV_FLOW, f32out=True, activation=activation)
    out = parity.Guarded((1, F), torch.bfloat16, dev)
    vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, 1, out=out.view, variant=capi.VPQ_QMV_FLOW, activation=activation)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), o64)
    parity.check_bf16(D.bits(out.view), o64, ob, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)
    out.assert_intact()


@pytest.mark.parametrize("variant", [SIMPLE, MFMA, RING, AUTO])
@pytest.mark.parametrize("K,F,M", QMV_SHAPES)
def test_qmv_swiglu(vpq, oracle, dev, D, K, F, M, variant):
    _, _, pack = fused_pack(oracle, F, K, 500 + K + F)
    x = synth.make_act(M, K, 600 + K + M)
    N = 2 * F
    y64, _ = oracle.qmv(*pack, x, K, N, M)
    o64, ob = oracle.swiglu(y64)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    f = vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, N, M, variant=variant, f32out=True)
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, N, M, out=out.view, variant=variant)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), o64)
    parity.check_bf16(D.bits(out.view), o64, ob)
    out.assert_intact()


def test_qmv_swiglu_general_k_and_the_workspace_free_contract(vpq, oracle, dev, D):
    # K not a multiple of 512 goes to the general kernel; the entry point carries no workspace,
    # so the split-K variant is refused instead of running without one
    K, F, M = 192, 10, 3
    _, _, pack = fused_pack(oracle, F, K, 77)
    x = synth.make_act(M, K, 78)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    got = vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, f32out=True)
    o64, _ = oracle.swiglu(oracle.qmv(*pack, x, K, 2 * F, M)[0])
    parity.check_f32(got.cpu().numpy(), o64)
    for variant in (MFMA, SPLITK, RING):
        with pytest.raises(capi.VpqError):
            vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, variant=variant)


def test_qmv_swiglu_equals_two_projections_and_an_activation(vpq, oracle, dev, D):
    # the fused launch computes what gate and up as separate QMVs + silu(gate)*up compute
    K, F, M = 4096, 96, 1
    gate, up, pack = fused_pack(oracle, F, K, 900)
    x = synth.make_act(M, K, 901)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    fused = vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, variant=MFMA, f32out=True)
    gw, gs, gb, _ = stage(D, dev, gate, x)
    uw, us, ub, _ = stage(D, dev, up, x)
    g = vpq.qmv_w4g64(gw, gs, gb, xd, K, F, M, variant=MFMA, f32out=True)
    u = vpq.qmv_w4g64(uw, us, ub, xd, K, F, M, variant=MFMA, f32out=True)
    torch.cuda.synchronize()
    want = (g.double() / (1.0 + torch.exp(-g.double())) * u.double()).cpu().numpy()
    assert parity.floor_rel_err(fused.cpu().numpy(), want) <= 1e-5


def test_qmv_swiglu_llama_mlp_shape_full(vpq, oracle, dev, D):
    # the decode call site (generative-models/llama3/metal-llama-model.cc:466-477): hidden 4096,
    # ffn 12288, one row; every output checked
    K, F, M = 4096, 12288, 1
    _, _, pack = fused_pack(oracle, F, K, 1200)
    x = synth.make_act(M, K, 1201)
    o64, ob = oracle.swiglu(oracle.qmv(*pack, x, K, 2 * F, M)[0])
    wd, sd, bd, xd = stage(D, dev, pack, x)
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.linear_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, out=out.view)
    torch.cuda.synchronize()
    parity.check_bf16(D.bits(out.view), o64, ob)
    out.assert_intact()


QMM_SHAPES = [
    # M, F, K: one tile, ragged M, ragged N (2F % 128 != 0, 2F % 4 == 2), several tiles, deep K
    (64, 64, 64), (17, 32, 256), (130, 160, 256), (33, 17, 128), (257, 65, 512), (300, 192, 2048), (40, 1, 64),
]


@pytest.mark.parametrize("M,F,K", QMM_SHAPES)
def test_qmm_swiglu(vpq, oracle, dev, D, M, F, K):
    _, _, pack = fused_pack(oracle, F, K, 1500 + M + F)
    x = synth.make_act(M, K, 1600 + M + K)
    N = 2 * F
    o64, ob = oracle.swiglu(oracle.qmm(*pack, x, K, N, M)[0])
    wd, sd, bd, xd = stage(D, dev, pack, x)
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.qmm_swiglu_w4g64(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    parity.check_bf16(D.bits(out.view), o64, ob)
    out.assert_intact()


@pytest.mark.parametrize("stride,off", [(200, 40), (201, 7), (96, 0)])
def test_qmm_swiglu_strided_output(vpq, oracle, dev, D, stride, off):
    # qmm_t_swiglu_rs_impl (gpu-kernels/metal/quant/affine_qmm_steel.metal:663-768): the result
    # lands in a column window of a wider row; everything outside the window is untouched
    M, F, K = 70, 96, 256
    _, _, pack = fused_pack(oracle, F, K, 1700)
    x = synth.make_act(M, K, 1701)
    o64, ob = oracle.swiglu(oracle.qmm(*pack, x, K, 2 * F, M)[0])
    wd, sd, bd, xd = stage(D, dev, pack, x)
    plain = vpq.qmm_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M)
    wide = torch.full((M, stride), 7.0, dtype=torch.bfloat16, device=dev)
    vpq.qmm_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, out=wide, out_stride=stride, out_off=off)
    torch.cuda.synchronize()
    assert torch.equal(wide[:, off:off + F], plain)
    keep = torch.ones(stride, dtype=torch.bool, device=dev)
    keep[off:off + F] = False
    assert (wide[:, keep] == 7.0).all().item()
    parity.check_bf16(D.bits(plain), o64, ob)


def test_qmm_swiglu_matches_gemm_then_activation(vpq, oracle, dev, D):
    # the reference's agreement arm (tests/unit-tests/minimax-h3-blocks.cc:807-846), M = 64:
    # unfused = QMM into [M, 2F] bf16 (gate block | up block layout), then the activation
    # reading those rounded values; fused = interleaved pack, register-local store.
    # rel-L2 < 3e-2 asserted there (the arms differ by one rounding); a gate/up mix-up scores O(1).
    M, F, K = 64, 1024, 1024
    gate, up, pack = fused_pack(oracle, F, K, 1800)
    x = synth.make_act(M, K, 1801)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    fused = vpq.qmm_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M).float()
    block = tuple(np.concatenate([a, b], axis=0) for a, b in zip(gate, up))
    bw, bs, bb, _ = stage(D, dev, block, x)
    wide = vpq.qmm_w4g64(bw, bs, bb, xd, K, 2 * F, M).float()
    g, u = wide[:, :F], wide[:, F:]
    ref = (g / (1.0 + torch.exp(-g)) * u).bfloat16().float()
    torch.cuda.synchronize()
    rl2 = (torch.linalg.norm(fused - ref) / torch.linalg.norm(ref)).item()
    assert rl2 < 3e-2
    assert rl2 < 5e-3      # what one extra bf16 rounding of gate and up explains


def test_qmm_swiglu_prefill_shape_sampled(vpq, oracle, dev, D):
    # prefill call site (generative-models/llama3/metal-llama-model.cc:800): M = 2048 rows over the
    # interleaved 4096 -> 2 x 12288 pack; the oracle checks a sample of rows against a sample of features
    M, F, K = 2048, 12288, 4096
    _, _, pack = fused_pack(oracle, F, K, 1900)
    x = synth.make_act(M, K, 1901)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.linear_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    rng = np.random.default_rng(3)
    rows = np.sort(rng.choice(M, 24, replace=False))
    feats = np.sort(rng.choice(F, 96, replace=False))
    sel = np.stack([2 * feats, 2 * feats + 1], 1).ravel()
    w, s, b = pack
    o64, ob = oracle.swiglu(oracle.qmm(w[sel], s[sel], b[sel], x[rows], K, len(sel), len(rows))[0])
    got = D.bits(out.view[torch.from_numpy(rows).to(dev)][:, torch.from_numpy(feats).to(dev)])
    parity.check_bf16(got, o64, ob)


# 1 + tanh(z) cancels for gates below about -3: evaluated in fp32, as the reference writes it, the
# product there is noise around a value of order 1e-6 of the rms (the float64 oracle gives the true
# tiny value), so which side of a bf16 boundary it lands on is arbitrary.  Those outputs are bounded by
# the absolute-error check; the mismatch rate is taken over the outputs that are not tiny.


@pytest.mark.parametrize("variant", [SIMPLE, MFMA, RING, AUTO])
@pytest.mark.parametrize("K,F,M", [(512, 17, 4), (2048, 80, 5), (4096, 47, 8), (2560, 32, 16), (8192, 264, 1)])
def test_qmv_geglu(vpq, oracle, dev, D, K, F, M, variant):
    # affine_qmv_geglu_w4g64 (gpu-kernels/metal/quant/affine_qmv.metal:1352-1447): the same fused pack,
    # gelu_tanh(gate) * up
    _, _, pack = fused_pack(oracle, F, K, 2500 + K + F)
    x = synth.make_act(M, K, 2600 + K + M)
    o64, ob = oracle.geglu(oracle.qmv(*pack, x, K, 2 * F, M)[0])
    wd, sd, bd, xd = stage(D, dev, pack, x)
    f = vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, variant=variant, f32out=True, activation=capi.VPQ_GATE_GEGLU)
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.qmv_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, out=out.view, variant=variant, activation=capi.VPQ_GATE_GEGLU)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), o64)
    parity.check_bf16(D.bits(out.view), o64, ob, mismatch_over_all=False)
    out.assert_intact()


@pytest.mark.parametrize("M,F,K", [(64, 64, 64), (130, 160, 256), (257, 65, 512), (300, 192, 2048), (9, 48, 1024)])
def test_qmm_and_linear_geglu(vpq, oracle, dev, D, M, F, K):
    _, _, pack = fused_pack(oracle, F, K, 2700 + M + F)
    x = synth.make_act(M, K, 2800 + M + K)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    o64, ob = oracle.geglu(oracle.qmm(*pack, x, K, 2 * F, M)[0])
    out = parity.Guarded((M, F), torch.bfloat16, dev)
    vpq.qmm_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, out=out.view, activation=capi.VPQ_GATE_GEGLU)
    torch.cuda.synchronize()
    parity.check_bf16(D.bits(out.view), o64, ob, mismatch_over_all=False)
    out.assert_intact()
    # the size-based entrance takes the GEMV arithmetic (in slabs of 16 rows) up to 64 rows
    arith = oracle.qmv if M <= 64 else oracle.qmm
    l64, lb = oracle.geglu(arith(*pack, x, K, 2 * F, M)[0])
    got = vpq.linear_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, activation=capi.VPQ_GATE_GEGLU)
    parity.check_bf16(D.bits(got), l64, lb, mismatch_over_all=False)
    with pytest.raises(capi.VpqError):
        vpq.qmm_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, activation=3)



# shapes whose tiles fill the CUs, so that the gated store of the large-tile GEMM kernel runs, at each of its
# tile widths (the library picks 128, 256, 192 for these), ragged M, strided and offset output windows
@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
@pytest.mark.parametrize("M,F,K,stride,off", [(4100, 2048, 512, 0, 0), (4100, 3072, 512, 3200, 64), (2048, 6144, 512, 6145, 1)])
def test_qmm_gated_store_of_the_large_tile_kernel(vpq, oracle, dev, D, M, F, K, stride, off, activation):
    _, _, pack = fused_pack(oracle, F, K, 2100 + F)
    x = synth.make_act(M, K, 2101 + M)
    wd, sd, bd, xd = stage(D, dev, pack, x)
    width = stride if stride > 0 else F
    out = parity.Guarded((M, width), torch.bfloat16, dev)
    out.view.fill_(7.0)
    vpq.qmm_swiglu_w4g64(wd, sd, bd, xd, K, 2 * F, M, out=out.view, out_stride=stride, out_off=off, activation=activation)
    torch.cuda.synchronize()
    out.assert_intact()
    got_all = out.view
    if stride > 0:      # nothing outside the window was touched
        assert bool((got_all[:, :off] == 7.0).all()) and bool((got_all[:, off + F:] == 7.0).all())
    rng = np.random.default_rng(F + M)
    rows = np.unique(np.concatenate([[0, M - 1, 255, 256, 2047 % M], rng.choice(M, 16, replace=False)]))
    feats = np.unique(np.concatenate([[0, F - 1, 63, 64, 95, 96, 127, 128], rng.choice(F, 64, replace=False)]))
    sel = np.stack([2 * feats, 2 * feats + 1], 1).ravel()
    w, s, b = pack
    y64 = oracle.qmm(w[sel], s[sel], b[sel], x[rows], K, len(sel), len(rows))[0]
    o64, ob = (oracle.swiglu if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu)(y64)
    got = D.bits(got_all[torch.from_numpy(rows).to(dev)][:, torch.from_numpy(off + feats).to(dev)])
    parity.check_bf16(got, o64, ob, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)


@pytest.mark.parametrize("K,N", [(4096, 300), (2048, 64), (12288, 512), (192, 10), (1024, 33)])
def test_qmv_gelu_mul(vpq, oracle, dev, D, K, N):
    """affine_qmv_gelu_mul_w4g64 (gpu-kernels/metal/quant/affine_qmv.metal:751-768, store :268-279): the GEMV's
    bf16-rounded result goes through gelu_tanh and is multiplied by mul[n].  The store is checked on the device's own
    GEMV output (whose parity other tests hold), so what is compared is the fused store against the oracle's
    gelu_tanh(v) * mul; and the whole against the oracle's GEMV by rel-L2."""
    w, s, b = synth.make_weight(N, K, 3100 + K + N)
    x = synth.make_act(1, K, 3200 + K)
    mul = synth.make_act(1, N, 3300 + N)
    wd, sd, bd, xd = stage(D, dev, (w, s, b), x)
    v_bits = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, 1))
    pairs = np.stack([synth.bf16_bits_to_f32(v_bits[0]).astype(np.float64),
                      synth.bf16_bits_to_f32(mul[0]).astype(np.float64)], axis=1).reshape(1, 2 * N)
    o64, ob = oracle.geglu(pairs)
    out = parity.Guarded((1, N), torch.bfloat16, dev)
    vpq.qmv_gelu_mul_w4g64(wd, sd, bd, xd, K, N, D.bf16(mul, dev), out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    got = D.bits(out.view)
    # (1 + tanh cancels in fp32 for strongly negative v, as in the reference: the tolerance of the GEGLU stores)
    parity.check_bf16(got, o64, ob, mismatch_over_all=False)
    # end to end against the oracle's GEMV (a 1-ulp difference in v moves the output by about as much)
    _, yb = oracle.qmv(w, s, b, x, K, N, 1)
    p2 = np.stack([synth.bf16_bits_to_f32(yb[0]).astype(np.float64),
                   synth.bf16_bits_to_f32(mul[0]).astype(np.float64)], axis=1).reshape(1, 2 * N)
    e64, _ = oracle.geglu(p2)
    assert parity.rel_l2(synth.bf16_bits_to_f32(got).astype(np.float64), e64) <= 4e-3
    L = vpq.load()
    p = out.view.data_ptr()
    assert L.vpq_qmv_gelu_mul_w4g64_bf16(None, p, p, p, p, p, K, N, None) == -1
    assert L.vpq_qmv_gelu_mul_w4g64_bf16(None, p, p, p, p, p, K + 8, N, p) == -2
