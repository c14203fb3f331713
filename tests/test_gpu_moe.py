"""GPU parity of the gathered expert projections of an MoE block (one launch for all the
(token, expert) pairs), through the C ABI: each pair against the CPU oracle's QMV on that
expert's slab, and bit-identical to the plain kernel on the same slab -- the reference's own
contract for its gather kernels (gpu-kernels/metal/quant/affine_qmv.metal:918-921: "a gathered
expert is token-EXACT with the same expert run through the plain kernels")."""
import numpy as np
import pytest
import torch

from tests import parity
from vpipe_amd import capi, synth

pytestmark = pytest.mark.gpu


def expert_batch(E, N, K, seed):
    """E independent packs stacked into [E, N, ...] arrays."""
    packs = [synth.make_weight(N, K, seed + 13 * e) for e in range(E)]
    return tuple(np.stack([p[i] for p in packs]) for i in range(3))


def ids_for(E, npair, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, E, size=npair, dtype=np.int32)


# K, inner, E, top_k, M: one-pass and multi-pass K, K <= 1024 (two row groups per wavefront), K not a
# multiple of 512, odd inner, several tokens
GATED_SHAPES = [(2048, 96, 8, 4, 1), (2048, 768, 16, 8, 1), (4096, 33, 5, 2, 3), (768, 64, 4, 3, 2), (1984, 40, 3, 2, 2),
                (5120, 24, 6, 1, 4)]


@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
@pytest.mark.parametrize("K,inner,E,top_k,M", GATED_SHAPES)
def test_gathered_gate_up(vpq, oracle, dev, D, K, inner, E, top_k, M, activation):
    N = 2 * inner
    w, s, b = expert_batch(E, N, K, 4000 + K + inner)
    x = synth.make_act(M, K, 4100 + K + M)
    npair = M * top_k
    eid = ids_for(E, npair, 4200 + K)
    wd, sd, bd, xd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)
    eidd = torch.from_numpy(eid).to(dev)
    out = parity.Guarded((npair, inner), torch.bfloat16, dev)
    vpq.gather_qmv_gated_w4g64(wd, sd, bd, xd, K, N, eidd, top_k, E, out=out.view, activation=activation)
    torch.cuda.synchronize()
    out.assert_intact()
    got = D.bits(out.view)
    act = oracle.swiglu if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu
    want64 = np.empty((npair, inner))
    wantb = np.empty((npair, inner), dtype=np.uint16)
    for p in range(npair):
        e, t = int(eid[p]), p // top_k
        y64, _ = oracle.qmv(w[e], s[e], b[e], x[t:t + 1], K, N, 1)
        want64[p], wantb[p] = (a[0] for a in act(y64))
        plain = vpq.qmv_swiglu_w4g64(wd[e], sd[e], bd[e], xd[t:t + 1], K, N, 1, variant=capi.VPQ_QMV_ROWS,
                                     activation=activation)
        assert np.array_equal(got[p], D.bits(plain)[0]), "pair %d differs from the plain kernel on expert %d" % (p, e)
    parity.check_bf16(got, want64, wantb, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)


# K (= inner), N (= hidden), E, npair
DOWN_SHAPES = [(768, 2048, 16, 8), (96 * 64 // 8, 256, 4, 5), (1024, 130, 3, 7), (2048, 64, 5, 1), (4608, 48, 2, 3)]


@pytest.mark.parametrize("K,N,E,npair", DOWN_SHAPES)
def test_gathered_down(vpq, oracle, dev, D, K, N, E, npair):
    w, s, b = expert_batch(E, N, K, 4300 + K + N)
    x = synth.make_act(npair, K, 4400 + K + npair)
    eid = ids_for(E, npair, 4500 + K)
    wd, sd, bd, xd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)
    out = parity.Guarded((npair, N), torch.bfloat16, dev)
    vpq.gather_down_qmv_w4g64(wd, sd, bd, xd, K, N, torch.from_numpy(eid).to(dev), E, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    got = D.bits(out.view)
    want64 = np.empty((npair, N))
    wantb = np.empty((npair, N), dtype=np.uint16)
    for p in range(npair):
        e = int(eid[p])
        y64, yb = oracle.qmv(w[e], s[e], b[e], x[p:p + 1], K, N, 1)
        want64[p], wantb[p] = y64[0], yb[0]
        plain = vpq.qmv_w4g64(wd[e], sd[e], bd[e], xd[p:p + 1], K, N, 1, variant=capi.VPQ_QMV_ROWS)
        assert np.array_equal(got[p], D.bits(plain)[0]), "pair %d differs from the plain kernel on expert %d" % (p, e)
    parity.check_bf16(got, want64, wantb)


def test_gather_expert_id_out_of_range_gives_zeros(vpq, oracle, dev, D):
    K, inner, E, top_k = 1024, 32, 3, 2
    w, s, b = expert_batch(E, 2 * inner, K, 4600)
    x = synth.make_act(2, K, 4601)
    eid = np.array([1, -1, E, 2], dtype=np.int32)
    wd, sd, bd, xd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)
    got = D.bits(vpq.gather_qmv_gated_w4g64(wd, sd, bd, xd, K, 2 * inner, torch.from_numpy(eid).to(dev), top_k, E))
    assert not got[1].any() and not got[2].any()
    assert got[0].any() and got[3].any()
    down = D.bits(vpq.gather_down_qmv_w4g64(wd, sd, bd, D.bf16(synth.make_act(4, K, 4602), dev), K, 2 * inner,
                                            torch.from_numpy(eid).to(dev), E))
    assert not down[1].any() and not down[2].any() and down[0].any() and down[3].any()


def test_gather_rejects_bad_arguments(vpq, dev):
    L = vpq.load()
    one = torch.zeros(4096, dtype=torch.int32, device=dev)
    p = one.data_ptr()
    assert L.vpq_gather_qmv_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, None, 1, 1, 1, capi.VPQ_GATE_SWIGLU) == -1
    assert L.vpq_gather_qmv_gated_w4g64_bf16(None, p, p, p, p, p, 64, 7, p, 1, 1, 1, capi.VPQ_GATE_SWIGLU) == -2   # odd N
    assert L.vpq_gather_qmv_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, p, 0, 1, 1, capi.VPQ_GATE_SWIGLU) == -2   # no pair
    assert L.vpq_gather_qmv_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, p, 1, 0, 1, capi.VPQ_GATE_SWIGLU) == -2   # top_k 0
    assert L.vpq_gather_qmv_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, p, 1, 1, 1, 7) == -2                      # activation
    assert L.vpq_gather_down_qmv_w4g64_bf16(None, p, p, p, p, p, 60, 8, p, 1, 1) == -2                             # K % 64
    assert L.vpq_gather_down_qmv_w4g64_bf16(None, p, p, p, p, p, 64, 8, p, 70000, 1) == -2                         # grid limit
