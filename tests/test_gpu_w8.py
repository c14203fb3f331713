"""GPU parity of the 8-bit group-64 twins (dense expansion bit-exact, QMV, the dequant-once GEMM route)
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from tests import parity
from vpipe_amd import synth

pytestmark = pytest.mark.gpu


def stage(D, dev, w, s, b, x=None):
    out = [D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev)]
    if x is not None:
        out.append(D.bf16(x, dev))
    return out


@pytest.mark.parametrize("N,K", [(1, 64), (33, 192), (257, 3840), (2048, 4096)])
def test_dequant_w8_bit_exact(vpq, oracle, dev, D, N, K):
    w, s, b = synth.make_weight8(N, K, 11 + N)
    wd, sd, bd = stage(D, dev, w, s, b)
    out = parity.Guarded((N, K), torch.bfloat16, dev)
    vpq.dequant_w8g64(wd, sd, bd, K, N, out=out.view)
    torch.cuda.synchronize()
    assert np.array_equal(D.bits(out.view), oracle.dequant8_bf16(w, s, b, K, N))
    out.assert_intact()


@pytest.mark.parametrize("K,N,M", [(64, 5, 1), (192, 33, 3), (1024, 48, 2), (3840, 16, 1), (4096, 95, 8), (2560, 64, 16),
                                  (5120, 4096, 1)])
def test_qmv_w8(vpq, oracle, dev, D, K, N, M):
    w, s, b = synth.make_weight8(N, K, 2000 + K + N)
    x = synth.make_act(M, K, 2100 + K + M)
    y64, yb = oracle.matmul8(w, s, b, x, K, N, M, rounded=False)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    f = vpq.qmv_w8g64(wd, sd, bd, xd, K, N, M, f32out=True)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w8g64(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    parity.check_f32(f.cpu().numpy(), y64)
    parity.check_bf16(D.bits(out.view), y64, yb)
    out.assert_intact()


def test_qmv_w8_residual_add(vpq, oracle, dev, D):
    K, N, M = 1024, 40, 2
    w, s, b = synth.make_weight8(N, K, 31)
    x = synth.make_act(M, K, 32)
    res = synth.make_act(M, N, 33)
    _, yb = oracle.matmul8(w, s, b, x, K, N, M, rounded=False)
    want = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(yb) + synth.bf16_bits_to_f32(res))
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    got = D.bits(vpq.qmv_w8g64(wd, sd, bd, xd, K, N, M, residual=D.bf16(res, dev)))
    assert (parity.bf16_ulp_distance(got, want) <= 1).all()


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (130, 320, 256), (257, 129, 512)])
def test_qmm_w8_dense_route(vpq, oracle, dev, D, M, N, K):
    w, s, b = synth.make_weight8(N, K, 4000 + N)
    x = synth.make_act(M, K, 4100 + M)
    y64, yb = oracle.matmul8(w, s, b, x, K, N, M, rounded=True)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    wdeq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    y = vpq.qmm_dense_route_w8g64(wd, sd, bd, xd, K, N, M, wdeq)
    torch.cuda.synchronize()
    assert np.array_equal(D.bits(wdeq), oracle.dequant8_bf16(w, s, b, K, N))
    parity.check_bf16(D.bits(y), y64, yb)
    y2 = vpq.qmm_dense_route_w8g64(wd, sd, bd, xd, K, N, M, wdeq, expand=False)
    assert torch.equal(y, y2)
