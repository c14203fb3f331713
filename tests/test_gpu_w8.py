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


def interleaved8(ffn, K, seed):
    """Gate and up 8-bit packs and their interleaved [2*ffn, ...] form (row 2g gate, 2g+1 up)."""
    g = synth.make_weight8(ffn, K, seed)
    u = synth.make_weight8(ffn, K, seed + 1)
    return tuple(np.stack([a, b], axis=1).reshape((2 * ffn,) + a.shape[1:]) for a, b in zip(g, u))


@pytest.mark.parametrize("activation", [1, 2])
@pytest.mark.parametrize("K,ffn,M", [(64, 3, 1), (1024, 40, 2), (3840, 17, 1), (4096, 96, 16)])
def test_qmv_w8_gated(vpq, oracle, dev, D, K, ffn, M, activation):
    w, s, b = interleaved8(ffn, K, 2300 + K + ffn)
    x = synth.make_act(M, K, 2400 + K + M)
    y64, _ = oracle.matmul8(w, s, b, x, K, 2 * ffn, M, rounded=False)
    want64, wantb = (oracle.swiglu if activation == 1 else oracle.geglu)(y64)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, ffn), torch.bfloat16, dev)
    vpq.qmv_gated_w8g64(wd, sd, bd, xd, K, 2 * ffn, M, out=out.view, activation=activation)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_bf16(D.bits(out.view), want64, wantb, mismatch_over_all=activation == 1)


@pytest.mark.parametrize("activation", [1, 2])
def test_gathered_expert_projections_w8(vpq, oracle, dev, D, activation):
    # the MoE block of the 4-bit gather tests with 8-bit experts: every pair against the oracle on its
    # expert's slab and bit for bit against the plain 8-bit calls on that slab
    K, inner, H, E, top_k, M = 1024, 48, 200, 5, 3, 2
    gu = [interleaved8(inner, K, 2500 + 7 * e) for e in range(E)]
    dn = [synth.make_weight8(H, 64 * ((inner + 63) // 64), 2600 + e) for e in range(E)]
    Kd = 64 * ((inner + 63) // 64)
    guw, gus, gub = (np.stack([p[i] for p in gu]) for i in range(3))
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(M, K, 2700)
    npair = M * top_k
    eid = np.array([4, 0, 2, 1, 4, 3], dtype=np.int32)
    eidd = torch.from_numpy(eid).to(dev)
    guwd, gusd, gubd, xd = stage(D, dev, guw, gus, gub, x)
    act = parity.Guarded((npair, inner), torch.bfloat16, dev)
    vpq.gather_qmv_gated_w8g64(guwd, gusd, gubd, xd, K, 2 * inner, eidd, top_k, E, out=act.view, activation=activation)
    torch.cuda.synchronize()
    act.assert_intact()
    got = D.bits(act.view)
    fn = oracle.swiglu if activation == 1 else oracle.geglu
    want64 = np.empty((npair, inner))
    wantb = np.empty((npair, inner), dtype=np.uint16)
    for p in range(npair):
        e, t = int(eid[p]), p // top_k
        y64, _ = oracle.matmul8(guw[e], gus[e], gub[e], x[t:t + 1], K, 2 * inner, 1, rounded=False)
        want64[p], wantb[p] = (a[0] for a in fn(y64))
        plain = vpq.qmv_gated_w8g64(guwd[e], gusd[e], gubd[e], xd[t:t + 1], K, 2 * inner, 1, activation=activation)
        assert np.array_equal(got[p], D.bits(plain)[0])
    parity.check_bf16(got, want64, wantb, mismatch_over_all=activation == 1)
    # down: x [npair, Kd] in pair order
    xs = synth.make_act(npair, Kd, 2701)
    dwd, dsd, dbd, xsd = stage(D, dev, dw, ds, db, xs)
    part = parity.Guarded((npair, H), torch.bfloat16, dev)
    vpq.gather_down_qmv_w8g64(dwd, dsd, dbd, xsd, Kd, H, eidd, E, out=part.view)
    torch.cuda.synchronize()
    part.assert_intact()
    gotd = D.bits(part.view)
    d64 = np.empty((npair, H))
    dbits = np.empty((npair, H), dtype=np.uint16)
    for p in range(npair):
        e = int(eid[p])
        a64, ab = oracle.matmul8(dw[e], ds[e], db[e], xs[p:p + 1], Kd, H, 1, rounded=False)
        d64[p], dbits[p] = a64[0], ab[0]
        plain = vpq.qmv_w8g64(dwd[e], dsd[e], dbd[e], xsd[p:p + 1], Kd, H, 1)
        assert np.array_equal(gotd[p], D.bits(plain)[0])
    parity.check_bf16(gotd, d64, dbits)


def test_w8_gather_ids_out_of_range_and_bad_arguments(vpq, dev, D):
    K, inner, E = 256, 8, 3
    w, s, b = (np.stack([p[i] for p in [interleaved8(inner, K, 2800 + e) for e in range(E)]]) for i in range(3))
    x = synth.make_act(2, K, 2801)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    eid = torch.tensor([1, -1, E, 2], dtype=torch.int32, device=dev)
    got = D.bits(vpq.gather_qmv_gated_w8g64(wd, sd, bd, xd, K, 2 * inner, eid, 2, E))
    assert not got[1].any() and not got[2].any() and got[0].any() and got[3].any()
    L = vpq.load()
    p = wd.data_ptr()
    assert L.vpq_qmv_gated_w8g64_bf16(None, p, p, p, p, p, 64, 7, 1, 1) == -2          # odd N
    assert L.vpq_qmv_gated_w8g64_bf16(None, p, p, p, p, p, 64, 8, 17, 1) == -2         # rows
    assert L.vpq_qmv_gated_w8g64_bf16(None, p, p, p, p, p, 64, 8, 1, 5) == -2          # activation
    assert L.vpq_gather_down_qmv_w8g64_bf16(None, p, p, p, p, p, 64, 8, None, 1, 1) == -1
    assert L.vpq_gather_qmv_gated_w8g64_bf16(None, p, p, p, p, p, 64, 8, p, 1, 0, 1, 1) == -2   # top_k 0


@pytest.mark.parametrize("activation", [1, 2])
@pytest.mark.parametrize("gate_bits,up_bits", [(4, 8), (8, 4), (4, 4), (8, 8)])
def test_gathered_gate_up_at_mixed_widths(vpq, oracle, dev, D, gate_bits, up_bits, activation):
    # gate and up as separate batched packs, each at its own width: every pair against the oracle's sums of
    # the two packs of its expert (4-bit: the QMV oracle, 8-bit: its byte twin) through the gated store
    K, ffn, E, top_k, M = 1024, 40, 4, 2, 3
    mk = {4: synth.make_weight, 8: synth.make_weight8}
    gate = [mk[gate_bits](ffn, K, 2900 + 3 * e) for e in range(E)]
    up = [mk[up_bits](ffn, K, 2950 + 3 * e) for e in range(E)]
    gs = tuple(np.stack([p[i] for p in gate]) for i in range(3))
    us = tuple(np.stack([p[i] for p in up]) for i in range(3))
    x = synth.make_act(M, K, 2990)
    eid = np.array([3, 0, 1, 1, 2, 3], dtype=np.int32)
    npair = eid.size
    gd, ud = stage(D, dev, *gs), stage(D, dev, *us)
    xd = D.bf16(x, dev)
    out = parity.Guarded((npair, ffn), torch.bfloat16, dev)
    vpq.gather_qmv_gated_split(gd, gate_bits, ud, up_bits, xd, K, ffn, torch.from_numpy(eid).to(dev), top_k, E, out=out.view,
                               activation=activation)
    torch.cuda.synchronize()
    out.assert_intact()

    def sums(bits, pack, xr):
        if bits == 4:
            return oracle.qmv(pack[0], pack[1], pack[2], xr, K, ffn, 1)[0]
        return oracle.matmul8(pack[0], pack[1], pack[2], xr, K, ffn, 1, rounded=False)[0]
    fn = oracle.swiglu if activation == 1 else oracle.geglu
    want64 = np.empty((npair, ffn))
    wantb = np.empty((npair, ffn), dtype=np.uint16)
    for p in range(npair):
        e, t = int(eid[p]), p // top_k
        y = np.empty((1, 2 * ffn))
        y[0, 0::2] = sums(gate_bits, gate[e], x[t:t + 1])[0]
        y[0, 1::2] = sums(up_bits, up[e], x[t:t + 1])[0]
        want64[p], wantb[p] = (a[0] for a in fn(y))
    parity.check_bf16(D.bits(out.view), want64, wantb, mismatch_over_all=activation == 1)
    # without experts: rows of x against expert 0's packs
    plain = vpq.gather_qmv_gated_split([t[0] for t in gd], gate_bits, [t[0] for t in ud], up_bits, xd, K, ffn, None, 1, 1,
                                       activation=activation)
    again = vpq.gather_qmv_gated_split(gd, gate_bits, ud, up_bits, xd, K, ffn, torch.zeros(M, dtype=torch.int32, device=dev), 1, E,
                                       activation=activation)
    assert torch.equal(plain, again)


def test_mixed_width_gather_rejects_bad_arguments(vpq, dev):
    L = vpq.load()
    p = torch.zeros(4096, dtype=torch.int32, device=dev).data_ptr()
    f = L.vpq_gather_qmv_gated_split_bf16
    assert f(None, p, p, p, 4, p, p, p, 8, p, p, 64, 8, p, 1, 1, 1, 1) == 0
    assert f(None, p, p, p, 5, p, p, p, 8, p, p, 64, 8, p, 1, 1, 1, 1) == -2     # width
    assert f(None, p, p, p, 4, None, p, p, 8, p, p, 64, 8, p, 1, 1, 1, 1) == -1
    assert f(None, p, p, p, 4, p, p, p, 8, p, p, 64, 8, None, 17, 1, 1, 1) == -2  # rows without experts
    assert f(None, p, p, p, 4, p, p, p, 8, p, p, 64, 8, p, 1, 1, 1, 3) == -2     # activation


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (300, 200, 128), (257, 129, 512), (40, 384, 1024), (520, 260, 1536)])
def test_qmm_w8_fused_tile_kernel(vpq, oracle, dev, D, M, N, K):
    # byte codes through the fused tile kernel: the GEMM oracle (bf16-rounded weights), and the expansion the
    # dequant-once route makes holds the same weights
    w, s, b = synth.make_weight8(N, K, 3400 + M)
    x = synth.make_act(M, K, 3401 + M)
    y64, yb = oracle.matmul8(w, s, b, x, K, N, M, rounded=True)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_w8g64(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_bf16(D.bits(out.view), y64, yb)


@pytest.mark.parametrize("tile_n", [192, -128])
@pytest.mark.parametrize("M,N,K", [(64, 64, 512), (300, 200, 1024), (257, 136, 512), (520, 392, 1536)])
def test_qmm_w8_large_tile_kernel(vpq, oracle, dev, D, M, N, K, tile_n):
    """Byte codes through the large-tile kernel (tiles of 192 and 128 weight rows): the GEMM oracle, the bits of
    the 256 x 128 tile kernel (same weights, same order of accumulation along K), both gated stores."""
    w, s, b = synth.make_weight8(N, K, 3600 + M)
    x = synth.make_act(M, K, 3601 + M)
    y64, yb = oracle.matmul8(w, s, b, x, K, N, M, rounded=True)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_w8g64(wd, sd, bd, xd, K, N, M, out=out.view, tile_n=tile_n)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_bf16(D.bits(out.view), y64, yb)
    assert torch.equal(out.view, vpq.qmm_w8g64(wd, sd, bd, xd, K, N, M, tile_n=128))
    for activation, fn in ((1, oracle.swiglu), (2, oracle.geglu)):
        want64, wantb = fn(y64)
        og = parity.Guarded((M, N // 2), torch.bfloat16, dev)
        vpq.qmm_w8g64(wd, sd, bd, xd, K, N, M, out=og.view, activation=activation, tile_n=tile_n)
        torch.cuda.synchronize()
        og.assert_intact()
        parity.check_bf16(D.bits(og.view), want64, wantb, mismatch_over_all=activation == 1)
        assert torch.equal(og.view, vpq.qmm_w8g64(wd, sd, bd, xd, K, N, M, activation=activation, tile_n=128))


def test_qmm_w8_kernel_names_reject(vpq, dev):
    L = vpq.load()
    p = torch.zeros(1 << 16, dtype=torch.int32, device=dev).data_ptr()
    assert L.vpq_qmm_tiled_w8g64_bf16(None, p, p, p, p, p, 512, 8, 4, 0, 256) == -2      # byte codes: up to 192 rows
    assert L.vpq_qmm_tiled_w8g64_bf16(None, p, p, p, p, p, 448, 8, 4, 0, 192) == -2      # K % 512
    assert L.vpq_qmm_tiled_w8g64_bf16(None, p, p, p, p, p, 512, 7, 4, 1, 192) == -2      # gated: even N


@pytest.mark.parametrize("activation", [1, 2])
def test_qmm_w8_gated_store(vpq, oracle, dev, D, activation):
    K, ffn, M = 512, 100, 270
    w, s, b = interleaved8(ffn, K, 3500)
    x = synth.make_act(M, K, 3501)
    y64, _ = oracle.matmul8(w, s, b, x, K, 2 * ffn, M, rounded=True)
    want64, wantb = (oracle.swiglu if activation == 1 else oracle.geglu)(y64)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    got = vpq.qmm_w8g64(wd, sd, bd, xd, K, 2 * ffn, M, activation=activation)
    parity.check_bf16(D.bits(got), want64, wantb, mismatch_over_all=activation == 1)


@pytest.mark.parametrize("activation", [1, 2])
@pytest.mark.parametrize("K,inner,H,E,T,top_k", [(512, 96, 200, 5, 9, 2), (1024, 40, 130, 16, 5, 3), (192, 64, 64, 3, 20, 1)])
def test_sorted_expert_gemv_w8_two_slots_per_tile(vpq, oracle, dev, D, K, inner, H, E, T, top_k, activation):
    """gpu-kernels/metal/quant/affine_qmv.metal:2718-2719 (`affine_grouped_swiglu_w8g64`, `affine_grouped_down_w8g64`,
    MAXM = 2) over 8-bit experts: QMV arithmetic against the oracle on every live slot, padding slots and unused
    tiles untouched, a live slot bit for bit the pair-gathered 8-bit call of its expert on its row."""
    from vpipe_amd import capi
    B = capi.VPQ_QMV_GROUPED_SLOTS
    Kd = 64 * ((inner + 63) // 64)
    gu = [interleaved8(inner, K, 3900 + 5 * e) for e in range(E)]
    dn = [synth.make_weight8(H, Kd, 3950 + e) for e in range(E)]
    guw, gus, gub = (np.stack([p[i] for p in gu]) for i in range(3))
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(T, K, 3990 + K)
    eid = np.random.default_rng(3991 + K).integers(0, E, size=T * top_k, dtype=np.int32)
    eid_d = torch.from_numpy(eid).to(dev)
    t2e_d, srow_d, sdst_d, _ = vpq.moe_sort_pairs(eid_d, top_k, E, block_rows=B)
    t2e, srow, sdst = (o.cpu().numpy() for o in (t2e_d, srow_d, sdst_d))
    npad = srow.size
    live = srow >= 0
    slots = np.nonzero(live)[0]
    assert slots.size == eid.size
    seven = D.bits(torch.full((1,), 7.0, dtype=torch.bfloat16))[0]

    guwd, gusd, gubd, xd = stage(D, dev, guw, gus, gub, x)
    act_out = parity.Guarded((npad, inner), torch.bfloat16, dev)
    act_out.view.fill_(7.0)
    vpq.qmv_grouped_gated_w8g64(guwd, gusd, gubd, xd, K, 2 * inner, t2e_d, srow_d, E, out=act_out.view, activation=activation)
    torch.cuda.synchronize()
    act_out.assert_intact()
    got = D.bits(act_out.view)
    assert (got[~live] == seven).all()
    y64 = np.concatenate([oracle.matmul8(guw[t2e[s // B]], gus[t2e[s // B]], gub[t2e[s // B]], x[srow[s]:srow[s] + 1], K, 2 * inner, 1,
                                         rounded=False)[0] for s in slots])
    want64, wantb = (oracle.swiglu if activation == 1 else oracle.geglu)(y64)
    parity.check_bf16(got[slots], want64, wantb, mismatch_over_all=activation == 1)
    pairwise = D.bits(vpq.gather_qmv_gated_w8g64(guwd, gusd, gubd, xd, K, 2 * inner, eid_d, top_k, E, activation=activation))
    assert np.array_equal(got[slots], pairwise[sdst[slots]])

    xs = synth.make_act(npad, Kd, 3995 + K)
    dwd, dsd, dbd, xsd = stage(D, dev, dw, ds, db, xs)
    down = parity.Guarded((npad, H), torch.bfloat16, dev)
    down.view.fill_(7.0)
    vpq.qmv_grouped_down_w8g64(dwd, dsd, dbd, xsd, Kd, H, t2e_d, srow_d, E, out=down.view)
    torch.cuda.synchronize()
    down.assert_intact()
    gotd = D.bits(down.view)
    assert (gotd[~live] == seven).all()
    pairs = [oracle.matmul8(dw[t2e[s // B]], ds[t2e[s // B]], db[t2e[s // B]], xs[s:s + 1], Kd, H, 1, rounded=False) for s in slots]
    parity.check_bf16(gotd[slots], np.concatenate([p[0] for p in pairs]), np.concatenate([p[1] for p in pairs]))
    slot_eid = torch.from_numpy(np.ascontiguousarray(t2e[slots // B]).astype(np.int32)).to(dev)
    pairwise = D.bits(vpq.gather_down_qmv_w8g64(dwd, dsd, dbd, xsd[torch.from_numpy(slots).to(dev)].contiguous(), Kd, H, slot_eid, E))
    assert np.array_equal(gotd[slots], pairwise)
    L = vpq.load()
    p = xsd.data_ptr()
    assert L.vpq_qmv_grouped_gated_w8g64_bf16(None, p, p, p, p, p, 64, 8, 3, p, p, 1, 1) == -2      # not whole tiles
    assert L.vpq_qmv_grouped_down_w8g64_bf16(None, p, p, p, p, p, 60, 8, 2, p, p, 1) == -2          # K % 64


@pytest.mark.parametrize("K,inner,H,E,T,top_k", [(512, 128, 300, 5, 150, 2), (1024, 64, 100, 4, 90, 2), (576, 96, 512, 3, 60, 1)])
def test_grouped_expert_gemms_w8(vpq, oracle, dev, D, K, inner, H, E, T, top_k):
    # the expert-sorted prefill GEMMs over 8-bit experts (K = 576: the per-step scale loads, K % 512 == 0: the
    # ring; N <= 128: the narrow tile), against the oracle on the same slots; a slot equals the plain fused
    # 8-bit GEMM on its row and slab bit for bit
    B = vpq.grouped_block_rows()
    Kd = 64 * ((inner + 63) // 64)
    gu = [interleaved8(inner, K, 3600 + 5 * e) for e in range(E)]
    dn = [synth.make_weight8(H, Kd, 3700 + e) for e in range(E)]
    guw, gus, gub = (np.stack([p[i] for p in gu]) for i in range(3))
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(T, K, 3800)
    eid = np.random.default_rng(3801 + K).integers(0, E, size=T * top_k, dtype=np.int32)
    npair = eid.size
    t2e_d, srow_d, sdst_d, ntiles_d = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E)
    t2e, srow, sdst = (o.cpu().numpy() for o in (t2e_d, srow_d, sdst_d))
    npad, used = srow.size, int(ntiles_d.cpu()[0])
    guwd, gusd, gubd, xd = stage(D, dev, guw, gus, gub, x)
    act = parity.Guarded((npad, inner), torch.bfloat16, dev)
    vpq.qmm_grouped_gated_w8g64(guwd, gusd, gubd, xd, K, 2 * inner, t2e_d, srow_d, E, out=act.view)
    torch.cuda.synchronize()
    act.assert_intact()
    got = D.bits(act.view)
    y64, _ = oracle.qmm_grouped(guw, gus, gub, x, K, 2 * inner, B, t2e, srow=srow, bits=8)
    want64, wantb = oracle.swiglu(y64[:used * B])
    live = srow[:used * B] >= 0
    assert not got[:used * B][~live].any()
    parity.check_bf16(got[:used * B][live], want64[live], wantb[live])
    for e in np.unique(eid):
        slots = np.nonzero((t2e[np.arange(npad) // B] == e) & (srow >= 0))[0]
        rows = torch.from_numpy(srow[slots].astype(np.int64)).to(dev)
        plain = vpq.qmm_w8g64(guwd[e], gusd[e], gubd[e], xd[rows].contiguous(), K, 2 * inner, len(slots), activation=1)
        assert np.array_equal(got[slots], D.bits(plain)), "expert %d" % e
    xs = synth.make_act(npad, Kd, 3802)
    dwd, dsd, dbd, xsd = stage(D, dev, dw, ds, db, xs)
    part = parity.Guarded((npair, H), torch.bfloat16, dev)
    vpq.qmm_grouped_down_w8g64(dwd, dsd, dbd, xsd, Kd, H, t2e_d, sdst_d, E, out=part.view)
    torch.cuda.synchronize()
    part.assert_intact()
    d64, dbits = oracle.qmm_grouped(dw, ds, db, xs, Kd, H, B, t2e, sdst=sdst, rows_y=npair, bits=8)
    parity.check_bf16(D.bits(part.view), d64, dbits)


@pytest.mark.parametrize("M", [1, 16, 40, 64, 65, 300])
def test_linear_entrances_of_the_format_twins(vpq, dev, D, M):
    # up to 64 rows slabs of the GEMV, above the fused GEMM: the bits of the direct calls
    K, N = 512, 136
    x = synth.make_act(M, K, 4100 + M)
    xd = D.bf16(x, dev)
    w8 = stage(D, dev, *synth.make_weight8(N, K, 4101))
    g32 = stage(D, dev, *synth.make_weight_g32(N, K, 4102))
    got8 = vpq.linear_twin("w8g64", *w8, xd, K, N, M)
    got32 = vpq.linear_twin("w4g32", *g32, xd, K, N, M)
    if M <= 64:
        want8 = torch.cat([vpq.qmv_w8g64(*w8, xd[m0:m0 + 16].contiguous(), K, N, min(16, M - m0)) for m0 in range(0, M, 16)])
        want32 = torch.cat([vpq.qmv_w4g32(*g32, xd[m0:m0 + 16].contiguous(), K, N, min(16, M - m0)) for m0 in range(0, M, 16)])
    else:
        want8 = vpq.qmm_w8g64(*w8, xd, K, N, M)
        want32 = vpq.qmm_w4g32(*g32, xd, K, N, M)
    assert torch.equal(got8, want8) and torch.equal(got32, want32)
    # a group-32 pack with K % 64 == 32 has no fused GEMM: slabs at every M
    K2 = 480
    g2 = stage(D, dev, *synth.make_weight_g32(N, K2, 4103))
    x2 = D.bf16(synth.make_act(M, K2, 4104), dev)
    got = vpq.linear_twin("w4g32", *g2, x2, K2, N, M)
    want = torch.cat([vpq.qmv_w4g32(*g2, x2[m0:m0 + 16].contiguous(), K2, N, min(16, M - m0)) for m0 in range(0, M, 16)])
    assert torch.equal(got, want)


@pytest.mark.parametrize("K,M", [(64, 1), (2048, 1), (2048, 37), (4096, 300)])
def test_moe_shared_expert_gate_w8(vpq, oracle, dev, D, K, M):
    """affine_moe_gate_w8g64 (gpu-kernels/metal/quant/affine_qmv.metal:1323-1349): gate[m] = sigmoid(W[1,K] . x[m]) over
    a one-row 8-bit pack, against the 8-bit GEMV oracle's float64 logits through numpy's logistic."""
    w, s, b = synth.make_weight8(1, K, 5000 + K)
    # logits of order 1: shrink the activations, otherwise every gate saturates
    x = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(synth.make_act(M, K, 5100 + K + M)) * np.float32(2.0 / np.sqrt(K)))
    y64, _ = oracle.matmul8(w, s, b, x, K, 1, M, rounded=False)
    want = 1.0 / (1.0 + np.exp(-y64[:, 0]))
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    out = parity.Guarded((M,), torch.bfloat16, dev)
    vpq.moe_gate_w8g64(wd, sd, bd, xd, K, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    got = synth.bf16_bits_to_f32(D.bits(out.view)).astype(np.float64)
    assert 0.05 < want.min() or M == 1 or want.std() > 0.01        # the case is not degenerate
    assert np.abs(got - want).max() <= 2e-3 * np.abs(want).max() + 2.0 ** -9
    L = vpq.load()
    p = out.view.data_ptr()
    assert L.vpq_moe_gate_w8g64_bf16(None, p, p, p, p, None, K, M) == -1
    assert L.vpq_moe_gate_w8g64_bf16(None, p, p, p, p, p, K, 0) == -2
    assert L.vpq_moe_gate_w8g64_bf16(None, p, p, p, p, p, K + 4, M) == -2


@pytest.mark.parametrize("K,M,rows", [(4096, 1, (256, 64, 64)), (192, 3, (33, 7)), (2048, 16, (48, 16, 16))])
def test_qmv_group_w8_is_the_separate_calls(vpq, dev, D, K, M, rows):
    """affine_qmv_qkv_w8g64 (gpu-kernels/metal/quant/affine_qmv.metal:540-559): the row-concatenated q|k|v pack behind
    one call; every output has the bits of its own vpq_qmv_w8g64_bf16 call, guard bands intact."""
    N = sum(rows)
    w, s, b = synth.make_weight8(N, K, 5400 + K + N)
    x = synth.make_act(M, K, 5500 + K + M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    packs, r0 = [], 0
    for n in rows:
        packs.append((wd[r0:r0 + n], sd[r0:r0 + n], bd[r0:r0 + n], n))
        r0 += n
    outs = [parity.Guarded((M, n), torch.bfloat16, dev) for n in rows]
    vpq.qmv_group_w8g64(packs, xd, K, M, outs=[o.view for o in outs])
    torch.cuda.synchronize()
    for o, p in zip(outs, packs):
        o.assert_intact()
        assert torch.equal(o.view, vpq.qmv_w8g64(p[0], p[1], p[2], xd, K, p[3], M))


@pytest.mark.parametrize("K,N,M", [(32, 5, 1), (96, 33, 3), (1024, 48, 2), (4096, 95, 8), (2560, 64, 16), (5120, 1024, 1)])
def test_w8g32_dequant_qmv_and_dense_route(vpq, oracle, dev, D, K, N, M):
    """affine_dequant_w8g32 (bit-exact), affine_qmv_w8g32 (QMV arithmetic, residual add) and affine_qmm_steel_w8g32 by the
    dequant-once route, against the oracle's group-32 8-bit twins."""
    w, s, b = synth.make_weight8(N, K, 5600 + K + N, group=32)
    x = synth.make_act(M, K, 5700 + K + M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    dq = parity.Guarded((N, K), torch.bfloat16, dev)
    vpq.dequant_w8g32(wd, sd, bd, K, N, out=dq.view)
    torch.cuda.synchronize()
    dq.assert_intact()
    assert np.array_equal(D.bits(dq.view), oracle.dequant8_g32(w, s, b, K, N))
    y64, yb = oracle.matmul8(w, s, b, x, K, N, M, rounded=False, group=32)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmv_w8g32(wd, sd, bd, xd, K, N, M, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_bf16(D.bits(out.view), y64, yb)
    res = synth.make_act(M, N, 5800 + N)
    got = D.bits(vpq.qmv_w8g32(wd, sd, bd, xd, K, N, M, residual=D.bf16(res, dev)))
    want = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(D.bits(out.view)) + synth.bf16_bits_to_f32(res))
    assert np.array_equal(got, want)
    r64, rb = oracle.matmul8(w, s, b, x, K, N, M, rounded=True, group=32)
    w_deq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    gemm = vpq.qmm_dense_route_w8g32(wd, sd, bd, xd, K, N, M, w_deq)
    parity.check_bf16(D.bits(gemm), r64, rb)
    assert torch.equal(w_deq, dq.view)
    L = vpq.load()
    p = out.view.data_ptr()
    assert L.vpq_qmv_w8g32_bf16(None, p, p, p, p, p, K + 8, N, M, None) == -2
    assert L.vpq_qmm_dense_route_w8g32_bf16(None, p, p, p, p, p, K, N, M, None, 1) == -4


@pytest.mark.parametrize("N,K", [(1, 64), (37, 320), (512, 4096), (1000, 2048)])
def test_requant_w8_to_w4_bit_exact(vpq, oracle, dev, D, N, K):
    """affine_requant_w8_to_w4_g64 (gpu-kernels/metal/quant/affine_dequant.metal:134-186): codes, scales and biases of
    the 4-bit copy, bit for bit against the oracle; one group of the pack is made constant (scale 0, codes 0)."""
    w8, s8, b8 = synth.make_weight8(N, K, 5200 + N + K)
    w8[N // 2, :16] = 0x3C3C3C3C
    want = oracle.requant_w8_to_w4(w8, s8, b8, K, N)
    wd, sd, bd = stage(D, dev, w8, s8, b8)
    w4, s4, b4 = vpq.requant_w8_to_w4(wd, sd, bd, K, N)
    torch.cuda.synchronize()
    assert np.array_equal(w4.cpu().numpy().view(np.uint32), want[0])
    assert np.array_equal(D.bits(s4), want[1]) and np.array_equal(D.bits(b4), want[2])
    assert want[1][N // 2, 0] == 0 and not want[0][N // 2, :8].any()
    # the copy is a pack of the 4-bit kernels: its expansion stays within half a step (+ the roundings of the stored
    # scale and bias and of both expansions) of the 8-bit one
    d8 = synth.bf16_bits_to_f32(D.bits(vpq.dequant_w8g64(wd, sd, bd, K, N))).astype(np.float64)
    d4 = synth.bf16_bits_to_f32(D.bits(vpq.dequant_w4g64(w4, s4, b4, K, N))).astype(np.float64)
    step = np.repeat(synth.bf16_bits_to_f32(want[1]).astype(np.float64), 64, axis=1)
    assert (np.abs(d4 - d8) <= 0.5 * step + 2.0 ** -7 * (np.abs(d8) + 15 * step)).all()
    L = vpq.load()
    p = wd.data_ptr()
    assert L.vpq_requant_w8_to_w4_g64_bf16(None, p, p, p, p, p, None, K, N) == -1
    assert L.vpq_requant_w8_to_w4_g64_bf16(None, p, p, p, p, p, p, K + 32, N) == -2
    assert L.vpq_requant_w8_to_w4_g64_bf16(None, p, p, p, p + 4, p, p, K, N) == -3


@pytest.mark.parametrize("K,N", [(4096, 300), (192, 10), (1024, 33)])
@pytest.mark.parametrize("fmt", ["w8g64", "w4g32"])
def test_qmv_gelu_mul_twins(vpq, oracle, dev, D, K, N, fmt):
    """affine_qmv_gelu_mul_w8g64 / affine_qmv_gelu_mul_w4g32 (gpu-kernels/metal/quant/affine_qmv.metal:769-805): the
    store of the group-64 4-bit form on the twins' GEMV.  The fused store against the oracle's gelu_tanh(v) * mul on
    the device's own GEMV output v (whose parity other tests hold)."""
    w, s, b = synth.make_weight8(N, K, 5300 + K + N) if fmt == "w8g64" else synth.make_weight_g32(N, K, 5301 + K + N)
    x = synth.make_act(1, K, 5302 + K)
    mul = synth.make_act(1, N, 5303 + N)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    plain = vpq.qmv_w8g64 if fmt == "w8g64" else vpq.qmv_w4g32
    fused = vpq.qmv_gelu_mul_w8g64 if fmt == "w8g64" else vpq.qmv_gelu_mul_w4g32
    v_bits = D.bits(plain(wd, sd, bd, xd, K, N, 1))
    pairs = np.stack([synth.bf16_bits_to_f32(v_bits[0]).astype(np.float64),
                      synth.bf16_bits_to_f32(mul[0]).astype(np.float64)], axis=1).reshape(1, 2 * N)
    o64, ob = oracle.geglu(pairs)
    out = parity.Guarded((1, N), torch.bfloat16, dev)
    fused(wd, sd, bd, xd, K, N, D.bf16(mul, dev), out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    parity.check_bf16(D.bits(out.view), o64, ob, mismatch_over_all=False)
    assert np.abs(o64).max() > 0
    L = vpq.load()
    p = out.view.data_ptr()
    if fmt == "w8g64":
        assert L.vpq_qmv_gelu_mul_w8g64_bf16(None, p, p, p, p, p, K, N, None) == -1
    else:
        assert L.vpq_qmv_gelu_mul_w4g32_bf16(None, p, p, p, p, p, K, N, None, 0) == -1


@pytest.mark.parametrize("M,N,K,r", [(130, 264, 512, 16), (300, 136, 1024, 8), (64, 72, 192, 40)])
@pytest.mark.parametrize("fmt", [1, 2, 3])
def test_dense_route_with_adapter_over_the_format_twins(vpq, oracle, dev, D, fmt, M, N, K, r):
    """vpq_qmm_dense_route_lora_bf16: the adapter over 4-bit group-32, 8-bit group-64 and 8-bit group-32 packs by the
    dequant-once route (`gemm_` with Linear.bits 4 or 8, minimax-h3/metal-minimax-h3-transformer.cc:2205-2259).  t is
    the pre-pass's (pinned by its own tests); y against float64 of x . W^T + t . B^T with W the oracle's expansion of
    the pack; alpha = 0 and the kept expansion give the bits of the plain route."""
    alpha = 0.75
    if fmt == 1:
        w, s, b = synth.make_weight_g32(N, K, 9100 + r)
        dense = oracle.dequant_g32_bf16(w, s, b, K, N)
        plain = vpq.qmm_dense_route_w4g32
    elif fmt == 2:
        w, s, b = synth.make_weight8(N, K, 9101 + r)
        dense = oracle.dequant8_bf16(w, s, b, K, N)
        plain = vpq.qmm_dense_route_w8g64
    else:
        w, s, b = synth.make_weight8(N, K, 9102 + r, group=32)
        dense = oracle.dequant8_g32(w, s, b, K, N)
        plain = vpq.qmm_dense_route_w8g32
    x = synth.make_act(M, K, 9103)
    A, B = synth.make_lora(N, K, r, 9104, std=0.05)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    Ad, Bd = D.bf16(A, dev), D.bf16(B, dev)
    w_deq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    t_ws = parity.Guarded((M, r), torch.bfloat16, dev)
    out = parity.Guarded((M, N), torch.bfloat16, dev)
    vpq.qmm_dense_route_lora(fmt, wd, sd, bd, xd, K, N, M, w_deq, Ad, Bd, r, alpha, out=out.view, t_ws=t_ws.view)
    torch.cuda.synchronize()
    out.assert_intact()
    t_ws.assert_intact()
    assert np.array_equal(D.bits(w_deq), dense)
    assert torch.equal(t_ws.view, vpq.lora_a(xd, Ad, M, K, r, alpha))
    f64 = lambda bits: synth.bf16_bits_to_f32(bits).astype(np.float64)
    want = f64(x) @ f64(dense).T + f64(D.bits(t_ws.view)) @ f64(B).T
    parity.check_bf16(D.bits(out.view), want, synth.f32_to_bf16_bits(want.astype(np.float32)))
    base = plain(wd, sd, bd, xd, K, N, M, w_deq)
    assert not torch.equal(base, out.view)
    kept = vpq.qmm_dense_route_lora(fmt, wd, sd, bd, xd, K, N, M, w_deq, Ad, Bd, r, alpha, expand=False)
    assert torch.equal(kept, out.view)
    off = vpq.qmm_dense_route_lora(fmt, wd, sd, bd, xd, K, N, M, w_deq, Ad, Bd, r, 0.0)
    assert torch.equal(off, base)
    L = vpq.load()
    p = out.view.data_ptr()
    assert L.vpq_qmm_dense_route_lora_bf16(None, 7, p, p, p, p, p, K, N, M, p, 1, p, p, r, 1.0, p) == -2
    assert L.vpq_qmm_dense_route_lora_bf16(None, fmt, p, p, p, p, p, K, N, M, p, 1, p, p, 12, 1.0, p) == -2
    assert L.vpq_qmm_dense_route_lora_bf16(None, fmt, p, p, p, p, p, K, N, M, p, 1, p, None, r, 1.0, p) == -1
