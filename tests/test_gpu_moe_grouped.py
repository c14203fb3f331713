"""GPU parity of the expert-sorted (grouped) MoE prefill path, through the C ABI: the pair sort
against the invariants of the reference's counting sort and the CPU oracle's block map, the two
grouped GEMMs against the CPU oracle on the same sorted slots, and every slot bit for bit against
the plain tiled GEMM on that expert's slab (the reference's contract:
gpu-kernels/metal/quant/affine_qmm_steel.metal:1027-1031, "token-exact with the per-pair paths")."""
import numpy as np
import pytest
import torch

from tests import parity
from vpipe_amd import capi, synth

pytestmark = pytest.mark.gpu


def expert_batch(E, N, K, seed):
    packs = [synth.make_weight(N, K, seed + 13 * e) for e in range(E)]
    return tuple(np.stack([p[i] for p in packs]) for i in range(3))


def routed(E, T, top_k, seed, skew=False):
    rng = np.random.default_rng(seed)
    if skew:                     # a few hot experts and some that get nothing
        p = np.zeros(E)
        p[: max(2, E // 3)] = rng.random(max(2, E // 3)) + 0.2
        p /= p.sum()
        return rng.choice(E, size=T * top_k, p=p).astype(np.int32)
    return rng.integers(0, E, size=T * top_k, dtype=np.int32)


def check_sort(eid, top_k, E, B, t2e, srow, sdst, ntiles, oracle):
    npair = eid.size
    want_t2e, _, _, used = oracle.moe_sort_pairs(eid, top_k, E, B, t2e.size)
    assert int(ntiles[0]) == used
    assert np.array_equal(t2e, want_t2e)                       # the block map depends on the histogram only
    live = sdst >= 0
    assert sorted(sdst[live].tolist()) == [p for p in range(npair) if 0 <= eid[p] < E]
    assert np.array_equal(srow[live], sdst[live] // top_k) and (srow[~live] == -1).all()
    slots = np.nonzero(live)[0]
    assert np.array_equal(t2e[slots // B], eid[sdst[slots]])   # every pair sits in a block of its expert
    # an expert's pairs fill its share from the front
    hist = np.bincount(eid[(eid >= 0) & (eid < E)], minlength=E)
    first = np.concatenate([[0], np.cumsum((hist + B - 1) // B)[:-1]]) * B
    for e in range(E):
        assert live[first[e]:first[e] + hist[e]].all()


SORT_CASES = [(8, 64, 2, 128, False), (128, 2048, 8, 128, False), (128, 300, 8, 128, True), (5, 7, 3, 32, True),
              (300, 1000, 4, 2, False), (64, 1, 8, 128, False)]


@pytest.mark.parametrize("E,T,top_k,B,skew", SORT_CASES)
def test_pair_sort(vpq, oracle, dev, E, T, top_k, B, skew):
    eid = routed(E, T, top_k, 5000 + E + T, skew)
    outs = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E, block_rows=B)
    torch.cuda.synchronize()
    t2e, srow, sdst, ntiles = (o.cpu().numpy() for o in outs)
    assert t2e.size == vpq.moe_max_tiles(eid.size, E, B)
    check_sort(eid, top_k, E, B, t2e, srow, sdst, ntiles, oracle)


def test_pair_sort_skips_ids_out_of_range_and_rejects_bad_arguments(vpq, oracle, dev):
    E, B = 4, 128
    eid = np.array([1, -1, E, 0, 3, 3], dtype=np.int32)
    outs = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), 2, E, block_rows=B)
    t2e, srow, sdst, ntiles = (o.cpu().numpy() for o in outs)
    check_sort(eid, 2, E, B, t2e, srow, sdst, ntiles, oracle)
    L = vpq.load()
    buf = torch.zeros(4096, dtype=torch.int32, device=dev)
    p = buf.data_ptr()
    assert L.vpq_moe_sort_pairs(None, None, 4, 1, 4, 128, 8, p, p, p, p, p, 48) == -1
    assert L.vpq_moe_sort_pairs(None, p, 0, 1, 4, 128, 8, p, p, p, p, p, 48) == -2
    assert L.vpq_moe_sort_pairs(None, p, 600, 1, 4, 128, 8, p, p, p, p, p, 48) == -2      # too few blocks
    assert L.vpq_moe_sort_pairs(None, p, 4, 1, 4, 128, 8, p, p, p, p, p, 47) == -4        # workspace
    assert L.vpq_qmm_grouped_block_rows() == 128


# K (hidden), inner, H (down out), E, T, top_k: the Qwen3-MoE block scaled down; K of the down GEMM = inner
GROUPED_SHAPES = [(512, 128, 512, 6, 150, 2, False), (2048, 768, 2048, 16, 200, 4, True), (576, 96, 200, 3, 40, 1, False),
                  (1024, 160, 1026, 9, 300, 3, True), (512, 64, 100, 4, 90, 2, False)]      # last: one 128-wide tile of N


@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
@pytest.mark.parametrize("K,inner,H,E,T,top_k,skew", GROUPED_SHAPES)
def test_grouped_expert_gemms(vpq, oracle, dev, D, K, inner, H, E, T, top_k, skew, activation):
    B = vpq.grouped_block_rows()
    Kd = ((inner + 63) // 64) * 64                       # the down GEMM's K: inner padded to a group
    guw, gus, gub = expert_batch(E, 2 * inner, K, 5100 + K)
    dw, ds, db = expert_batch(E, H, Kd, 5200 + K)
    x = synth.make_act(T, K, 5300 + K)
    eid = routed(E, T, top_k, 5400 + K, skew)
    npair = eid.size
    t2e_d, srow_d, sdst_d, ntiles_d = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E)
    t2e, srow, sdst = (o.cpu().numpy() for o in (t2e_d, srow_d, sdst_d))
    npad = srow.size
    used = int(ntiles_d.cpu()[0])

    # ---- gate|up + activation over the gathered rows ----
    guwd, gusd, gubd, xd = D.u32(guw, dev), D.bf16(gus, dev), D.bf16(gub, dev), D.bf16(x, dev)
    act_out = parity.Guarded((npad, inner), torch.bfloat16, dev)
    act_out.view.fill_(7.0)                              # blocks no expert owns must stay as they are
    vpq.qmm_grouped_gated_w4g64(guwd, gusd, gubd, xd, K, 2 * inner, t2e_d, srow_d, E, out=act_out.view, activation=activation)
    torch.cuda.synchronize()
    act_out.assert_intact()
    got = D.bits(act_out.view)
    seven = D.bits(torch.full((1,), 7.0, dtype=torch.bfloat16))[0]
    assert (got[used * B:] == seven).all()
    y64, _ = oracle.qmm_grouped(guw, gus, gub, x, K, 2 * inner, B, t2e, srow=srow)
    act = oracle.swiglu if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu
    want64, wantb = act(y64[:used * B])
    live = srow[:used * B] >= 0
    assert not got[:used * B][~live].any()               # padding slots: zeros
    parity.check_bf16(got[:used * B][live], want64[live], wantb[live], mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)
    # bit for bit the plain tiled GEMM with the gated store, per expert, on the rows it was given
    for e in np.unique(eid):
        slots = np.nonzero((t2e[np.arange(npad) // B] == e) & (srow >= 0))[0]
        rows = torch.from_numpy(srow[slots].astype(np.int64)).to(dev)
        plain = vpq.qmm_swiglu_w4g64(guwd[e], gusd[e], gubd[e], xd[rows].contiguous(), K, 2 * inner, len(slots),
                                     activation=activation)
        assert np.array_equal(got[slots], D.bits(plain)), "expert %d" % e

    # ---- down over the sorted activations, scattered to pair order ----
    xs = synth.make_act(npad, Kd, 5500 + K)
    dwd, dsd, dbd, xsd = D.u32(dw, dev), D.bf16(ds, dev), D.bf16(db, dev), D.bf16(xs, dev)
    part = parity.Guarded((npair, H), torch.bfloat16, dev)
    part.view.fill_(7.0)
    vpq.qmm_grouped_down_w4g64(dwd, dsd, dbd, xsd, Kd, H, t2e_d, sdst_d, E, out=part.view)
    torch.cuda.synchronize()
    part.assert_intact()
    gotd = D.bits(part.view)
    d64, dbits = oracle.qmm_grouped(dw, ds, db, xs, Kd, H, B, t2e, sdst=sdst, rows_y=npair)
    parity.check_bf16(gotd, d64, dbits)
    for e in np.unique(eid):
        slots = np.nonzero((t2e[np.arange(npad) // B] == e) & (sdst >= 0))[0]
        rows = torch.from_numpy(slots.astype(np.int64)).to(dev)
        plain = vpq.qmm_w4g64(dwd[e], dsd[e], dbd[e], xsd[rows].contiguous(), Kd, H, len(slots), tile_n=128)
        assert np.array_equal(gotd[sdst[slots]], D.bits(plain)), "expert %d" % e


def test_grouped_gemms_reject_bad_arguments(vpq, dev):
    L = vpq.load()
    buf = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    p = buf.data_ptr()
    act = capi.VPQ_GATE_SWIGLU
    assert L.vpq_qmm_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, 128, p, None, 1, 1, act) == -1
    assert L.vpq_qmm_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, 100, p, p, 1, 1, act) == -2     # not whole blocks
    assert L.vpq_qmm_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 7, 128, p, p, 1, 1, act) == -2     # odd N
    assert L.vpq_qmm_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, 128, p, p, 1, 1, 9) == -2       # activation
    assert L.vpq_qmm_grouped_down_w4g64_bf16(None, p, p, p, p, p, 60, 8, 128, p, p, 1, 1) == -2           # K % 64
    assert L.vpq_qmm_grouped_down_w4g64_bf16(None, p, p, p, p, p, 64, 8, 128, p, p, 0, 1) == -2           # no expert
    assert L.vpq_qmm_grouped_down_w4g64_bf16(None, p, p, p, p, p, 64, 8, 128, None, p, 1, 1) == -1


def test_grouped_gemms_take_the_slots_of_a_block_in_any_order(vpq, oracle, dev, D):
    # padding slots need not trail: a permutation of the slots inside every block permutes the gate|up
    # rows and leaves the down rows (pair order) as they were, bit for bit
    K, inner, H, E, T, top_k = 512, 128, 300, 4, 50, 2
    B = vpq.grouped_block_rows()
    guw, gus, gub = expert_batch(E, 2 * inner, K, 5600)
    dw, ds, db = expert_batch(E, H, inner, 5601)
    x = synth.make_act(T, K, 5602)
    eid = routed(E, T, top_k, 5603)
    t2e, srow, sdst, _ = oracle.moe_sort_pairs(eid, top_k, E, B, vpq.moe_max_tiles(eid.size, E, B))
    npad = srow.size
    rng = np.random.default_rng(5604)
    perm = np.concatenate([t * B + rng.permutation(B) for t in range(npad // B)])
    xs = synth.make_act(npad, inner, 5605)
    guwd, gusd, gubd, xd = D.u32(guw, dev), D.bf16(gus, dev), D.bf16(gub, dev), D.bf16(x, dev)
    dwd, dsd, dbd = D.u32(dw, dev), D.bf16(ds, dev), D.bf16(db, dev)
    t2e_d = torch.from_numpy(t2e).to(dev)

    def run(srow_, sdst_, xs_):
        act = vpq.qmm_grouped_gated_w4g64(guwd, gusd, gubd, xd, K, 2 * inner, t2e_d, torch.from_numpy(srow_).to(dev), E)
        part = torch.zeros((eid.size, H), dtype=torch.bfloat16, device=dev)
        vpq.qmm_grouped_down_w4g64(dwd, dsd, dbd, D.bf16(xs_, dev), inner, H, t2e_d, torch.from_numpy(sdst_).to(dev), E,
                                   out=part)
        return D.bits(act), D.bits(part)
    act0, part0 = run(srow, sdst, xs)
    act1, part1 = run(np.ascontiguousarray(srow[perm]), np.ascontiguousarray(sdst[perm]), np.ascontiguousarray(xs[perm]))
    used = t2e >= 0
    rows_used = np.repeat(used, B)
    assert np.array_equal(act1[rows_used], act0[perm][rows_used])
    assert np.array_equal(part1, part0)
    y64, _ = oracle.qmm_grouped(guw, gus, gub, x, K, 2 * inner, B, t2e, srow=srow)
    a64, ab = oracle.swiglu(y64)
    live = srow >= 0
    parity.check_bf16(act0[live], a64[live], ab[live])


# K (hidden), inner, H (down out), E, T, top_k: a few rows per expert, the case the two-slot tiles are for
SORTED_QMV_SHAPES = [(512, 128, 512, 6, 9, 2, False), (2048, 768, 2048, 16, 20, 4, True), (576, 96, 200, 3, 5, 1, False),
                     (1024, 160, 1026, 40, 16, 8, True)]


@pytest.mark.parametrize("activation", [capi.VPQ_GATE_SWIGLU, capi.VPQ_GATE_GEGLU])
@pytest.mark.parametrize("K,inner,H,E,T,top_k,skew", SORTED_QMV_SHAPES)
def test_sorted_expert_gemv_two_slots_per_tile(vpq, oracle, dev, D, K, inner, H, E, T, top_k, skew, activation):
    """gpu-kernels/metal/quant/affine_qmv.metal:2551-2719 (`affine_grouped_swiglu_w4g64`, `affine_grouped_down_w4g64`,
    MAXM = 2): QMV arithmetic (weight never rounded) over pairs sorted into per-expert tiles of two slots; padding
    slots and unused tiles are left untouched; a live slot is bit for bit the plain row-streaming QMV."""
    B = capi.VPQ_QMV_GROUPED_SLOTS
    Kd = ((inner + 63) // 64) * 64
    guw, gus, gub = expert_batch(E, 2 * inner, K, 6100 + K)
    dw, ds, db = expert_batch(E, H, Kd, 6200 + K)
    x = synth.make_act(T, K, 6300 + K)
    eid = routed(E, T, top_k, 6400 + K, skew)
    t2e_d, srow_d, sdst_d, ntiles_d = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E, block_rows=B)
    t2e, srow, sdst = (o.cpu().numpy() for o in (t2e_d, srow_d, sdst_d))
    check_sort(eid, top_k, E, B, t2e, srow, sdst, ntiles_d.cpu().numpy(), oracle)
    npad = srow.size
    live = srow >= 0
    seven = D.bits(torch.full((1,), 7.0, dtype=torch.bfloat16))[0]

    # ---- gate|up + activation, x rows gathered through srow ----
    guwd, gusd, gubd, xd = D.u32(guw, dev), D.bf16(gus, dev), D.bf16(gub, dev), D.bf16(x, dev)
    act_out = parity.Guarded((npad, inner), torch.bfloat16, dev)
    act_out.view.fill_(7.0)
    vpq.qmv_grouped_gated_w4g64(guwd, gusd, gubd, xd, K, 2 * inner, t2e_d, srow_d, E, out=act_out.view, activation=activation)
    torch.cuda.synchronize()
    act_out.assert_intact()
    got = D.bits(act_out.view)
    assert (got[~live] == seven).all()                   # padding slots and unused tiles: untouched
    act = oracle.swiglu if activation == capi.VPQ_GATE_SWIGLU else oracle.geglu
    slots = np.nonzero(live)[0]
    y64 = np.concatenate([oracle.qmv(guw[t2e[s // B]], gus[t2e[s // B]], gub[t2e[s // B]], x[srow[s]:srow[s] + 1], K, 2 * inner, 1)[0]
                          for s in slots])
    want64, wantb = act(y64)
    parity.check_bf16(got[slots], want64, wantb, mismatch_over_all=activation == capi.VPQ_GATE_SWIGLU)
    for s in slots:
        e = int(t2e[s // B])
        plain = vpq.qmv_swiglu_w4g64(guwd[e], gusd[e], gubd[e], xd[int(srow[s]):int(srow[s]) + 1].contiguous(), K, 2 * inner, 1,
                                     variant=capi.VPQ_QMV_ROWS, activation=activation)
        assert np.array_equal(got[s], D.bits(plain)[0]), "slot %d" % s

    # ---- down over the sorted activations, y in slot order ----
    xs = synth.make_act(npad, Kd, 6500 + K)
    dwd, dsd, dbd, xsd = D.u32(dw, dev), D.bf16(ds, dev), D.bf16(db, dev), D.bf16(xs, dev)
    down = parity.Guarded((npad, H), torch.bfloat16, dev)
    down.view.fill_(7.0)
    vpq.qmv_grouped_down_w4g64(dwd, dsd, dbd, xsd, Kd, H, t2e_d, srow_d, E, out=down.view)
    torch.cuda.synchronize()
    down.assert_intact()
    gotd = D.bits(down.view)
    assert (gotd[~live] == seven).all()
    pairs = [oracle.qmv(dw[t2e[s // B]], ds[t2e[s // B]], db[t2e[s // B]], xs[s:s + 1], Kd, H, 1) for s in slots]
    parity.check_bf16(gotd[slots], np.concatenate([p[0] for p in pairs]), np.concatenate([p[1] for p in pairs]))
    for s in slots:
        e = int(t2e[s // B])
        plain = vpq.qmv_w4g64(dwd[e], dsd[e], dbd[e], xsd[int(s):int(s) + 1].contiguous(), Kd, H, 1, variant=capi.VPQ_QMV_ROWS)
        assert np.array_equal(gotd[s], D.bits(plain)[0]), "slot %d" % s


@pytest.mark.parametrize("H", [64, 100, 2048])
def test_scatter_back_to_pair_order(vpq, dev, D, H):
    """llm_elementwise.metal:328-342: rows in slot order go to the pair each slot names; padding slots and names
    outside [0, npair) write nothing; rows no slot names keep what they held."""
    E, T, top_k, B = 6, 11, 2, capi.VPQ_QMV_GROUPED_SLOTS
    eid = np.random.default_rng(6600 + H).integers(0, E, size=T * top_k, dtype=np.int32)
    eid[3] = -1                                            # a pair without a slot
    _, _, sdst_d, _ = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E, block_rows=B)
    sdst = sdst_d.cpu().numpy()
    npad, npair = sdst.size, eid.size
    rows = synth.make_act(npad, H, 6601 + H)
    rows_d = D.bf16(rows, dev)
    out = parity.Guarded((npair, H), torch.bfloat16, dev)
    out.view.fill_(7.0)
    vpq.moe_scatter_back(rows_d, sdst_d, npair, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    seven = D.bits(torch.full((1,), 7.0, dtype=torch.bfloat16))[0]
    want = np.full((npair, H), seven, dtype=np.uint16)
    for s_, p_ in enumerate(sdst):
        if p_ >= 0:
            want[p_] = rows[s_]
    assert np.array_equal(D.bits(out.view), want)
    assert (want[3] == seven).all() and (want[eid >= 0] != seven).any()
    # a name past the pairs is skipped, not followed
    bad = sdst.copy()
    bad[np.nonzero(bad >= 0)[0][0]] = npair + 5
    out.view.fill_(7.0)
    vpq.moe_scatter_back(rows_d, torch.from_numpy(bad).to(dev), npair, out=out.view)
    torch.cuda.synchronize()
    out.assert_intact()
    L = vpq.load()
    p = rows_d.data_ptr()
    assert L.vpq_moe_scatter_back_bf16(None, p, sdst_d.data_ptr(), None, npad, H, npair) == -1
    assert L.vpq_moe_scatter_back_bf16(None, p, sdst_d.data_ptr(), p, 0, H, npair) == -2


def test_sorted_expert_gemv_rejects_bad_arguments(vpq, dev):
    L = vpq.load()
    buf = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    p = buf.data_ptr()
    act = capi.VPQ_GATE_SWIGLU
    assert L.vpq_qmv_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, 2, p, None, 1, act) == -1
    assert L.vpq_qmv_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, 3, p, p, 1, act) == -2      # not whole tiles
    assert L.vpq_qmv_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 7, 2, p, p, 1, act) == -2      # odd N
    assert L.vpq_qmv_grouped_gated_w4g64_bf16(None, p, p, p, p, p, 64, 8, 2, p, p, 1, 9) == -2        # activation
    assert L.vpq_qmv_grouped_down_w4g64_bf16(None, p, p, p, p, p, 60, 8, 2, p, p, 1) == -2            # K % 64
    assert L.vpq_qmv_grouped_down_w4g64_bf16(None, p, p, p, p, p, 64, 8, 2, p, p, 0) == -2            # no expert
    assert L.vpq_qmv_grouped_down_w4g64_bf16(None, p, p, p, p, p, 64, 8, 2, None, p, 1) == -1
