"""GPU parity of the stochastic sampler tail (gpu-kernels/metal/ops/llm_elementwise.metal:3116-3262) against the CPU
oracle, through the C ABI.  The draw is index work: the kernel fixes exp, log and the reduction order, so the token,
the cached weights and the seen flags must equal the oracle's exactly."""
import numpy as np
import pytest
import torch

from vpipe_amd import synth

pytestmark = pytest.mark.gpu

SETTINGS = [
    # temp, top_p, top_k, min_p, rep, pres, n_iter
    (1.0, 1.0, 0, 0.0, 1.0, 0.0, 24),
    (0.7, 0.9, 0, 0.0, 1.0, 0.0, 24),
    (1.3, 1.0, 40, 0.0, 1.1, 0.0, 20),
    (0.9, 0.95, 50, 0.05, 1.2, 0.4, 24),
    (1e-4, 1.0, 0, 0.0, 1.0, 0.0, 8),           # temperature -> 0: the argmax
    (1.0, 1e-6, 0, 0.0, 1.0, 0.0, 24),          # a nucleus of one
    (2.0, 0.99, 100000, 0.0, 1.0, 0.0, 0),      # top_k >= V is off; no bisection steps at all
]


def row(V, seed, scale=3.0):
    rng = np.random.default_rng(seed)
    return synth.f32_to_bf16_bits((rng.standard_normal(V) * scale).astype(np.float32))


@pytest.mark.parametrize("V", [1, 255, 1024, 5000, 151936])
@pytest.mark.parametrize("setting", range(len(SETTINGS)))
def test_sampler_matches_the_oracle(vpq, oracle, dev, D, V, setting):
    temp, top_p, top_k, min_p, rep, pres, n_iter = SETTINGS[setting]
    bits = row(V, 8000 + V + setting)
    rng = np.random.default_rng(8100 + V)
    seen = (rng.random(V) < 0.1).astype(np.uint8)
    ld = D.bf16(bits, dev)
    for seed in (0, 1, 0xdeadbeef, 12345 + V):
        want, ws_want, seen_want = oracle.sample_topp(bits, seen, temp, top_p, seed, n_iter=n_iter, rep=rep, pres=pres,
                                                      top_k=top_k, min_p=min_p)
        seen_d = torch.from_numpy(seen.copy()).to(dev)
        ws_d = torch.zeros((V,), dtype=torch.bfloat16, device=dev)
        got = vpq.sample_topp_bf16(ld, seen_d, temp, top_p, seed, ws=ws_d, n_iter=n_iter, rep=rep, pres=pres, top_k=top_k,
                                   min_p=min_p)
        torch.cuda.synchronize()
        assert int(got.cpu()[0]) == want, (seed, int(got.cpu()[0]), want)
        assert np.array_equal(D.bits(ws_d), ws_want)
        assert np.array_equal(seen_d.cpu().numpy(), seen_want)


def test_sampler_decode_steps_carry_the_seen_flags(vpq, oracle, dev, D):
    # eight steps over the same logits with a strong repetition penalty: each step marks its token, which the next
    # step penalises; device and oracle walk the same sequence
    V = 4096
    bits = row(V, 8200, scale=1.5)
    seen = np.zeros(V, dtype=np.uint8)
    seen_d = torch.zeros((V,), dtype=torch.uint8, device=dev)
    ld = D.bf16(bits, dev)
    toks = []
    for step in range(8):
        want, _, seen = oracle.sample_topp(bits, seen, 0.8, 0.9, 100 + step, rep=1.8, pres=0.5, top_k=30)
        got = vpq.sample_topp_bf16(ld, seen_d, 0.8, 0.9, 100 + step, rep=1.8, pres=0.5, top_k=30)
        torch.cuda.synchronize()
        assert int(got.cpu()[0]) == want, step
        toks.append(want)
    assert np.array_equal(seen_d.cpu().numpy(), seen) and seen.sum() == len(set(toks))


def test_sampler_special_rows(vpq, oracle, dev, D):
    V = 3000
    cases = []
    allnan = np.full(V, 0x7FC0, dtype=np.uint16)
    cases.append(allnan)                                     # nothing is kept: token 0
    ninf = np.full(V, 0xFF80, dtype=np.uint16); ninf[777] = 0x4000
    cases.append(ninf)                                       # one finite logit
    flat = np.full(V, 0x3F80, dtype=np.uint16)
    cases.append(flat)                                       # all equal: a uniform draw
    mixed = row(V, 8300); mixed[5] = 0x7FC0; mixed[6] = 0x7F80     # a NaN and +inf among the logits
    cases.append(mixed)
    seen = np.zeros(V, dtype=np.uint8)
    for bits in cases:
        for seed in (3, 4):
            want, ws_want, _ = oracle.sample_topp(bits, seen, 1.0, 0.9, seed, top_k=20)
            ws_d = torch.zeros((V,), dtype=torch.bfloat16, device=dev)
            got = vpq.sample_topp_bf16(D.bf16(bits, dev), torch.zeros((V,), dtype=torch.uint8, device=dev), 1.0, 0.9, seed,
                                       ws=ws_d, top_k=20)
            torch.cuda.synchronize()
            assert int(got.cpu()[0]) == want
            assert np.array_equal(D.bits(ws_d), ws_want)
    assert oracle.sample_topp(allnan, seen, 1.0, 0.9, 3)[0] == 0 and oracle.sample_topp(ninf, seen, 1.0, 0.9, 3)[0] == 777


def test_sampler_rejects_bad_arguments(vpq, dev):
    L = vpq.load()
    buf = torch.zeros(4096, dtype=torch.int32, device=dev)
    p = buf.data_ptr()
    assert L.vpq_sample_topp_bf16(None, None, p, 10, 1.0, 1.0, 0, p, 8, 1.0, 0.0, 0, 0.0, p) == -1
    assert L.vpq_sample_topp_bf16(None, p, p, 0, 1.0, 1.0, 0, p, 8, 1.0, 0.0, 0, 0.0, p) == -2      # no logits
    assert L.vpq_sample_topp_bf16(None, p, p, 10, 1.0, 1.0, 0, p, -1, 1.0, 0.0, 0, 0.0, p) == -2    # negative steps
    assert L.vpq_sample_topp_bf16(None, p, p, 10, 1.0, 1.0, 0, p, 8, 0.0, 0.0, 0, 0.0, p) == -2     # division by rep
    assert L.vpq_sample_topp_bf16(None, p, p + 2, 10, 1.0, 1.0, 0, p, 8, 1.0, 0.0, 0, 0.0, p) == -3


HIST_SETTINGS = [
    # temp, top_p, top_k, min_p, rep, pres
    (1.0, 1.0, 0, 0.0, 1.0, 0.0),
    (0.7, 0.9, 0, 0.0, 1.0, 0.0),
    (1.3, 1.0, 40, 0.0, 1.1, 0.0),
    (0.9, 0.95, 50, 0.05, 1.2, 0.4),
    (1e-4, 1.0, 0, 0.0, 1.0, 0.0),
    (1.0, 1e-6, 0, 0.0, 1.0, 0.0),
    (2.0, 0.99, 100000, 0.0, 1.0, 0.0),
]


@pytest.mark.parametrize("V,n_slabs", [(1, 1), (255, 1), (255, 4), (5000, 3), (5000, 64), (151936, 0), (151936, 128), (151936, 9)])
@pytest.mark.parametrize("setting", range(len(HIST_SETTINGS)))
def test_histogram_sampler_matches_the_oracle(vpq, oracle, dev, D, V, n_slabs, setting):
    """The sampler over many workgroups (llm_elementwise.metal:3255-3640): token, cached weights, seen flags and the
    weight threshold equal the oracle's exactly (counts and fixed-point masses are integer sums, everything else has
    a fixed order)."""
    temp, top_p, top_k, min_p, rep, pres = HIST_SETTINGS[setting]
    if n_slabs == 0:
        n_slabs = vpq.sample_hist_slabs(V)
    bits = row(V, 8500 + V + setting)
    rng = np.random.default_rng(8600 + V)
    seen = (rng.random(V) < 0.1).astype(np.uint8)
    ld = D.bf16(bits, dev)
    words = vpq.load().vpq_sample_hist_workspace_bytes(n_slabs) // 4
    wt_at = n_slabs + n_slabs * 2049 + 2049
    for seed in (0, 0xdeadbeef, 777 + V):
        want, ws_want, seen_want, wt_want = oracle.sample_hist(bits, seen, temp, top_p, seed, n_slabs, rep=rep, pres=pres,
                                                               top_k=top_k, min_p=min_p)
        seen_d = torch.from_numpy(seen.copy()).to(dev)
        ws_d = torch.zeros((V,), dtype=torch.bfloat16, device=dev)
        work = torch.full((words + 64,), float("nan"), dtype=torch.float32, device=dev)
        got = vpq.sample_hist_bf16(ld, seen_d, temp, top_p, seed, ws=ws_d, work=work[:words], n_slabs=n_slabs, rep=rep, pres=pres,
                                   top_k=top_k, min_p=min_p)
        torch.cuda.synchronize()
        assert int(got.cpu()[0]) == want, (seed, int(got.cpu()[0]), want)
        assert np.array_equal(D.bits(ws_d), ws_want)
        assert np.array_equal(seen_d.cpu().numpy(), seen_want)
        wk = work.cpu().numpy()
        assert wk[wt_at] == np.float32(wt_want)
        assert np.isnan(wk[words:]).all()                     # nothing written past the stated workspace


def test_histogram_sampler_rejects_bad_arguments(vpq, dev):
    L = vpq.load()
    buf = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    p = buf.data_ptr()
    nb = L.vpq_sample_hist_workspace_bytes(4)
    assert nb == 4 * (4 + 4 * 2049 + 2049 + 1 + 8) and L.vpq_sample_hist_workspace_bytes(0) == 0
    assert L.vpq_sample_hist_bf16(None, p, p, 100, 1.0, 0.9, 1, p, 1.0, 0.0, 0, 0.0, p, 4, p, nb) == 0
    assert L.vpq_sample_hist_bf16(None, p, p, 100, 1.0, 0.9, 1, p, 1.0, 0.0, 0, 0.0, p, 4, p, nb - 1) == -4     # workspace
    assert L.vpq_sample_hist_bf16(None, p, p, 100, 1.0, 0.9, 1, p, 1.0, 0.0, 0, 0.0, p, 0, p, nb) == -2         # slabs
    assert L.vpq_sample_hist_bf16(None, p, p, 200000, 1.0, 0.9, 1, p, 1.0, 0.0, 0, 0.0, p, 2, p, nb) == -2      # slab too long
    assert L.vpq_sample_hist_bf16(None, p, p, 100, 1.0, 0.9, 1, p, 0.0, 0.0, 0, 0.0, p, 4, p, nb) == -2         # rep == 0
    assert L.vpq_sample_hist_bf16(None, None, p, 100, 1.0, 0.9, 1, p, 1.0, 0.0, 0, 0.0, p, 4, p, nb) == -1
    torch.cuda.synchronize()
