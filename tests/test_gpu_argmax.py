"""GPU parity of the greedy argmax tail (index work: exact) against the CPU oracle, through the C ABI
and through the host layer's kernel names."""
import numpy as np
import pytest
import torch

from vpipe_amd import synth

pytestmark = pytest.mark.gpu

NAN, NINF = 0x7FC0, 0xFF80


def rows_of(V, rows, seed, ties):
    rng = np.random.default_rng(seed)
    if ties:
        vals = rng.integers(-30, 30, size=(rows, V)).astype(np.float32) / 2.0     # many equal maxima
    else:
        vals = rng.standard_normal(size=(rows, V)).astype(np.float32) * 5.0
    return synth.f32_to_bf16_bits(vals)


@pytest.mark.parametrize("two_stage", [False, True])
@pytest.mark.parametrize("ties", [False, True])
@pytest.mark.parametrize("V,rows", [(1, 1), (255, 2), (2048, 1), (2049, 3), (151936, 1), (262144, 2), (600001, 1)])
def test_argmax_matches_the_oracle(vpq, oracle, dev, D, V, rows, ties, two_stage):
    bits = rows_of(V, rows, 5000 + V + rows, ties)
    got = vpq.argmax_bf16(D.bf16(bits, dev), two_stage=two_stage).cpu().numpy()
    assert np.array_equal(got, oracle.argmax(bits))


@pytest.mark.parametrize("two_stage", [False, True])
def test_argmax_special_values_and_slab_boundaries(vpq, oracle, dev, D, two_stage):
    V = 10000
    base = synth.f32_to_bf16_bits(np.full((V,), -3.0, dtype=np.float32))
    rows = []
    for first in (0, 2047, 2048, 4095, 4096, 9999):      # equal maxima either side of the slab boundaries
        r = base.copy()
        r[first] = 0x4000
        r[min(first + 1, V - 1)] = 0x4000
        r[V - 1] = 0x4000
        rows.append(r)
    r = np.full((V,), NINF, dtype=np.uint16)             # nothing but -inf: the first entry
    rows.append(r)
    r = np.full((V,), NAN, dtype=np.uint16)              # nothing but NaN: 0
    rows.append(r)
    r = np.full((V,), NAN, dtype=np.uint16)              # a NaN never wins, -inf does
    r[7777] = NINF
    rows.append(r)
    r = base.copy()
    r[:5000] = NAN
    r[6000] = 0x7F80                                     # +inf
    r[6001] = 0x7F80
    rows.append(r)
    bits = np.stack(rows)
    got = vpq.argmax_bf16(D.bf16(bits, dev), two_stage=two_stage).cpu().numpy()
    want = oracle.argmax(bits)
    assert np.array_equal(got, want)
    assert list(want) == [0, 2047, 2048, 4095, 4096, 9999, 0, 0, 7777, 6000]


@pytest.mark.parametrize("parts", [1, 7, 256, 300, 1000])
def test_argmax_partial_and_combine_for_any_slab_count(vpq, oracle, dev, D, parts):
    V = 151936
    bits = rows_of(V, 1, 5100 + parts, True)
    L = vpq.load()
    logits = D.bf16(bits, dev)
    partials = torch.zeros((2 * parts,), dtype=torch.float32, device=dev)
    out = torch.full((1,), -5, dtype=torch.int32, device=dev)
    assert L.vpq_argmax_partial_bf16(None, logits.data_ptr(), partials.data_ptr(), V, parts) == 0
    assert L.vpq_argmax_combine(None, partials.data_ptr(), out.data_ptr(), parts) == 0
    torch.cuda.synchronize()
    assert int(out.item()) == int(oracle.argmax(bits)[0])


def test_argmax_rejects_bad_arguments(vpq, dev):
    L = vpq.load()
    t = torch.zeros(64, dtype=torch.int32, device=dev)
    p = t.data_ptr()
    assert L.vpq_argmax_bf16(None, None, p, 8, 1, None, 0) == -1
    assert L.vpq_argmax_bf16(None, p, p, 0, 1, None, 0) == -2
    assert L.vpq_argmax_bf16(None, p, p, 8, 0, None, 0) == -2
    assert L.vpq_argmax_bf16(None, p, p, 8, 1, p, 4) == L.vpq_argmax_bf16(None, p, p, 8, 1, p, 0) != 0    # workspace too small
    assert L.vpq_argmax_partial_bf16(None, p, p, 8, 0) == -2
    assert L.vpq_argmax_combine(None, p, p, 0) == -2
