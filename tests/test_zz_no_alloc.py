"""The entry point that allocates nothing (vpq_argmax_bf16_static: slab pairs in a static device array of the
library) against the workspace form of the same kernels, through the C ABI.  Runs last: the static array is
shared by every call of the process."""
import numpy as np
import pytest
import torch

from vpipe_amd import capi, synth

pytestmark = pytest.mark.gpu


def _rows(V, rows, seed):
    rng = np.random.default_rng(seed)
    vals = rng.integers(-40, 40, size=(rows, V)).astype(np.float32) / 2.0     # many equal maxima
    return synth.f32_to_bf16_bits(vals)


def test_static_scratch_argmax_equals_the_workspace_form(vpq, oracle, dev, D):
    # two calls in a row on one stream, the second smaller (fewer rows, fewer slabs): the stale pairs of the
    # first call must not be read
    assert vpq.load().vpq_init() == 0          # resolves the static array's address for this device
    for V, rows, seed in ((151936, 7, 1), (5000, 2, 2), (600001, 64, 3), (1, 1, 4)):
        bits = _rows(V, rows, seed)
        logits = D.bf16(bits, dev)
        want = vpq.argmax_bf16(logits, two_stage=True)
        out = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        got = vpq.argmax_bf16_static(logits, out)          # inputs and outputs exist: the call itself allocates nothing
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was allocated by the static entry point"
        assert torch.equal(got, want), (V, rows)
        assert np.array_equal(got.cpu().numpy(), oracle.argmax(bits)), (V, rows)


def test_static_scratch_argmax_under_graph_capture(vpq, oracle, dev, D):
    """The callers the entry point is for cannot allocate: recorded into a HIP graph (an allocation or a symbol
    lookup inside the call would fail the capture), replayed on fresh logits with eager work between the replays,
    every replay checked."""
    assert vpq.load().vpq_init() == 0
    V, rows = 151936, 5
    logits = D.bf16(_rows(V, rows, 20), dev)
    out = torch.full((rows,), -7, dtype=torch.int32, device=dev)
    vpq.argmax_bf16_static(logits, out)                    # (first call on this device done outside the capture)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        vpq.argmax_bf16_static(logits, out)
    for rep in range(4):
        bits = _rows(V, rows, 21 + rep)
        logits.copy_(D.bf16(bits, dev))
        out.fill_(-7)
        other = vpq.argmax_bf16(D.bf16(_rows(999, 3, 40 + rep), dev), two_stage=True)   # eager work of the same kernels
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), oracle.argmax(bits)), rep
        assert other.shape[0] == 3


def test_static_scratch_argmax_rejects_what_its_array_cannot_hold(vpq, dev, D):
    bits = _rows(64, capi.VPQ_ARGMAX_STATIC_MAX_ROWS + 1, 9)
    logits = D.bf16(bits, dev)
    out = torch.zeros((capi.VPQ_ARGMAX_STATIC_MAX_ROWS + 1,), dtype=torch.int32, device=dev)
    with pytest.raises(capi.VpqError) as e:
        vpq.argmax_bf16_static(logits, out)
    assert e.value.status == capi.VPQ_ERR_WORKSPACE
    assert "static scratch holds" in str(e.value)
