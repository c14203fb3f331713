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
    free_before = torch.cuda.mem_get_info()[0]
    for V, rows, seed in ((151936, 7, 1), (5000, 2, 2), (600001, 64, 3), (1, 1, 4)):
        bits = _rows(V, rows, seed)
        logits = D.bf16(bits, dev)
        want = vpq.argmax_bf16(logits, two_stage=True)
        out = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        got = vpq.argmax_bf16_static(logits, out)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (V, rows)
        assert np.array_equal(got.cpu().numpy(), oracle.argmax(bits)), (V, rows)
    assert torch.cuda.mem_get_info()[0] <= free_before + (64 << 20)   # (sanity: nothing large appeared)


def test_static_scratch_argmax_rejects_what_its_array_cannot_hold(vpq, dev, D):
    bits = _rows(64, capi.VPQ_ARGMAX_STATIC_MAX_ROWS + 1, 9)
    logits = D.bf16(bits, dev)
    out = torch.zeros((capi.VPQ_ARGMAX_STATIC_MAX_ROWS + 1,), dtype=torch.int32, device=dev)
    with pytest.raises(capi.VpqError) as e:
        vpq.argmax_bf16_static(logits, out)
    assert e.value.status == capi.VPQ_ERR_WORKSPACE
    assert "static scratch holds" in str(e.value)
