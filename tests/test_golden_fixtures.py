"""The committed known-answer files (tests/golden/*.npz, written by tests/golden/make_fixtures.py
from the reference tests' generators with numpy-float64 expected outputs) against the CPU oracle
(CPU tests) and against the HIP path through the C ABI (GPU tests, no oracle involved)."""
import glob
import os

import numpy as np
import pytest

from tests import parity
from vpipe_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
IDS = [os.path.basename(f)[:-4] for f in FILES]


def load(path):
    z = np.load(path, allow_pickle=False)
    return {k: z[k] for k in z.files}


def test_fixtures_are_present():
    assert len(FILES) == 5, FILES


@pytest.mark.parametrize("path", FILES, ids=IDS)
def test_oracle_reproduces_fixture(oracle, path):
    c = load(path)
    K, N, M = int(c["K"]), int(c["N"]), int(c["M"])
    assert np.array_equal(oracle.dequant_bf16(c["w"], c["scales"], c["biases"], K, N), c["w_deq"])
    y64, yb = oracle.qmv(c["w"], c["scales"], c["biases"], c["x"], K, N, M)
    scale = np.abs(c["y_qmv"]).max()
    assert np.abs(y64 - c["y_qmv"]).max() <= 1e-12 * scale
    assert parity.bf16_ulp_distance(yb, synth.f32_to_bf16_bits(c["y_qmv"].astype(np.float32))).max() <= 1
    y64, yb = oracle.qmm(c["w"], c["scales"], c["biases"], c["x"], K, N, M)
    assert np.abs(y64 - c["y_qmm"]).max() <= 1e-12 * np.abs(c["y_qmm"]).max()
    if "A" in c:
        r, alpha = int(c["r"]), float(c["alpha"])
        t = oracle.lora_t(c["x"], c["A"], M, K, r, alpha)
        assert parity.bf16_ulp_distance(t, c["t"]).max() <= 1
        y64, _ = oracle.qmm(c["w"], c["scales"], c["biases"], c["x"], K, N, M, t=c["t"], B=c["B"], r=r)
        assert np.abs(y64 - c["y_lora"]).max() <= 1e-12 * np.abs(c["y_lora"]).max()


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=IDS)
def test_hip_path_reproduces_fixture(vpq, dev, D, path):
    import torch
    c = load(path)
    K, N, M = int(c["K"]), int(c["N"]), int(c["M"])
    wd, sd, bd, xd = D.u32(c["w"], dev), D.bf16(c["scales"], dev), D.bf16(c["biases"], dev), D.bf16(c["x"], dev)
    assert np.array_equal(D.bits(vpq.dequant_w4g64(wd, sd, bd, K, N)), c["w_deq"])
    if M <= 16:
        for variant in (0, 1):
            got = D.bits(vpq.qmv_w4g64(wd, sd, bd, xd, K, N, M, variant=variant))
            parity.check_bf16(got, c["y_qmv"])
    got = D.bits(vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M))
    parity.check_bf16(got, c["y_qmm"])
    if "A" in c:
        r, alpha = int(c["r"]), float(c["alpha"])
        t_ws = torch.zeros((M, r), dtype=torch.bfloat16, device=dev)
        got = D.bits(vpq.qmm_w4g64(wd, sd, bd, xd, K, N, M, lora_A=D.bf16(c["A"], dev), lora_B=D.bf16(c["B"], dev),
                                   r=r, alpha=alpha, t_ws=t_ws))
        assert parity.bf16_ulp_distance(D.bits(t_ws), c["t"]).max() <= 1
        parity.check_bf16(got, c["y_lora"])
