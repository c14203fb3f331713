"""Shared helpers of the GPU parity tests: tolerance checks and input staging.

Tolerances (written once, used by every GPU test):
  * dequantized weights: bit-exact.
  * fp32 result before the store vs the float64 oracle:
        max |d| / max(|ref|, 1e-2 * rms(ref))  <=  2e-3
    (relative error with a floor, since zero-mean weights put outputs near 0).
  * bf16 output: the bound above plus one bf16 step at |ref| (one rounding, and
    the fp32 and float64 sums may sit on either side of a rounding boundary);
    every element that is not tiny against the rms within one bf16 ulp of
    bf16_rne(oracle); at most 2% of elements differing from it at all; rel-L2
    against the float64 oracle <= 2e-3 on outputs of 256 elements or more (the
    noise of one bf16 store alone is ~1.6e-3 rms; smaller outputs add the 2^-8
    worst case of a single rounding).
"""
import numpy as np

from vpipe_amd import synth

F32_TOL = 2e-3
REL_L2_TOL = 2e-3


def floor_rel_err(got, ref64):
    ref64 = np.asarray(ref64, dtype=np.float64)
    rms = np.sqrt((ref64 ** 2).mean())
    denom = np.maximum(np.abs(ref64), 1e-2 * rms + 1e-30)
    return (np.abs(np.asarray(got, dtype=np.float64) - ref64) / denom).max()


def rel_l2(got, ref64):
    ref64 = np.asarray(ref64, dtype=np.float64)
    num = ((np.asarray(got, dtype=np.float64) - ref64) ** 2).sum()
    den = (ref64 ** 2).sum()
    return np.sqrt(num / den) if den > 0 else np.sqrt(num)


def bf16_ulp_distance(a_bits, b_bits):
    """Distance in units of bf16 steps on the ordered number line."""
    def key(x):
        x = np.asarray(x, dtype=np.uint16).astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def check_f32(got_f32, ref64, tol=F32_TOL):
    e = floor_rel_err(got_f32, ref64)
    assert e <= tol, "fp32 result off by %.3e (tol %.1e)" % (e, tol)
    return e


def bf16_ulp(v):
    """Spacing of bf16 numbers at magnitude |v| (8 significant bits)."""
    v = np.abs(np.asarray(v, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(v, 2.0 ** -126)))
    return 2.0 ** (e - 7)


def check_bf16(got_bits, ref64, ref_bits=None, mismatch_over_all=True):
    """bf16 output = (fp32 result within the floored 2e-3 of the oracle) rounded once:
    |got - ref| <= 2e-3 * max(|ref|, 1e-2 rms) + one bf16 step at |ref|.  Where the
    output is not tiny against the rms this is the same as `within one bf16 ulp of
    bf16(oracle)`; the mismatch rate and rel-L2 are bounded as well."""
    ref64 = np.asarray(ref64, dtype=np.float64)
    if ref_bits is None:
        ref_bits = synth.f32_to_bf16_bits(ref64.astype(np.float32))
    got = synth.bf16_bits_to_f32(got_bits).astype(np.float64)
    rms = np.sqrt((ref64 ** 2).mean())
    allowed = F32_TOL * np.maximum(np.abs(ref64), 1e-2 * rms) + bf16_ulp(ref64)
    worst = (np.abs(got - ref64) / allowed).max()
    assert worst <= 1.0, "bf16 output off by %.2f x the allowed error" % worst
    d = bf16_ulp_distance(got_bits, ref_bits)
    big = np.abs(ref64) >= 0.05 * rms
    assert d[big].max(initial=0) <= 1, "bf16 output differs by %d ulp on a non-tiny element" % d[big].max()
    # mismatch_over_all=False: the rate is taken over the non-tiny elements only (for outputs whose
    # near-zero values are fp32 noise by construction)
    counted = d if mismatch_over_all else d[big]
    mismatch = float((counted != 0).mean()) if counted.size else 0.0
    assert mismatch <= 0.02, "bf16 output differs from bf16(oracle) on %.2f%% of elements" % (100 * mismatch)
    r = rel_l2(got, ref64)
    # One bf16 store alone is worth ~1.6e-3 rms (up to 2^-8 on a single element), so below a few hundred
    # elements the sample's own rounding noise can pass 2e-3: there the single-rounding worst case is added
    # (the per-element bounds above are what binds on tiny outputs).
    tol = REL_L2_TOL if got.size >= 256 else REL_L2_TOL + 2.0 ** -8
    assert r <= tol, "rel-L2 %.3e" % r
    return mismatch, r


class Guarded:
    """An output buffer with sentinel-filled guard bands on both sides, to catch
    stores outside [M,N]."""

    def __init__(self, shape, dtype, dev, guard=4096):
        import torch
        self.n = int(np.prod(shape))
        self.guard = guard
        self.buf = torch.full((self.n + 2 * guard,), -7.0, dtype=dtype, device=dev)
        self.view = self.buf[guard:guard + self.n].view(shape)

    def assert_intact(self):
        import torch
        g = self.guard
        lo, hi = self.buf[:g].float(), self.buf[g + self.n:].float()
        assert torch.all(lo == -7.0).item() and torch.all(hi == -7.0).item(), "kernel wrote outside its output"
