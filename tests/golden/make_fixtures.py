"""Writes tests/golden/*.npz: small known-answer cases for the w4g64 path.

    python -m tests.golden.make_fixtures

Inputs are the reference tests' own portable generators (refgen.py: the Knuth-hash case of
tests/unit-tests/metal-lm/quant-gemv.cc:215-253 and the LCG case of
tests/unit-tests/minimax-h3-blocks.cc:121-158), rounded to bf16 as those tests do.  Expected
outputs are computed HERE in numpy float64 from the layout and formulas alone (nibble i of
word j = q[n, 8j+i]; W = s*q + b), independently of the C oracle and of the HIP kernels, so
the same files pin both.  Nothing of the reference is imported or run.

Each file holds: w (uint32 [N,K/8]), scales/biases/x (bf16 bit patterns), K, N, M, and
  y_qmv  float64 [M,N]  x . (s*q+b)^T with the weight NOT rounded          (QMV semantics)
  y_qmm  float64 [M,N]  x . bf16_rne(fp32(s*q+b))^T                          (QMM semantics)
  w_deq  uint16  [N,K]  bf16_rne(fp32(s*q+b)) bit patterns                   (dense expansion)
and for the LoRA case A, B (bf16 bits), r, alpha, t (bf16 bits of bf16(alpha*bf16(x.A^T))) and
  y_lora float64 [M,N]  x . bf16(W)^T + t . B^T.
"""
import os

import numpy as np

from tests.golden import refgen
from vpipe_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))


def unpack(w, N, K):
    shifts = (np.arange(8, dtype=np.uint32) * np.uint32(4))[None, None, :]
    return ((w[:, :, None] >> shifts) & np.uint32(0xF)).reshape(N, K).astype(np.float32)


def expected(w, s_bits, b_bits, x_bits, K, N):
    q = unpack(w, N, K)
    s = np.repeat(synth.bf16_bits_to_f32(s_bits), 64, axis=1)
    b = np.repeat(synth.bf16_bits_to_f32(b_bits), 64, axis=1)
    x = synth.bf16_bits_to_f32(x_bits).astype(np.float64)
    w64 = s.astype(np.float64) * q.astype(np.float64) + b.astype(np.float64)
    w32 = (s * q + b).astype(np.float32)          # s*q is exact in fp32: one rounding, as an fma
    w_deq = synth.f32_to_bf16_bits(w32)
    wq = synth.bf16_bits_to_f32(w_deq).astype(np.float64)
    return x @ w64.T, x @ wq.T, w_deq


def knuth_case(N, K, M):
    c = refgen.knuth_qmv_case(N, K, group=64)
    w = c["packed"][:N].copy()
    s_bits = synth.f32_to_bf16_bits(c["scales"])
    b_bits = synth.f32_to_bf16_bits(c["biases"])
    rows = [c["x"][:K]]
    for m in range(1, M):
        rows.append(refgen.lcg_act(K, 100 + m) * np.float32(10.0))
    x_bits = synth.f32_to_bf16_bits(np.stack(rows).astype(np.float32))
    return w, s_bits, b_bits, x_bits


def lcg_case(N, K, M, seed):
    w, s0, b0 = refgen.lcg_qweight(N, K, seed)
    s_bits = synth.f32_to_bf16_bits(np.full((N, K // 64), s0, dtype=np.float32))
    b_bits = synth.f32_to_bf16_bits(np.full((N, K // 64), b0, dtype=np.float32))
    x_bits = synth.f32_to_bf16_bits(refgen.lcg_act(M * K, 21).reshape(M, K))
    return w, s_bits, b_bits, x_bits


def save(name, w, s_bits, b_bits, x_bits, K, N, M, **extra):
    y_qmv, y_qmm, w_deq = expected(w, s_bits, b_bits, x_bits, K, N)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), w=w, scales=s_bits, biases=b_bits, x=x_bits,
                        K=K, N=N, M=M, y_qmv=y_qmv, y_qmm=y_qmm, w_deq=w_deq, **extra)
    return y_qmm


def main():
    # K = 3840 is not a multiple of 512: the reference's tail case (quant-gemv.cc:215-222)
    save("knuth_n16_k3840_m1", *knuth_case(16, 3840, 1), 3840, 16, 1)
    save("knuth_n64_k1024_m2", *knuth_case(64, 1024, 2), 1024, 64, 2)
    # make_qw_/make_act_ (minimax-h3-blocks.cc:121-158): m = 7 rows in an 8-row tile, ragged N
    save("lcg_n64_k768_m7", *lcg_case(64, 768, 7, 0xBEEF), 768, 64, 7)
    save("lcg_n33_k128_m33", *lcg_case(33, 128, 33, 0x1234), 128, 33, 33)
    # runtime LoRA at the reference test's strength (minimax-h3-blocks.cc:1162-1296), reduced sizes
    N, K, M, r, alpha = 96, 512, 40, 64, 0.625
    w, s_bits, b_bits, x_bits = lcg_case(N, K, M, 0xC0DE)
    A = synth.f32_to_bf16_bits(refgen.lcg_act(r * K, 29).reshape(r, K))
    B = synth.f32_to_bf16_bits(refgen.lcg_act(N * r, 31).reshape(N, r))
    x = synth.bf16_bits_to_f32(x_bits).astype(np.float64)
    xa = (x @ synth.bf16_bits_to_f32(A).astype(np.float64).T).astype(np.float32)
    t0 = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(xa))
    t = synth.f32_to_bf16_bits((np.float32(alpha) * t0).astype(np.float32))
    _, y_qmm, _ = expected(w, s_bits, b_bits, x_bits, K, N)
    y_lora = y_qmm + synth.bf16_bits_to_f32(t).astype(np.float64) @ synth.bf16_bits_to_f32(B).astype(np.float64).T
    save("lcg_lora_n96_k512_m40_r64", w, s_bits, b_bits, x_bits, K, N, M, A=A, B=B, r=r, alpha=alpha, t=t, y_lora=y_lora)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
