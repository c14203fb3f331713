"""GPU parity through the C++ host layer: the quantized-linear call sites are written in the
reference's encoder protocol (library/function by name, buffers in slots 0-4, K/N[/M] as
constants 5-7, dispatch with the reference's grid expressions, errors at the fence) -- the
form of llama3/metal-llama-model.cc:354-366, qwen3/metal-qwen-model.cc:3981-3991 and
minimax-h3/metal-minimax-h3-transformer.cc:1813-1828 -- and checked against the CPU oracle."""
import ctypes
import os

import numpy as np
import pytest
import torch

from tests import parity
from vpipe_amd import capi, synth

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


class Driver:
    def __init__(self):
        path = os.path.join(HERE, "host", "libhost_driver.so")
        assert os.path.exists(path), "tests/host/libhost_driver.so is not built (python -m vpipe_amd.build)"
        L = ctypes.CDLL(path)
        L.hd_open.restype = ctypes.c_void_p
        L.hd_close.argtypes = [ctypes.c_void_p]
        L.hd_set_function.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p]
        L.hd_set_buffer.argtypes = [ctypes.c_void_p, ctypes.c_uint, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
        L.hd_set_constant_i32.argtypes = [ctypes.c_void_p, ctypes.c_uint, ctypes.c_int]
        L.hd_dispatch.argtypes = [ctypes.c_void_p] + [ctypes.c_uint] * 6
        L.hd_scope_begin.argtypes = [ctypes.c_void_p]
        L.hd_scope_end.argtypes = [ctypes.c_void_p]
        L.hd_dispatch_count.argtypes = [ctypes.c_void_p]
        L.hd_dispatch_count.restype = ctypes.c_long
        L.hd_wait_ok.argtypes = [ctypes.c_void_p]
        L.hd_reason.argtypes = [ctypes.c_void_p]
        L.hd_reason.restype = ctypes.c_char_p
        L.hd_quant_linear.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_void_p]
        self.L = L
        self.h = L.hd_open()
        assert self.h, "CommandStream::create failed"

    def close(self):
        self.L.hd_close(self.h)
        self.h = None

    def set_function(self, lib, fn):
        return self.L.hd_set_function(self.h, lib.encode(), fn.encode())

    def set_buffer(self, index, t, byte_offset=0):
        if t is None:
            self.L.hd_set_buffer(self.h, index, None, 0, 0)
        else:
            self.L.hd_set_buffer(self.h, index, t.data_ptr(), t.numel() * t.element_size(), byte_offset)

    def set_constant(self, index, v):
        self.L.hd_set_constant_i32(self.h, index, int(v))

    def set_constant_f32(self, index, v):
        self.L.hd_set_constant_f32.argtypes = [ctypes.c_void_p, ctypes.c_uint, ctypes.c_float]
        self.L.hd_set_constant_f32(self.h, index, float(v))

    def dispatch(self, grid, tg):
        torch.cuda.synchronize()   # the tests stage their tensors on torch's stream
        self.L.hd_dispatch(self.h, *grid, *tg)

    def wait_ok(self):
        ok = self.L.hd_wait_ok(self.h)
        return bool(ok), self.L.hd_reason(self.h).decode()


@pytest.fixture()
def enc(vpq, dev):
    torch.cuda.synchronize()
    d = Driver()
    yield d
    d.close()


def stage(D, dev, w, s, b, x):
    return D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)


def encode_linear(enc, lib, fn, wd, sd, bd, xd, yd, K, N, M=None, grid=(32, 1, 1), tg=(32, 2, 1), x_off=0, y_off=0):
    assert enc.set_function(lib, fn) == 1
    enc.set_buffer(0, wd)
    enc.set_buffer(1, sd)
    enc.set_buffer(2, bd)
    enc.set_buffer(3, xd, x_off)
    enc.set_buffer(4, yd, y_off)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    if M is not None:
        enc.set_constant(7, M)
    enc.dispatch(grid, tg)


def test_qmv_call_site(enc, oracle, dev, D):
    # llama decode projection: dispatch {32, N/4, 1}, threadgroup {32, 2, 1}
    K, N = 1024, 512
    w, s, b = synth.make_weight(N, K, 3)
    x = synth.make_act(1, K, 4)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    yd = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w4g64", wd, sd, bd, xd, yd, K, N, grid=(32, N // 4, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    y64, yb = oracle.qmv(w, s, b, x, K, N, 1)
    parity.check_bf16(D.bits(yd), y64, yb)


def test_qmv_add_and_batch_call_sites(enc, oracle, dev, D):
    K, N, M = 512, 256, 4
    w, s, b = synth.make_weight(N, K, 5)
    x = synth.make_act(M, K, 6)
    res = synth.make_act(1, N, 7)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    # _add: slot 7 holds the residual; one x row
    yd = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    resd = D.bf16(res, dev)
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_w4g64_add") == 1
    for i, t in enumerate((wd, sd, bd, xd, yd)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.set_buffer(7, resd)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    # batch: slot 7 = m_total, rows tiled on grid.z
    yb_d = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_batch_w4g64", wd, sd, bd, xd, yb_d, K, N, M=M,
                  grid=(32, N // 4, (M + 1) // 2))
    ok, why = enc.wait_ok()
    assert ok, why
    _, yr = oracle.qmv(w, s, b, x[:1], K, N, 1, residual=res)   # the fp64 value is the one before the add
    assert parity.bf16_ulp_distance(D.bits(yd), yr).max() <= 1
    y64, yb = oracle.qmv(w, s, b, x, K, N, M)
    parity.check_bf16(D.bits(yb_d), y64, yb)


@pytest.mark.parametrize("lib,fn", [("affine_qmm_steel_bf16", "affine_qmm_steel_w4g64"),
                                    ("affine_qmm_steel_bf16", "affine_qmm_steel_w4g64_bm64"),
                                    ("affine_qmm_mma_bf16", "affine_qmm_mma_w4g64")])
def test_qmm_call_site_with_byte_offsets(enc, oracle, dev, D, lib, fn):
    # minimax-h3 qmm_dispatch_: x and y bound with byte offsets (element offset * 2)
    K, N, M = 256, 192, 70
    w, s, b = synth.make_weight(N, K, 8)
    x = synth.make_act(M, K, 9)
    wd, sd, bd, _ = stage(D, dev, w, s, b, x)
    xpad = torch.zeros((M + 3) * K, dtype=torch.bfloat16, device=dev)
    xpad[3 * K:] = D.bf16(x, dev).reshape(-1)
    ypad = torch.zeros((M + 2) * N, dtype=torch.bfloat16, device=dev)
    encode_linear(enc, lib, fn, wd, sd, bd, xpad, ypad, K, N, M=M, grid=(((N + 31) // 32) * 32, ((M + 63) // 64) * 2, 2),
                  tg=(32, 2, 2), x_off=3 * K * 2, y_off=2 * N * 2)
    ok, why = enc.wait_ok()
    assert ok, why
    y64, yb = oracle.qmm(w, s, b, x, K, N, M)
    got = D.bits(ypad)
    assert not got[:2 * N].any(), "rows before the offset were written"
    parity.check_bf16(got[2 * N:].reshape(M, N), y64, yb)


def test_dequant_call_site(enc, oracle, dev, D):
    K, N = 320, 48
    w, s, b = synth.make_weight(N, K, 10)
    wd, sd, bd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev)
    out = torch.zeros((N, K), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_dequant_bf16", "affine_dequant_w4g64") == 1
    for i, t in enumerate((wd, sd, bd, out)):
        enc.set_buffer(i, t)
    enc.set_constant(4, K)
    enc.set_constant(5, N)
    enc.dispatch((K // 8, N, 1), (64, 1, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert np.array_equal(D.bits(out), oracle.dequant_bf16(w, s, b, K, N))


def test_concurrent_scope_qkv(enc, oracle, dev, D):
    # unfused q|k|v inside a concurrent scope, then a dependent projection on the joined stream
    K, Nq, Nkv = 1024, 1024, 256
    ws = [synth.make_weight(n, K, 20 + i) for i, n in enumerate((Nq, Nkv, Nkv))]
    x = synth.make_act(1, K, 30)
    xd = D.bf16(x, dev)
    outs = [torch.zeros((1, n), dtype=torch.bfloat16, device=dev) for n in (Nq, Nkv, Nkv)]
    staged = [(D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev)) for (w, s, b) in ws]
    wo, so, bo = synth.make_weight(K, Nq, 40)
    wod, sod, bod = D.u32(wo, dev), D.bf16(so, dev), D.bf16(bo, dev)
    yo = torch.zeros((1, K), dtype=torch.bfloat16, device=dev)
    for rep in range(3):
        enc.L.hd_scope_begin(enc.h)
        for (wd, sd, bd), yd, n in zip(staged, outs, (Nq, Nkv, Nkv)):
            encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w4g64", wd, sd, bd, xd, yd, K, n, grid=(32, n // 4, 1))
        enc.L.hd_scope_end(enc.h)
        # depends on q: must see the finished q projection
        encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w4g64", wod, sod, bod, outs[0], yo, Nq, K, grid=(32, K // 4, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert enc.L.hd_dispatch_count(enc.h) == 12
    for (w, s, b), yd, n in zip(ws, outs, (Nq, Nkv, Nkv)):
        y64, yb = oracle.qmv(w, s, b, x, K, n, 1)
        parity.check_bf16(D.bits(yd), y64, yb)
    q_bits = D.bits(outs[0])
    y64, yb = oracle.qmv(wo, so, bo, q_bits, Nq, K, 1)
    parity.check_bf16(D.bits(yo), y64, yb)


def test_errors_surface_at_the_fence(enc, dev, D):
    K, N = 128, 64
    w, s, b = synth.make_weight(N, K, 11)
    x = synth.make_act(1, K, 12)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    yd = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    # an unknown function name gives an invalid function; dispatching it is an error at the fence
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_w3g64") == 0
    enc.dispatch((32, 1, 1), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert not ok and "function" in why
    # a missing slot (set_buffer of an empty buffer is a no-op) is reported, nothing is launched
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_w4g64") == 1
    enc.set_buffer(0, wd)
    enc.set_buffer(1, sd)
    enc.set_buffer(2, None)
    enc.set_buffer(3, xd)
    enc.set_buffer(4, yd)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert not ok and "affine_qmv_w4g64" in why
    assert not D.bits(yd).any()
    # a bad shape (K not a multiple of the group) is the library's own status text
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w4g64", wd, sd, bd, xd, yd, 100, N, grid=(32, N // 4, 1))
    ok, why = enc.wait_ok()
    assert not ok
    # the stream is usable again after the error was reported
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w4g64", wd, sd, bd, xd, yd, K, N, grid=(32, N // 4, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert D.bits(yd).any()


@pytest.mark.parametrize("M", [1, 8, 40, 100])
def test_quant_linear_forward_routes_by_m(enc, oracle, dev, D, M):
    K, N = 512, 320
    w, s, b = synth.make_weight(N, K, 13)
    x = synth.make_act(M, K, 14 + M)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    yd = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    enc.L.hd_quant_linear(enc.h, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), K, N, xd.data_ptr(), yd.data_ptr(), M,
                          None, None, 0, 0.0, None)
    ok, why = enc.wait_ok()
    assert ok, why
    y64, yb = (oracle.qmv if M <= 64 else oracle.qmm)(w, s, b, x, K, N, M)
    parity.check_bf16(D.bits(yd), y64, yb)


def test_quant_linear_forward_with_lora(enc, oracle, dev, D):
    K, N, M, r, strength = 512, 256, 48, 32, 0.625
    w, s, b = synth.make_weight(N, K, 15)
    x = synth.make_act(M, K, 16)
    A, B = synth.make_lora(N, K, r, 17, std=0.05)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    Ad, Bd = D.bf16(A, dev), D.bf16(B, dev)
    td = torch.zeros((M, r), dtype=torch.bfloat16, device=dev)
    yd = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    enc.L.hd_quant_linear(enc.h, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), K, N, xd.data_ptr(), yd.data_ptr(), M,
                          Ad.data_ptr(), Bd.data_ptr(), r, strength, td.data_ptr())
    ok, why = enc.wait_ok()
    assert ok, why
    t = oracle.lora_t(x, A, M, K, r, strength)
    y64, yb = oracle.qmm(w, s, b, x, K, N, M, t=t, B=B, r=r)
    parity.check_bf16(D.bits(yd), y64, yb)


@pytest.mark.parametrize("bits,group,fmt", [(8, 64, 2), (4, 32, 1), (8, 32, 3)])
def test_quant_linear_forward_with_lora_over_the_format_twins(vpq, enc, dev, D, bits, group, fmt):
    # `gemm_` with an adapter over a Linear of another width or group (minimax-h3/metal-minimax-h3-transformer.cc:
    # 2205-2259): the host takes the dequant-once route with the expansion in scratch of the stream; the bits of the
    # C ABI's call
    K, N, M, r, strength = 512, 136, 70, 24, 0.5
    if bits == 8:
        w, s, b = synth.make_weight8(N, K, 4300, group=group)
    else:
        w, s, b = synth.make_weight_g32(N, K, 4301)
    x = synth.make_act(M, K, 4302)
    A, B = synth.make_lora(N, K, r, 4303, std=0.05)
    wd, sd, bd, xd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)
    Ad, Bd = D.bf16(A, dev), D.bf16(B, dev)
    td = torch.zeros((M, r), dtype=torch.bfloat16, device=dev)
    yd = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    L = enc.L
    L.hd_quant_linear_fmt.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                      ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_void_p]
    L.hd_quant_linear_fmt(enc.h, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), bits, group, K, N, xd.data_ptr(), yd.data_ptr(), M,
                          Ad.data_ptr(), Bd.data_ptr(), r, strength, td.data_ptr())
    ok, why = enc.wait_ok()
    assert ok, why
    w_deq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    want = vpq.qmm_dense_route_lora(fmt, wd, sd, bd, xd, K, N, M, w_deq, Ad, Bd, r, strength)
    assert torch.equal(yd, want)
    assert yd.abs().sum() > 0


@pytest.mark.parametrize("group", [64, 32])
def test_eight_bit_functions_of_the_binary16_libraries(vpq, enc, dev, D, group):
    # the codec's call sites (generative-models/moss/metal-moss-codec.cc:181-183, 579-581): affine_dequant_w8g32 of
    # library "affine_dequant" (0:w 1:scales 2:biases 3:w_deq 4:K 5:N) and affine_qmm_steel_w8g32 of "affine_qmm_steel"
    # (the GEMM slots, 7 = M), and their group-64 twins: the C ABI's results, bit for bit
    K, N, M = 512, 72, 90
    rng = np.random.default_rng(4400 + group)
    w = rng.integers(0, 2**32, size=(N, K // 4), dtype=np.uint32)
    s = rng.uniform(0.0003, 0.0012, size=(N, K // group)).astype(np.float16)
    b = (-128.0 * s.astype(np.float32)).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    wd = torch.from_numpy(w.view(np.int32)).to(dev)
    sd, bd, xd = torch.from_numpy(s).to(dev), torch.from_numpy(b).to(dev), torch.from_numpy(x).to(dev)
    dq = torch.zeros((N, K), dtype=torch.float16, device=dev)
    y = torch.zeros((M, N), dtype=torch.float16, device=dev)
    assert enc.set_function("affine_dequant", "affine_dequant_w8g%d" % group) == 1
    for i, t in enumerate((wd, sd, bd, dq)):
        enc.set_buffer(i, t)
    enc.set_constant(4, K)
    enc.set_constant(5, N)
    enc.dispatch((K // 4, N, 1), (64, 1, 1))
    assert enc.set_function("affine_qmm_steel", "affine_qmm_steel_w8g%d" % group) == 1
    for i, t in enumerate((wd, sd, bd, xd, y)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.set_constant(7, M)
    enc.dispatch((N, M, 2), (32, 2, 2))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(dq, vpq.dequant_w8_f16(wd, sd, bd, K, N, group=group))
    w_deq = torch.empty((N, K), dtype=torch.float16, device=dev)
    assert torch.equal(y, vpq.qmm_dense_route_w8_f16(wd, sd, bd, xd, K, N, M, w_deq, group=group))
    assert dq.abs().sum() > 0 and y.abs().sum() > 0


def test_batched_gemv_names_of_every_tiling_and_format(vpq, enc, dev, D):
    # gpu-kernels/metal/quant/affine_qmv.metal:1674-2549, 2725-2745, 2854-2872, 3003-3026: the batched GEMVs (rows =
    # m_total in slot 7, grid {32, N/4, ceil(m_total / MAXM)}) in their tilings, gated forms and pack formats are the
    # C ABI's QMV over m_total rows, bit for bit
    K, N = 1024, 96
    w, s, b = synth.make_weight(N, K, 4500)
    w8, s8, b8 = synth.make_weight8(N, K, 4501)
    wg, sg, bg = synth.make_weight_g32(N, K, 4502)
    p4 = (D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev))
    p8 = (D.u32(w8, dev), D.bf16(s8, dev), D.bf16(b8, dev))
    pg = (D.u32(wg, dev), D.bf16(sg, dev), D.bf16(bg, dev))
    cases = [("affine_qmv_batch8_xh16_w4g64", p4, 8, 0), ("affine_qmv_batch8_tg4_w4g64", p4, 5, 0),
             ("affine_qmv_batch4_swiglu_w4g64", p4, 3, 1), ("affine_qmv_batch8_xp2_swiglu_w4g64", p4, 7, 1),
             ("affine_qmv_batch_geglu_w4g64", p4, 2, 2), ("affine_qmv_batch_w8g64", p8, 2, 0),
             ("affine_qmv_batch8_xd_w8g64", p8, 6, 0), ("affine_qmv_batch_w4g32", pg, 2, 0),
             ("affine_qmv_batch_geglu_w4g32", pg, 2, 2)]
    outs = []
    for name, pack, M, act in cases:
        x = D.bf16(synth.make_act(M, K, 4510 + M), dev)
        y = torch.zeros((M, N // 2 if act else N), dtype=torch.bfloat16, device=dev)
        assert enc.set_function("affine_qmv_bf16", name) == 1, name
        for i, t in enumerate(pack + (x, y)):
            enc.set_buffer(i, t)
        enc.set_constant(5, K)
        enc.set_constant(6, N)
        enc.set_constant(7, M)
        enc.dispatch((32, N // 4, (M + 1) // 2), (32, 2, 1))
        outs.append((name, pack, M, act, x, y))
    ok, why = enc.wait_ok()
    assert ok, why
    for name, pack, M, act, x, y in outs:
        if pack is p4:
            want = vpq.qmv_swiglu_w4g64(*pack, x, K, N, M, activation=act) if act else vpq.qmv_w4g64(*pack, x, K, N, M)
        elif pack is p8:
            want = vpq.qmv_w8g64(*pack, x, K, N, M)
        else:
            want = vpq.qmv_w4g32(*pack, x, K, N, M, activation=act)
        assert torch.equal(y, want), name
        assert y.abs().sum() > 0


@pytest.mark.parametrize("lib,name,bits,group", [("affine_dequant_bf16", "affine_quant_w4_g64", 4, 64),
                                                 ("affine_dequant", "affine_quant_w8_g32", 8, 32),
                                                 ("affine_dequant", "affine_quant_w4_g32", 4, 32),
                                                 ("affine_dequant_bf16", "affine_quant_w8_g64", 8, 64)])
def test_packer_function_names(vpq, enc, dev, D, lib, name, bits, group):
    # AffineQuantizer::quantize_linear's dispatch (generative-models/quantize/affine-quantizer.cc:52-84): 0:x 1:w
    # 2:scales 3:biases 4:K 5:N 6:clip, grid {K / group, N, 1}; the binary16 library takes a binary16 source
    K, N, clip = 512, 40, 0.9
    v = np.random.default_rng(4600 + bits + group).standard_normal((N, K)).astype(np.float32) * 0.05
    src = torch.from_numpy(v.astype(np.float16)).to(dev) if lib == "affine_dequant" else D.bf16(synth.f32_to_bf16_bits(v), dev)
    w = torch.zeros((N, K * bits // 32), dtype=torch.int32, device=dev)
    s = torch.zeros((N, K // group), dtype=torch.float16, device=dev)
    b = torch.zeros((N, K // group), dtype=torch.float16, device=dev)
    assert enc.set_function(lib, name) == 1
    for i, t in enumerate((src, w, s, b)):
        enc.set_buffer(i, t)
    enc.set_constant(4, K)
    enc.set_constant(5, N)
    enc.L.hd_set_constant_f32.argtypes = [ctypes.c_void_p, ctypes.c_uint, ctypes.c_float]
    enc.L.hd_set_constant_f32(enc.h, 6, clip)
    enc.dispatch((K // group, N, 1), (K // group, 1, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    want = vpq.quantize(src, K, N, bits=bits, group=group, clip=clip)
    assert torch.equal(w, want[0]) and torch.equal(s, want[1]) and torch.equal(b, want[2])
    assert w.abs().sum() > 0


def test_batched_gemv_names_of_the_binary16_library(vpq, enc, dev, D):
    # the half build's batched GEMVs (library "affine_qmv", rows = m_total in slot 7): the C ABI's binary16 QMV
    K, N = 1024, 64
    rng = np.random.default_rng(4700)
    w = rng.integers(0, 2**32, size=(N, K // 8), dtype=np.uint32)
    s = rng.uniform(0.005, 0.02, size=(N, K // 64)).astype(np.float16)
    b = (-8.0 * s.astype(np.float32)).astype(np.float16)
    wd = torch.from_numpy(w.view(np.int32)).to(dev)
    sd, bd = torch.from_numpy(s).to(dev), torch.from_numpy(b).to(dev)
    outs = []
    for name, M, act in (("affine_qmv_batch4_w4g64", 3, 0), ("affine_qmv_batch8_xp2_w4g64", 8, 0),
                         ("affine_qmv_batch_swiglu_w4g64", 2, 1), ("affine_qmv_batch_geglu_w4g64", 2, 2)):
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float16)).to(dev)
        y = torch.zeros((M, N // 2 if act else N), dtype=torch.float16, device=dev)
        assert enc.set_function("affine_qmv", name) == 1, name
        for i, t in enumerate((wd, sd, bd, x, y)):
            enc.set_buffer(i, t)
        enc.set_constant(5, K)
        enc.set_constant(6, N)
        enc.set_constant(7, M)
        enc.dispatch((32, N // 4, (M + 1) // 2), (32, 2, 1))
        outs.append((name, M, act, x, y))
    ok, why = enc.wait_ok()
    assert ok, why
    for name, M, act, x, y in outs:
        want = vpq.qmv_w4g64_f16(wd, sd, bd, x, K, N, M, activation=act) if act else vpq.qmv_w4g64_f16(wd, sd, bd, x, K, N, M)
        assert torch.equal(y, want), name
        assert y.abs().sum() > 0


def test_fused_qkv_call_site(enc, oracle, dev, D):
    # llama decode: one dispatch over the row-concatenated q|k|v pack, three output buffers
    # (gpu-kernels/metal/quant/affine_qmv.metal:405-516)
    K, rows = 1024, (512, 128, 128)
    N = sum(rows)
    w, s, b = synth.make_weight(N, K, 50)
    x = synth.make_act(1, K, 51)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    outs = [torch.zeros((1, r), dtype=torch.bfloat16, device=dev) for r in rows]
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_qkv_w4g64") == 1
    for i, t in enumerate((wd, sd, bd, xd, outs[0], outs[1], outs[2])):
        enc.set_buffer(i, t)
    enc.set_constant(7, K)
    for i, r in enumerate(rows):
        enc.set_constant(8 + i, r)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    y64, yb = oracle.qmv(w, s, b, x, K, N, 1)
    got = np.concatenate([D.bits(o) for o in outs], axis=1)
    parity.check_bf16(got, y64, yb)


def test_fused_mlp_call_sites(enc, oracle, dev, D):
    # llama decode (generative-models/llama3/metal-llama-model.cc:466-477): the interleaved gate|up
    # pack, dispatch {32, ffn/2, 1}; prefill (:634-650): the same pack through affine_qmm_swiglu
    # with M in slot 7; FLUX.2's strided twin adds out_stride / out_off in slots 8 and 9
    K, F = 1024, 192
    gate, up = synth.make_weight(F, K, 60), synth.make_weight(F, K, 61)
    w, s, b = (oracle.interleave(a, c) for a, c in zip(gate, up))
    x = synth.make_act(40, K, 62)
    wd, sd, bd, xd = stage(D, dev, w, s, b, x)
    y1 = torch.zeros((1, F), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_swiglu_w4g64", wd, sd, bd, xd, y1, K, 2 * F,
                  grid=(32, F // 2, 1))
    y40 = torch.zeros((40, F), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64", wd, sd, bd, xd, y40, K, 2 * F, M=40,
                  grid=(((2 * F + 31) // 32) * 32, ((40 + 31) // 32) * 2, 2), tg=(32, 2, 2))
    wide = torch.full((40, 2 * F + 8), 3.0, dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm64_rs") == 1
    for i, t in enumerate((wd, sd, bd, xd, wide)):
        enc.set_buffer(i, t)
    for i, v in enumerate((K, 2 * F, 40, 2 * F + 8, F)):
        enc.set_constant(5 + i, v)
    enc.dispatch((((2 * F + 31) // 32) * 32, ((40 + 63) // 64) * 2, 2), (32, 2, 2))
    ok, why = enc.wait_ok()
    assert ok, why
    o1, ob1 = oracle.swiglu(oracle.qmv(w, s, b, x[:1], K, 2 * F, 1)[0])
    parity.check_bf16(D.bits(y1), o1, ob1)
    o40, ob40 = oracle.swiglu(oracle.qmm(w, s, b, x, K, 2 * F, 40)[0])
    parity.check_bf16(D.bits(y40), o40, ob40)
    assert torch.equal(wide[:, F:2 * F], y40)
    assert (wide[:, :F] == 3.0).all().item() and (wide[:, 2 * F:] == 3.0).all().item()
    # Gemma's twin of the same call site: gelu_tanh(gate) * up
    yg = torch.zeros((1, F), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_geglu_w4g64", wd, sd, bd, xd, yg, K, 2 * F, grid=(32, F // 2, 1))
    yg40 = torch.zeros((40, F), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmm_steel_bf16", "affine_qmm_geglu_w4g64", wd, sd, bd, xd, yg40, K, 2 * F, M=40,
                  grid=(((2 * F + 31) // 32) * 32, ((40 + 31) // 32) * 2, 2), tg=(32, 2, 2))
    ok, why = enc.wait_ok()
    assert ok, why
    g1, gb1 = oracle.geglu(oracle.qmv(w, s, b, x[:1], K, 2 * F, 1)[0])
    parity.check_bf16(D.bits(yg), g1, gb1, mismatch_over_all=False)
    g40, gb40 = oracle.geglu(oracle.qmm(w, s, b, x, K, 2 * F, 40)[0])
    parity.check_bf16(D.bits(yg40), g40, gb40, mismatch_over_all=False)


@pytest.mark.parametrize("M", [1, 40])
def test_quantize_write_read_load_run(enc, oracle, dev, D, tmp_path, M):
    # the producer and the consumer of the on-disk pack: a bf16 weight is quantized on the device and
    # written as `<prefix>.weight/.scales/.biases` (U32 / F16 / F16), the directory is opened again,
    # the Linear is loaded (scales and zero points converted F16 -> bf16 on the device, once) and run
    import safetensors.numpy as stnp
    L = enc.L
    L.hw_open.restype = ctypes.c_void_p
    L.hw_open.argtypes = [ctypes.c_char_p, ctypes.c_ulonglong]
    L.hw_close.argtypes = [ctypes.c_void_p]
    L.hr_open.restype = ctypes.c_void_p
    L.hr_open.argtypes = [ctypes.c_char_p, ctypes.c_int]
    L.hr_close.argtypes = [ctypes.c_void_p]
    L.hr_why.restype = ctypes.c_char_p
    L.hd_quantize_and_add.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_float]
    L.hd_load_and_run.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_void_p,
                                  ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int)]
    K, N = 1024, 96
    rng = np.random.default_rng(70 + M)
    src_bits = synth.f32_to_bf16_bits((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    src = D.bf16(src_bits, dev)
    x = synth.make_act(M, K, 71)
    xd = D.bf16(x, dev)
    torch.cuda.synchronize()
    w = L.hw_open(str(tmp_path).encode(), 1 << 30)
    prefix = b"model.layers.0.mlp.down_proj"
    assert L.hd_quantize_and_add(enc.h, w, prefix, src.data_ptr(), K, N, 1.0) == 1, L.hr_why()
    assert L.hw_close(w) == 1
    # what is on disk is the oracle's packer output, bit for bit, readable by the format's own library
    codes, s16, b16 = oracle.quantize(synth.bf16_bits_to_f32(src_bits), K, N)
    disk = stnp.load_file(str(tmp_path / "model-00001-of-00001.safetensors"))
    assert np.array_equal(disk[prefix.decode() + ".weight"], codes)
    assert np.array_equal(disk[prefix.decode() + ".scales"].view(np.uint16), s16)
    assert np.array_equal(disk[prefix.decode() + ".biases"].view(np.uint16), b16)
    r = L.hr_open(str(tmp_path).encode(), 1)
    assert r, L.hr_why()
    yd = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    kn = (ctypes.c_int * 2)()
    assert L.hd_load_and_run(enc.h, r, prefix, 0, xd.data_ptr(), yd.data_ptr(), M, kn) == 1, L.hr_why()
    assert tuple(kn) == (K, N)
    assert L.hd_load_and_run(enc.h, r, b"model.layers.1.mlp.down_proj", 0, xd.data_ptr(), yd.data_ptr(), M, kn) == 0
    assert L.hd_load_and_run(enc.h, r, prefix, 2048, xd.data_ptr(), yd.data_ptr(), M, kn) == 0    # a 2-bit reading
    L.hr_close(r)
    sb, bb = oracle.f16_to_bf16(s16), oracle.f16_to_bf16(b16)
    y64, yb = (oracle.qmv if M <= 64 else oracle.qmm)(codes, sb, bb, x, K, N, M)
    parity.check_bf16(D.bits(yd), y64, yb)


def test_embedding_gather_call_site(enc, oracle, dev, D):
    # llama decode (generative-models/llama3/metal-llama-model.cc:82): slots 0:ids 1:w 2:scales 3:biases
    # 4:out 5:H, grid (H, T, 1); the table is the (tied) lm_head pack
    vocab, H, T = 500, 1024, 6
    w, s, b = synth.make_weight(vocab, H, 80)
    ids = np.array([3, 499, 0, 77, 77, 250], dtype=np.int32)
    idd = torch.from_numpy(ids).to(dev)
    wd, sd, bd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev)
    out = torch.zeros((T, H), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("llm_elementwise_bf16", "dequant_embed_gather_f16") == 1
    for i, t in enumerate((idd, wd, sd, bd, out)):
        enc.set_buffer(i, t)
    enc.set_constant(5, H)
    enc.dispatch((H, T, 1), (256, 1, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert np.array_equal(D.bits(out), oracle.embed_gather(ids, w, s, b, H, vocab))



def test_moe_grouped_expert_call_sites(vpq, enc, oracle, dev, D):
    # Qwen MoE block at prefill, expert-sorted (generative-models/qwen3/metal-qwen-model.cc:4239-4264):
    # gate|up + SwiGLU over the gathered hidden rows -> gact[npad, I] (slots 0..4, 5:H 6:2*I 7:npad
    # 8:tile2e 9:srow), then down -> part[np, H] scattered to pair order (5:I 6:H 7:npad 8:tile2e 9:sdst)
    H, I, E, top_k, T = 512, 128, 5, 2, 70
    gu = [synth.make_weight(2 * I, H, 1900 + e) for e in range(E)]
    dn = [synth.make_weight(H, I, 1950 + e) for e in range(E)]
    guw, gus, gub = (np.stack([p[i] for p in gu]) for i in range(3))
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(T, H, 1990)
    eid = np.random.default_rng(1991).integers(0, E, size=T * top_k, dtype=np.int32)
    npair = eid.size
    B = vpq.grouped_block_rows()
    t2e_d, srow_d, sdst_d, _ = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E)
    t2e, srow, sdst = (o.cpu().numpy() for o in (t2e_d, srow_d, sdst_d))
    npad = srow.size
    gact = torch.zeros((npad, I), dtype=torch.bfloat16, device=dev)
    part = torch.zeros((npair, H), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()               # the encoder's stream is not ordered after torch's fills
    assert enc.set_function("affine_qmm_steel_bf16", "affine_qmm_grouped_swiglu_w4g64") == 1
    # staged tensors stay alive until the stream has run: a freed one may be handed to the next upload
    gu_d = (D.u32(guw, dev), D.bf16(gus, dev), D.bf16(gub, dev), D.bf16(x, dev), gact)
    for i, t in enumerate(gu_d):
        enc.set_buffer(i, t)
    enc.set_constant(5, H)
    enc.set_constant(6, 2 * I)
    enc.set_constant(7, npad)
    enc.set_buffer(8, t2e_d)
    enc.set_buffer(9, srow_d)
    enc.dispatch((((2 * I + 31) // 32) * 32, ((npad + 31) // 32) * 2, 2), (32, 2, 2))
    assert enc.set_function("affine_qmm_steel_bf16", "affine_qmm_grouped_w4g64") == 1
    dn_d = (D.u32(dw, dev), D.bf16(ds, dev), D.bf16(db, dev), gact, part)
    for i, t in enumerate(dn_d):
        enc.set_buffer(i, t)
    enc.set_constant(5, I)
    enc.set_constant(6, H)
    enc.set_constant(7, npad)
    enc.set_buffer(8, t2e_d)
    enc.set_buffer(9, sdst_d)
    enc.dispatch((((H + 31) // 32) * 32, ((npad + 31) // 32) * 2, 2), (32, 2, 2))
    ok, why = enc.wait_ok()
    assert ok, why
    gact_bits = D.bits(gact)
    y64, _ = oracle.qmm_grouped(guw, gus, gub, x, H, 2 * I, B, t2e, srow=srow)
    a64, ab = oracle.swiglu(y64)
    live = srow >= 0
    parity.check_bf16(gact_bits[live], a64[live], ab[live])
    assert not gact_bits[~live].any()
    # the down projection reads the activation the device produced
    d64, dbits = oracle.qmm_grouped(dw, ds, db, gact_bits, I, H, B, t2e, sdst=sdst, rows_y=npair)
    parity.check_bf16(D.bits(part), d64, dbits)


def test_moe_sorted_gemv_call_sites(vpq, enc, oracle, dev, D):
    # a few rows per expert: tiles of two sorted slots (gpu-kernels/metal/quant/affine_qmv.metal:2682-2708; slots 0..4,
    # 5:K 6:N 7:srow 8:tile2e, one tile per grid.z): gate|up + SwiGLU over the gathered hidden rows -> gact[npad, I],
    # then down over gact in slot order -> part[npad, H]
    H, I, E, top_k, T = 512, 128, 7, 2, 6
    gu = [synth.make_weight(2 * I, H, 2900 + e) for e in range(E)]
    dn = [synth.make_weight(H, I, 2950 + e) for e in range(E)]
    guw, gus, gub = (np.stack([p[i] for p in gu]) for i in range(3))
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(T, H, 2990)
    eid = np.random.default_rng(2991).integers(0, E, size=T * top_k, dtype=np.int32)
    B = capi.VPQ_QMV_GROUPED_SLOTS
    t2e_d, srow_d, _, _ = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E, block_rows=B)
    t2e, srow = t2e_d.cpu().numpy(), srow_d.cpu().numpy()
    npad = srow.size
    gact = torch.zeros((npad, I), dtype=torch.bfloat16, device=dev)
    part = torch.zeros((npad, H), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()               # the encoder's stream is not ordered after torch's fills
    assert enc.set_function("affine_qmv_bf16", "affine_grouped_swiglu_w4g64") == 1
    gu_d = (D.u32(guw, dev), D.bf16(gus, dev), D.bf16(gub, dev), D.bf16(x, dev), gact)
    for i, t in enumerate(gu_d):
        enc.set_buffer(i, t)
    enc.set_constant(5, H)
    enc.set_constant(6, 2 * I)
    enc.set_buffer(7, srow_d)
    enc.set_buffer(8, t2e_d)
    enc.dispatch((32, 2 * ((2 * I + 7) // 8), npad // B), (32, 2, 1))
    assert enc.set_function("affine_qmv_bf16", "affine_grouped_down_w4g64") == 1
    dn_d = (D.u32(dw, dev), D.bf16(ds, dev), D.bf16(db, dev), gact, part)
    for i, t in enumerate(dn_d):
        enc.set_buffer(i, t)
    enc.set_constant(5, I)
    enc.set_constant(6, H)
    enc.set_buffer(7, srow_d)
    enc.set_buffer(8, t2e_d)
    enc.dispatch((32, 2 * ((H + 7) // 8), npad // B), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    live = np.nonzero(srow >= 0)[0]
    gact_bits = D.bits(gact)
    y64 = np.concatenate([oracle.qmv(guw[t2e[s // B]], gus[t2e[s // B]], gub[t2e[s // B]], x[srow[s]:srow[s] + 1], H, 2 * I, 1)[0]
                          for s in live])
    a64, ab = oracle.swiglu(y64)
    parity.check_bf16(gact_bits[live], a64, ab)
    assert not gact_bits[srow < 0].any()
    # the down projection reads the activation the device produced
    pairs = [oracle.qmv(dw[t2e[s // B]], ds[t2e[s // B]], db[t2e[s // B]], gact_bits[s:s + 1], I, H, 1) for s in live]
    parity.check_bf16(D.bits(part)[live], np.concatenate([p[0] for p in pairs]), np.concatenate([p[1] for p in pairs]))
    assert not D.bits(part)[srow < 0].any()


def test_moe_sorted_gemv_w8_call_sites(vpq, enc, dev, D):
    # the 8-bit twins under their function names (affine_qmv.metal:2718-2719): same slots as the 4-bit functions
    H, I, E, top_k, T = 256, 64, 5, 2, 5
    gu = [synth.make_weight8(2 * I, H, 2800 + e) for e in range(E)]
    dn = [synth.make_weight8(H, I, 2850 + e) for e in range(E)]
    gu_d = tuple(f(np.stack([p[i] for p in gu]), dev) for i, f in enumerate((D.u32, D.bf16, D.bf16)))
    dn_d = tuple(f(np.stack([p[i] for p in dn]), dev) for i, f in enumerate((D.u32, D.bf16, D.bf16)))
    xd = D.bf16(synth.make_act(T, H, 2890), dev)
    eid = np.random.default_rng(2891).integers(0, E, size=T * top_k, dtype=np.int32)
    B = capi.VPQ_QMV_GROUPED_SLOTS
    t2e_d, srow_d, _, _ = vpq.moe_sort_pairs(torch.from_numpy(eid).to(dev), top_k, E, block_rows=B)
    npad = srow_d.numel()
    gact = torch.zeros((npad, I), dtype=torch.bfloat16, device=dev)
    part = torch.zeros((npad, H), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    assert enc.set_function("affine_qmv_bf16", "affine_grouped_swiglu_w8g64") == 1
    for i, t in enumerate(gu_d + (xd, gact)):
        enc.set_buffer(i, t)
    enc.set_constant(5, H)
    enc.set_constant(6, 2 * I)
    enc.set_buffer(7, srow_d)
    enc.set_buffer(8, t2e_d)
    enc.dispatch((32, 2 * ((2 * I + 7) // 8), npad // B), (32, 2, 1))
    assert enc.set_function("affine_qmv_bf16", "affine_grouped_down_w8g64") == 1
    for i, t in enumerate(dn_d + (gact, part)):
        enc.set_buffer(i, t)
    enc.set_constant(5, I)
    enc.set_constant(6, H)
    enc.set_buffer(7, srow_d)
    enc.set_buffer(8, t2e_d)
    enc.dispatch((32, 2 * ((H + 7) // 8), npad // B), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    want_act = torch.zeros_like(gact)
    vpq.qmv_grouped_gated_w8g64(*gu_d, xd, H, 2 * I, t2e_d, srow_d, E, out=want_act)
    want_part = torch.zeros_like(part)
    vpq.qmv_grouped_down_w8g64(*dn_d, want_act, I, H, t2e_d, srow_d, E, out=want_part)
    assert torch.equal(gact, want_act) and torch.equal(part, want_part)
    assert gact.abs().sum() > 0 and part.abs().sum() > 0


def test_moe_gathered_expert_call_sites(enc, oracle, dev, D):
    # Qwen MoE block, pair-batched (generative-models/qwen3/metal-qwen-model.cc:4190-4206):
    # gathered gate|up + SwiGLU -> act[np, I] (slots 0..4, 5:H 6:2*I 7:eid 8:top_k, grid {32, I/2, np}),
    # then gathered down -> part[np, H] (5:I 6:H 7:eid, grid {32, H/4, np}); tg {32, 2, 1}
    H, I, E, top_k, M = 1024, 128, 6, 3, 2
    npair = M * top_k
    gu = [synth.make_weight(2 * I, H, 900 + e) for e in range(E)]
    dn = [synth.make_weight(H, I, 950 + e) for e in range(E)]
    guw, gus, gub = (np.stack([p[i] for p in gu]) for i in range(3))
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(M, H, 990)
    eid = np.array([4, 0, 5, 1, 4, 2], dtype=np.int32)
    eidd = torch.from_numpy(eid).to(dev)
    act = torch.zeros((npair, I), dtype=torch.bfloat16, device=dev)
    part = torch.zeros((npair, H), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_qmv_bf16", "affine_gather_qmv_swiglu_w4g64") == 1
    gu_d = (D.u32(guw, dev), D.bf16(gus, dev), D.bf16(gub, dev), D.bf16(x, dev), act)   # kept alive until the stream has run
    for i, t in enumerate(gu_d):
        enc.set_buffer(i, t)
    enc.set_constant(5, H)
    enc.set_constant(6, 2 * I)
    enc.set_buffer(7, eidd)
    enc.set_constant(8, top_k)
    enc.dispatch((32, I // 2, npair), (32, 2, 1))
    assert enc.set_function("affine_qmv_bf16", "affine_gather_down_qmv_w4g64") == 1
    dn_d = (D.u32(dw, dev), D.bf16(ds, dev), D.bf16(db, dev), act, part)
    for i, t in enumerate(dn_d):
        enc.set_buffer(i, t)
    enc.set_constant(5, I)
    enc.set_constant(6, H)
    enc.set_buffer(7, eidd)
    enc.dispatch((32, H // 4, npair), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    act_bits = D.bits(act)
    a64 = np.empty((npair, I))
    ab = np.empty((npair, I), dtype=np.uint16)
    p64 = np.empty((npair, H))
    pb = np.empty((npair, H), dtype=np.uint16)
    for p in range(npair):
        e, t = int(eid[p]), p // top_k
        y64, _ = oracle.qmv(guw[e], gus[e], gub[e], x[t:t + 1], H, 2 * I, 1)
        o64, ob = oracle.swiglu(y64)
        a64[p], ab[p] = o64[0], ob[0]
        # the down projection reads the activation the device produced
        d64, dbits = oracle.qmv(dw[e], ds[e], db[e], act_bits[p:p + 1], I, H, 1)
        p64[p], pb[p] = d64[0], dbits[0]
    parity.check_bf16(act_bits, a64, ab)
    parity.check_bf16(D.bits(part), p64, pb)


def test_argmax_call_sites_of_the_host_layer(enc, oracle, dev, D):
    # the pipelined decode loop's tail (generative-models: argmax_partial_f16 + argmax_combine_f16 over the
    # lm_head's logits, or the single-threadgroup argmax_f16); grids as the reference dispatches them
    V, M = 151936, 64
    bits = synth.f32_to_bf16_bits(np.random.default_rng(5200).integers(-30, 30, size=(1, V)).astype(np.float32) / 2.0)
    logits = D.bf16(bits, dev)
    want = int(oracle.argmax(bits)[0])
    out = torch.full((2,), -1, dtype=torch.int32, device=dev)
    partials = torch.zeros((2 * M,), dtype=torch.float32, device=dev)
    assert enc.set_function("llm_elementwise_bf16", "argmax_f16") == 1
    enc.set_buffer(0, logits)
    enc.set_buffer(1, out)
    enc.set_constant(2, V)
    enc.dispatch((256, 1, 1), (256, 1, 1))
    assert enc.set_function("llm_elementwise_bf16", "argmax_partial_f16") == 1
    enc.set_buffer(0, logits)
    enc.set_buffer(1, partials)
    enc.set_constant(2, V)
    enc.set_constant(3, M)
    enc.dispatch((256 * M, 1, 1), (256, 1, 1))
    assert enc.set_function("llm_elementwise_bf16", "argmax_combine_f16") == 1
    enc.set_buffer(0, partials)
    enc.set_buffer(1, out, 4)
    enc.set_constant(2, M)
    enc.dispatch((256, 1, 1), (256, 1, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert out.cpu().tolist() == [want, want]


def test_sampler_call_site_of_the_host_layer(enc, oracle, dev, D):
    # llm::Sampler on the device (gpu-kernels/metal/ops/llm_elementwise.metal:3116-3130): one threadgroup, thirteen slots
    V = 6000
    bits = synth.f32_to_bf16_bits((np.random.default_rng(2300).standard_normal(V) * 3).astype(np.float32))
    seen = np.zeros(V, dtype=np.uint8)
    seen[::7] = 1
    want, ws_want, seen_want = oracle.sample_topp(bits, seen, 0.8, 0.9, 4242, n_iter=20, rep=1.3, pres=0.2, top_k=64, min_p=0.01)
    ld, out = D.bf16(bits, dev), torch.zeros((1,), dtype=torch.int32, device=dev)
    ws = torch.zeros((V,), dtype=torch.bfloat16, device=dev)
    seen_d = torch.from_numpy(seen.copy()).to(dev)
    torch.cuda.synchronize()
    assert enc.set_function("llm_elementwise_bf16", "sample_topp_f16") == 1
    enc.set_buffer(0, ld)
    enc.set_buffer(1, out)
    enc.set_constant(2, V)
    enc.set_constant_f32(3, 0.8)
    enc.set_constant_f32(4, 0.9)
    enc.set_constant(5, 4242)
    enc.set_buffer(6, ws)
    enc.set_constant(7, 20)
    enc.set_constant_f32(8, 1.3)
    enc.set_constant_f32(9, 0.2)
    enc.set_constant(10, 64)
    enc.set_constant_f32(11, 0.01)
    enc.set_buffer(12, seen_d)
    enc.dispatch((1, 1, 1), (256, 1, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert int(out.cpu()[0]) == want
    assert np.array_equal(D.bits(ws), ws_want) and np.array_equal(seen_d.cpu().numpy(), seen_want)


def test_eight_bit_and_group32_function_names(enc, oracle, dev, D):
    # the twins keep the slot layout of the 4-bit group-64 functions; the Q4_0 names ignore slot 2
    K, N = 1024, 96
    x = synth.make_act(1, K, 1200)
    xd = D.bf16(x, dev)
    res = synth.make_act(1, N, 1201)

    w8, s8, b8 = synth.make_weight8(N, K, 1202)
    y8 = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w8g64", D.u32(w8, dev), D.bf16(s8, dev), D.bf16(b8, dev), xd, y8,
                  K, N, grid=(32, N // 4, 1))
    wq, sq, bq = synth.make_weight_g32(N, K, 1203, q40=True)
    wqd, sqd, bqd = D.u32(wq, dev), D.bf16(sq, dev), D.bf16(bq, dev)
    ya = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    yq = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    yr = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    junk = torch.zeros((4,), dtype=torch.bfloat16, device=dev)          # slot 2 of a Q4_0 call: "pass anything"
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w4g32", wqd, sqd, bqd, xd, ya, K, N, grid=(32, N // 4, 1))
    encode_linear(enc, "affine_qmv_bf16", "affine_qmv_w4g32_q40", wqd, sqd, junk, xd, yq, K, N, grid=(32, N // 4, 1))
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_w4g32_add_q40") == 1
    for i, t in enumerate((wqd, sqd, junk, xd, yr)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.set_buffer(7, D.bf16(res, dev))
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    dense = torch.zeros((N, K), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_dequant_bf16", "affine_dequant_w4g32") == 1
    for i, t in enumerate((wqd, sqd, bqd, dense)):
        enc.set_buffer(i, t)
    enc.set_constant(4, K)
    enc.set_constant(5, N)
    enc.dispatch((K // 8, N, 1), (64, 1, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    y64, yb = oracle.matmul8(w8, s8, b8, x, K, N, 1, rounded=False)
    parity.check_bf16(D.bits(y8), y64, yb)
    y64, yb = oracle.qmv_g32(wq, sq, None, x, K, N, 1, scale_only=True)
    parity.check_bf16(D.bits(yq), y64, yb)
    assert torch.equal(ya, yq)
    want = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(D.bits(yq)) + synth.bf16_bits_to_f32(res))
    assert np.array_equal(D.bits(yr), want)
    assert np.array_equal(D.bits(dense), oracle.dequant_g32_bf16(wq, sq, bq, K, N))


def test_eight_bit_gated_and_gathered_function_names(vpq, enc, dev, D):
    # affine_qmv_swiglu_w8g64 / affine_qmv_geglu_w8g64 (slots 0..6, rows from grid.x) and the 8-bit MoE gathers
    # (slot 7 = pair_eid, 8 = top_k, pairs = grid.z): the encoder's results are the C ABI's, bit for bit
    K, inner, H, E, top_k, M = 512, 24, 72, 4, 2, 2
    packs = []
    for e in range(E):
        g, u = synth.make_weight8(inner, K, 3000 + 2 * e), synth.make_weight8(inner, K, 3001 + 2 * e)
        packs.append(tuple(np.stack([a, b], axis=1).reshape((2 * inner,) + a.shape[1:]) for a, b in zip(g, u)))
    guw, gus, gub = (np.stack([p[i] for p in packs]) for i in range(3))
    dn = [synth.make_weight8(H, 64, 3100 + e) for e in range(E)]
    dw, ds, db = (np.stack([p[i] for p in dn]) for i in range(3))
    x = synth.make_act(M, K, 3200)
    xs = synth.make_act(M * top_k, 64, 3201)
    eid = torch.tensor([3, 0, 1, 3], dtype=torch.int32, device=dev)
    gu_d = (D.u32(guw, dev), D.bf16(gus, dev), D.bf16(gub, dev), D.bf16(x, dev))
    dn_d = (D.u32(dw, dev), D.bf16(ds, dev), D.bf16(db, dev), D.bf16(xs, dev))
    y_sw = torch.zeros((M, inner), dtype=torch.bfloat16, device=dev)
    y_ge = torch.zeros((M, inner), dtype=torch.bfloat16, device=dev)
    act = torch.zeros((M * top_k, inner), dtype=torch.bfloat16, device=dev)
    part = torch.zeros((M * top_k, H), dtype=torch.bfloat16, device=dev)
    for name, y in (("affine_qmv_swiglu_w8g64", y_sw), ("affine_qmv_geglu_w8g64", y_ge)):
        assert enc.set_function("affine_qmv_bf16", name) == 1
        for i, t in enumerate((gu_d[0][1], gu_d[1][1], gu_d[2][1], gu_d[3], y)):      # expert 1's slab as a plain pack
            enc.set_buffer(i, t)
        enc.set_constant(5, K)
        enc.set_constant(6, 2 * inner)
        enc.dispatch((32 * M, inner // 2, 1), (32, 2, 1))
    assert enc.set_function("affine_qmv_bf16", "affine_gather_qmv_swiglu_w8g64") == 1
    for i, t in enumerate(gu_d + (act,)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, 2 * inner)
    enc.set_buffer(7, eid)
    enc.set_constant(8, top_k)
    enc.dispatch((32, inner // 2, M * top_k), (32, 2, 1))
    assert enc.set_function("affine_qmv_bf16", "affine_gather_down_qmv_w8g64") == 1
    for i, t in enumerate(dn_d + (part,)):
        enc.set_buffer(i, t)
    enc.set_constant(5, 64)
    enc.set_constant(6, H)
    enc.set_buffer(7, eid)
    enc.dispatch((32, H // 4, M * top_k), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(y_sw, vpq.qmv_gated_w8g64(gu_d[0][1], gu_d[1][1], gu_d[2][1], gu_d[3], K, 2 * inner, M, activation=1))
    assert torch.equal(y_ge, vpq.qmv_gated_w8g64(gu_d[0][1], gu_d[1][1], gu_d[2][1], gu_d[3], K, 2 * inner, M, activation=2))
    assert torch.equal(act, vpq.gather_qmv_gated_w8g64(*gu_d, K, 2 * inner, eid, top_k, E))
    assert torch.equal(part, vpq.gather_down_qmv_w8g64(*dn_d, 64, H, eid, E))
    assert y_sw.abs().sum() > 0 and not torch.equal(y_sw, y_ge)


def test_binary16_library_names(vpq, enc, oracle, dev, D):
    # the metallibs without the `_bf16` suffix hold the IEEE binary16 build of the same function names
    from tests.test_oracle_pins import f16_pack
    K, N = 512, 48
    w, s, b = f16_pack(N, K, 77)
    x = np.random.default_rng(78).standard_normal((1, K)).astype(np.float16).view(np.uint16)
    as16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(dev).view(torch.float16)
    wd, sd, bd, xd = D.u32(w, dev), as16(s), as16(b), as16(x)
    dense = torch.zeros((N, K), dtype=torch.float16, device=dev)
    y = torch.zeros((1, N), dtype=torch.float16, device=dev)
    assert enc.set_function("affine_dequant", "affine_dequant_w4g64") == 1
    for i, t in enumerate((wd, sd, bd, dense)):
        enc.set_buffer(i, t)
    enc.set_constant(4, K)
    enc.set_constant(5, N)
    enc.dispatch((K // 8, N, 1), (64, 1, 1))
    encode_linear(enc, "affine_qmv", "affine_qmv_w4g64", wd, sd, bd, xd, y, K, N, grid=(32, N // 4, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert np.array_equal(dense.view(torch.int16).cpu().numpy().view(np.uint16), oracle.dequant_f16(w, s, b, K, N))
    assert torch.equal(y, vpq.qmv_w4g64_f16(wd, sd, bd, xd, K, N, 1))
    assert enc.set_function("affine_qmv", "affine_qmm_steel_w4g64") == 0       # not in that library
    # the fused q|k|v GEMV of the binary16 build (slots 4..6 the three outputs, 7:K 8..10 the row counts)
    rows = (24, 16, 8)
    qo, ko, vo = (torch.zeros((1, r), dtype=torch.float16, device=dev) for r in rows)
    assert enc.set_function("affine_qmv", "affine_qmv_qkv_w4g64") == 1
    for i, t in enumerate((wd, sd, bd, xd, qo, ko, vo)):
        enc.set_buffer(i, t)
    enc.set_constant(7, K)
    for i, r in enumerate(rows):
        enc.set_constant(8 + i, r)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(torch.cat((qo, ko, vo), dim=1), y)
    # the fused GEMM of the binary16 build, plain and gated, under its function names (slot 7 = M)
    M = 70
    xm = as16(np.random.default_rng(79).standard_normal((M, K)).astype(np.float16).view(np.uint16))
    ym = torch.zeros((M, N), dtype=torch.float16, device=dev)
    yg = torch.zeros((M, N // 2), dtype=torch.float16, device=dev)
    encode_linear(enc, "affine_qmm_steel", "affine_qmm_steel_w4g64_bm64", wd, sd, bd, xm, ym, K, N, M=M, grid=(1, 2, 1))
    encode_linear(enc, "affine_qmm_steel", "affine_qmm_swiglu_w4g64", wd, sd, bd, xm, yg, K, N, M=M, grid=(1, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(ym, vpq.qmm_w4g64_f16(wd, sd, bd, xm, K, N, M))
    assert torch.equal(yg, vpq.qmm_w4g64_f16(wd, sd, bd, xm, K, N, M, activation=1))
    assert ym.abs().sum() > 0 and yg.abs().sum() > 0


def test_mixed_width_gather_function_names(vpq, enc, dev, D):
    # affine_gather_qmv_swiglu_w4w8g64 / _w8w4g64: slots 0..2 gate pack, 3..5 up pack, 6:x 7:y 8:K 9:ffn 10:pair_eid 11:top_k
    K, ffn, E, top_k, M = 512, 24, 3, 2, 2
    g4 = [synth.make_weight(ffn, K, 3300 + e) for e in range(E)]
    u8 = [synth.make_weight8(ffn, K, 3310 + e) for e in range(E)]
    gd = tuple(f(np.stack([p[i] for p in g4]), dev) for i, f in enumerate((D.u32, D.bf16, D.bf16)))
    ud = tuple(f(np.stack([p[i] for p in u8]), dev) for i, f in enumerate((D.u32, D.bf16, D.bf16)))
    xd = D.bf16(synth.make_act(M, K, 3320), dev)
    eid = torch.tensor([2, 0, 1, 2], dtype=torch.int32, device=dev)
    for name, gate, up, gb, ub in (("affine_gather_qmv_swiglu_w4w8g64", gd, ud, 4, 8), ("affine_gather_qmv_swiglu_w8w4g64", ud, gd, 8, 4)):
        y = torch.zeros((M * top_k, ffn), dtype=torch.bfloat16, device=dev)
        assert enc.set_function("affine_qmv_bf16", name) == 1
        for i, t in enumerate(gate + up + (xd, y)):
            enc.set_buffer(i, t)
        enc.set_constant(8, K)
        enc.set_constant(9, ffn)
        enc.set_buffer(10, eid)
        enc.set_constant(11, top_k)
        enc.dispatch((32, ffn // 4, M * top_k), (32, 2, 1))
        ok, why = enc.wait_ok()
        assert ok, why
        assert torch.equal(y, vpq.gather_qmv_gated_split(gate, gb, up, ub, xd, K, ffn, eid, top_k, E))
        assert y.abs().sum() > 0


def test_eight_bit_gemm_function_names(vpq, enc, dev, D):
    # affine_qmm_steel_w8g64 (slot 7 = M), affine_qmm_swiglu_w8g64, and the 8-bit expert-sorted pair
    # (slot 7 = npad, 8 = tile2e, 9 = srow / sdst): the encoder's results are the C ABI's
    K, ffn, H, E, top_k, T = 512, 64, 96, 3, 2, 40
    packs = []
    for e in range(E):
        g, u = synth.make_weight8(ffn, K, 3900 + 2 * e), synth.make_weight8(ffn, K, 3901 + 2 * e)
        packs.append(tuple(np.stack([a, b], axis=1).reshape((2 * ffn,) + a.shape[1:]) for a, b in zip(g, u)))
    gu_d = tuple(f(np.stack([p[i] for p in packs]), dev) for i, f in enumerate((D.u32, D.bf16, D.bf16)))
    dn = [synth.make_weight8(H, ffn, 3950 + e) for e in range(E)]
    dn_d = tuple(f(np.stack([p[i] for p in dn]), dev) for i, f in enumerate((D.u32, D.bf16, D.bf16)))
    xd = D.bf16(synth.make_act(T, K, 3960), dev)
    eid = torch.from_numpy(np.random.default_rng(3961).integers(0, E, size=T * top_k, dtype=np.int32)).to(dev)
    t2e, srow, sdst, _ = vpq.moe_sort_pairs(eid, top_k, E)
    npad = srow.numel()
    y = torch.zeros((T, 2 * ffn), dtype=torch.bfloat16, device=dev)
    yg = torch.zeros((T, ffn), dtype=torch.bfloat16, device=dev)
    gact = torch.zeros((npad, ffn), dtype=torch.bfloat16, device=dev)
    part = torch.zeros((T * top_k, H), dtype=torch.bfloat16, device=dev)
    one = tuple(t[1] for t in gu_d)                       # expert 1's slab as a plain pack
    encode_linear(enc, "affine_qmm_steel_bf16", "affine_qmm_steel_w8g64", *one, xd, y, K, 2 * ffn, M=T, grid=(2 * ffn, T, 2), tg=(32, 2, 2))
    encode_linear(enc, "affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64", *one, xd, yg, K, 2 * ffn, M=T, grid=(2 * ffn, T, 2), tg=(32, 2, 2))
    for name, pack, src, dst, kk, nn, idx in (("affine_qmm_grouped_swiglu_w8g64", gu_d, xd, gact, K, 2 * ffn, srow),
                                               ("affine_qmm_grouped_w8g64", dn_d, gact, part, ffn, H, sdst)):
        assert enc.set_function("affine_qmm_steel_bf16", name) == 1
        for i, t in enumerate(pack + (src, dst)):
            enc.set_buffer(i, t)
        enc.set_constant(5, kk)
        enc.set_constant(6, nn)
        enc.set_constant(7, npad)
        enc.set_buffer(8, t2e)
        enc.set_buffer(9, idx)
        enc.dispatch((((nn + 31) // 32) * 32, ((npad + 31) // 32) * 2, 2), (32, 2, 2))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(y, vpq.qmm_w8g64(*one, xd, K, 2 * ffn, T))
    assert torch.equal(yg, vpq.qmm_w8g64(*one, xd, K, 2 * ffn, T, activation=1))
    want_act = vpq.qmm_grouped_gated_w8g64(*gu_d, xd, K, 2 * ffn, t2e, srow, E)
    live = (srow >= 0)
    assert torch.equal(gact[live], want_act[live])
    want_part = torch.zeros_like(part)
    vpq.qmm_grouped_down_w8g64(*dn_d, gact, ffn, H, t2e, sdst, E, out=want_part)
    assert torch.equal(part, want_part) and part.abs().sum() > 0


def test_group32_gemm_function_names(vpq, enc, dev, D):
    K, N, M = 256, 72, 50
    w, s, b = synth.make_weight_g32(N, K, 4000)
    wd, sd, bd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev)
    xd = D.bf16(synth.make_act(M, K, 4001), dev)
    y = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    yg = torch.zeros((M, N // 2), dtype=torch.bfloat16, device=dev)
    encode_linear(enc, "affine_qmm_steel_bf16", "affine_qmm_steel_w4g32", wd, sd, bd, xd, y, K, N, M=M, grid=(N, M, 2), tg=(32, 2, 2))
    encode_linear(enc, "affine_qmm_steel_bf16", "affine_qmm_geglu_w4g32", wd, sd, bd, xd, yg, K, N, M=M, grid=(N, M, 2), tg=(32, 2, 2))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(y, vpq.qmm_w4g32(wd, sd, bd, xd, K, N, M))
    assert torch.equal(yg, vpq.qmm_w4g32(wd, sd, bd, xd, K, N, M, activation=2))


@pytest.mark.parametrize("M", [3, 100])
def test_load_and_run_eight_bit_and_group32_packs(vpq, enc, dev, D, tmp_path, M):
    # packs of the other two formats written with the format's own library, opened again, their width and
    # group recovered from the shapes, loaded and run through quant_linear_forward: the bits of the C ABI's
    # size-based entrances on the same tensors
    L = enc.L
    L.hr_open.restype = ctypes.c_void_p
    L.hr_open.argtypes = [ctypes.c_char_p, ctypes.c_int]
    L.hr_close.argtypes = [ctypes.c_void_p]
    L.hr_why.restype = ctypes.c_char_p
    L.hd_load_and_run.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_void_p,
                                  ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int)]
    K, N = 512, 72
    w8, s8, b8 = synth.make_weight8(N, K, 4200)
    w32, s32, b32 = synth.make_weight_g32(N, K, 4201)
    as_bf16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)
    import safetensors.torch as sttorch
    sttorch.save_file({"a.weight": torch.from_numpy(w8.view(np.int32)),
                       "a.scales": as_bf16(s8), "a.biases": as_bf16(b8),
                       "b.weight": torch.from_numpy(w32.view(np.int32)), "b.scales": as_bf16(s32), "b.biases": as_bf16(b32)},
                      str(tmp_path / "model.safetensors"))
    # the reader wants U32 weights: rewrite the header's dtype of the two code tensors (I32 -> U32, same bytes)
    raw = (tmp_path / "model.safetensors").read_bytes()
    hlen = int.from_bytes(raw[:8], "little")
    header = raw[8:8 + hlen].replace(b'"I32"', b'"U32"')
    assert len(header) == hlen
    (tmp_path / "model.safetensors").write_bytes(raw[:8] + header + raw[8 + hlen:])
    r = L.hr_open(str(tmp_path / "model.safetensors").encode(), 0)
    assert r, L.hr_why()
    xd = D.bf16(synth.make_act(M, K, 4202), dev)
    kn = (ctypes.c_int * 2)()
    for prefix, kind, pack in ((b"a", "w8g64", (w8, s8, b8)), (b"b", "w4g32", (w32, s32, b32))):
        yd = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
        torch.cuda.synchronize()
        assert L.hd_load_and_run(enc.h, r, prefix, K, xd.data_ptr(), yd.data_ptr(), M, kn) == 1, L.hr_why()
        assert tuple(kn) == (K, N)
        want = vpq.linear_twin(kind, D.u32(pack[0], dev), D.bf16(pack[1], dev), D.bf16(pack[2], dev), xd, K, N, M)
        assert torch.equal(yd, want) and yd.abs().sum() > 0
    # without K: the 8-bit group-64 pack is the one pair of served formats its two shapes agree on; the 4-bit
    # group-32 shapes fit no group-64 format and the loader asks for K instead of guessing
    yd = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    assert L.hd_load_and_run(enc.h, r, b"a", 0, xd.data_ptr(), yd.data_ptr(), M, kn) == 1, L.hr_why()
    assert tuple(kn) == (K, N)
    assert torch.equal(yd, vpq.linear_twin("w8g64", D.u32(w8, dev), D.bf16(s8, dev), D.bf16(b8, dev), xd, K, N, M))
    assert L.hd_load_and_run(enc.h, r, b"b", 0, xd.data_ptr(), yd.data_ptr(), M, kn) == 0
    assert b"pass K" in L.hr_why()
    L.hr_close(r)
    # 8-bit codes in groups of 32: the GEMV in slabs up to 64 rows, the dequant-once route above
    w3, s3, b3 = synth.make_weight8(N, K, 4203, group=32)
    sttorch.save_file({"c.weight": torch.from_numpy(w3.view(np.int32)), "c.scales": as_bf16(s3), "c.biases": as_bf16(b3)},
                      str(tmp_path / "c.safetensors"))
    raw = (tmp_path / "c.safetensors").read_bytes()
    hlen = int.from_bytes(raw[:8], "little")
    (tmp_path / "c.safetensors").write_bytes(raw[:8] + raw[8:8 + hlen].replace(b'"I32"', b'"U32"') + raw[8 + hlen:])
    r = L.hr_open(str(tmp_path / "c.safetensors").encode(), 0)
    assert r, L.hr_why()
    yd = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    assert L.hd_load_and_run(enc.h, r, b"c", K, xd.data_ptr(), yd.data_ptr(), M, kn) == 1, L.hr_why()
    p3 = (D.u32(w3, dev), D.bf16(s3, dev), D.bf16(b3, dev))
    if M <= 64:
        want = torch.cat([vpq.qmv_w8g32(*p3, xd[m0:m0 + 16], K, N, min(16, M - m0)) for m0 in range(0, M, 16)])
    else:
        want = vpq.qmm_dense_route_w8g32(*p3, xd, K, N, M, torch.empty((N, K), dtype=torch.bfloat16, device=dev))
    assert torch.equal(yd, want) and yd.abs().sum() > 0
    L.hr_close(r)


def test_gelu_mul_and_shared_expert_gate_function_names(vpq, enc, dev, D):
    # affine_qmv_gelu_mul_w4g64 (slots 0..6 as the GEMV, 7 = the multiplier) and affine_moe_gate_w8g64 (0:w 1:scales
    # 2:biases 3:x 4:gate 5:K, rows of x = grid.y): the encoder's results are the C ABI's, bit for bit
    K, N, M = 2048, 96, 5
    w, s, b = synth.make_weight(N, K, 4100)
    x1 = synth.make_act(1, K, 4101)
    mul = synth.make_act(1, N, 4102)
    pd = (D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x1, dev))
    muld = D.bf16(mul, dev)
    y = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_gelu_mul_w4g64") == 1
    for i, t in enumerate(pd + (y,)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.set_buffer(7, muld)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    w8, s8, b8 = synth.make_weight8(1, K, 4103)
    xm = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(synth.make_act(M, K, 4104)) * np.float32(0.05))
    gd = (D.u32(w8, dev), D.bf16(s8, dev), D.bf16(b8, dev), D.bf16(xm, dev))
    gate = torch.zeros((M,), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_qmv_bf16", "affine_moe_gate_w8g64") == 1
    for i, t in enumerate(gd + (gate,)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.dispatch((32, M, 1), (32, 1, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(y, vpq.qmv_gelu_mul_w4g64(*pd, K, N, muld))
    assert torch.equal(gate, vpq.moe_gate_w8g64(*gd, K, M))
    assert y.abs().sum() > 0 and gate.float().std() > 0


def test_requantizer_gelu_mul_twins_and_variant_names(vpq, enc, dev, D):
    # affine_requant_w8_to_w4_g64 (0:w8 1:s8 2:b8 3:w4 4:s4 5:b4 6:K 7:N), the gelu-mul twins (the slots of the
    # group-64 4-bit form), and the names the reference keeps for tiling / accumulator variants of the same
    # mathematics: all are the C ABI's results, bit for bit
    K, N = 1024, 48
    w8, s8, b8 = synth.make_weight8(N, K, 4200)
    wd, sd, bd = D.u32(w8, dev), D.bf16(s8, dev), D.bf16(b8, dev)
    w4 = torch.zeros((N, K // 8), dtype=torch.int32, device=dev)
    s4 = torch.zeros((N, K // 64), dtype=torch.bfloat16, device=dev)
    b4 = torch.zeros((N, K // 64), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_dequant_bf16", "affine_requant_w8_to_w4_g64") == 1
    for i, t in enumerate((wd, sd, bd, w4, s4, b4)):
        enc.set_buffer(i, t)
    enc.set_constant(6, K)
    enc.set_constant(7, N)
    enc.dispatch((K // 64, N, 1), (K // 64, 1, 1))
    x = D.bf16(synth.make_act(1, K, 4201), dev)
    mul = D.bf16(synth.make_act(1, N, 4202), dev)
    y8 = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_gelu_mul_w8g64") == 1
    for i, t in enumerate((wd, sd, bd, x, y8)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.set_buffer(7, mul)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    g = synth.make_weight_g32(N, K, 4203)
    gd = (D.u32(g[0], dev), D.bf16(g[1], dev), D.bf16(g[2], dev))
    y32 = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_gelu_mul_w4g32") == 1
    for i, t in enumerate(gd + (x, y32)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.set_buffer(7, mul)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    yv = torch.zeros((1, N), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_w8g64_r8p2") == 1
    for i, t in enumerate((wd, sd, bd, x, yv)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.dispatch((1, N // 16, 1), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    want = vpq.requant_w8_to_w4(wd, sd, bd, K, N)
    assert torch.equal(w4, want[0]) and torch.equal(s4, want[1]) and torch.equal(b4, want[2])
    assert torch.equal(y8, vpq.qmv_gelu_mul_w8g64(wd, sd, bd, x, K, N, mul))
    assert torch.equal(y32, vpq.qmv_gelu_mul_w4g32(*gd, x, K, N, mul))
    assert torch.equal(yv, vpq.qmv_w8g64(wd, sd, bd, x, K, N, 1))
    assert w4.abs().sum() > 0 and y8.abs().sum() > 0 and y32.abs().sum() > 0
    for lib, name in [("affine_qmv_bf16", "affine_qmv_w4g64_r8p2"), ("affine_qmm", "affine_qmm_w4g64"),
                      ("affine_qmm_steel_bf16", "affine_qmm_steel_w4g64_bm64_acc16"),
                      ("affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_acc16"),
                      ("affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm64_acc16"),
                      ("affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm64_rs_acc16"),
                      ("affine_qmm_steel_bf16", "affine_qmm_steel_w8g64_bm64_acc16"),
                      ("affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_acc16"),
                      ("affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_bm64_acc16"),
                      ("affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_bm64_rs_acc16")]:
        assert enc.set_function(lib, name) == 1, name


@pytest.mark.parametrize("name", ["affine_qmv_qkv_w8g64", "affine_qmv_qkv_w4g32"])
def test_fused_qkv_call_sites_of_the_format_twins(vpq, enc, dev, D, name):
    # gpu-kernels/metal/quant/affine_qmv.metal:518-559: the slots of affine_qmv_qkv_w4g64 over the 8-bit and the
    # group-32 pack; the three outputs are the C ABI's plain QMV over the whole pack, bit for bit
    K, rows = 1024, (256, 64, 64)
    N = sum(rows)
    eight = name.endswith("w8g64")
    w, s, b = synth.make_weight8(N, K, 60) if eight else synth.make_weight_g32(N, K, 61)
    x = synth.make_act(1, K, 62)
    wd, sd, bd, xd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev)
    outs = [torch.zeros((1, r), dtype=torch.bfloat16, device=dev) for r in rows]
    assert enc.set_function("affine_qmv_bf16", name) == 1
    for i, t in enumerate((wd, sd, bd, xd, outs[0], outs[1], outs[2])):
        enc.set_buffer(i, t)
    enc.set_constant(7, K)
    for i, r in enumerate(rows):
        enc.set_constant(8 + i, r)
    enc.dispatch((32, N // 4, 1), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    whole = vpq.qmv_w8g64(wd, sd, bd, xd, K, N, 1) if eight else vpq.qmv_w4g32(wd, sd, bd, xd, K, N, 1)
    assert torch.equal(torch.cat(outs, dim=1), whole)
    assert whole.abs().sum() > 0


@pytest.mark.parametrize("name,fmt", [("affine_qmv_qkv_rms_w4g64", 0), ("affine_qmv_qkv_rms_w4g32", 1),
                                      ("affine_qmv_qkv_rms_w8g64", 2)])
def test_rmsnorm_fused_qkv_call_sites(vpq, enc, dev, D, name, fmt):
    # gpu-kernels/metal/quant/affine_qmv.metal:671-740: slots 0:w 1:scales 2:biases 3:x 4:norm_w 5:q 6:k 7:v 8:K
    # 9..11 rows 12:eps; the outputs are the C ABI's composed call, bit for bit
    K, rows, eps = 1024, (256, 64, 64), 1e-6
    N = sum(rows)
    w, s, b = (synth.make_weight, synth.make_weight_g32, synth.make_weight8)[fmt](N, K, 70 + fmt)
    x = synth.make_act(1, K, 73)
    nw = synth.f32_to_bf16_bits((1.0 + 0.1 * np.random.default_rng(74).standard_normal(K)).astype(np.float32))
    wd, sd, bd, xd, nwd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev), D.bf16(nw, dev)
    outs = [torch.zeros((1, r), dtype=torch.bfloat16, device=dev) for r in rows]
    assert enc.set_function("affine_qmv_bf16", name) == 1
    for i, t in enumerate((wd, sd, bd, xd, nwd, outs[0], outs[1], outs[2])):
        enc.set_buffer(i, t)
    enc.set_constant(8, K)
    for i, r in enumerate(rows):
        enc.set_constant(9 + i, r)
    enc.set_constant_f32(12, eps)
    enc.dispatch((32, N // 8, 1), (32, 2, 1))
    ok, why = enc.wait_ok()
    assert ok, why
    packs, r0 = [], 0
    for n in rows:
        packs.append((wd[r0:r0 + n], sd[r0:r0 + n], bd[r0:r0 + n], n))
        r0 += n
    for o, ref in zip(outs, vpq.qmv_qkv_rms(fmt, packs, xd, nwd, K, eps)):
        assert torch.equal(o, ref)
    assert outs[0].abs().sum() > 0


def test_eight_bit_group32_function_names(vpq, enc, dev, D):
    # affine_dequant_w8g32, affine_qmv_w8g32, affine_qmm_steel_w8g32 (slots of the 4-bit functions; the GEMM's
    # expansion goes through scratch of the stream): the encoder's results are the C ABI's, bit for bit
    K, N, M, Mq = 512, 40, 2, 70
    w, s, b = synth.make_weight8(N, K, 90, group=32)
    x, xq = synth.make_act(M, K, 91), synth.make_act(Mq, K, 92)
    wd, sd, bd, xd, xqd = D.u32(w, dev), D.bf16(s, dev), D.bf16(b, dev), D.bf16(x, dev), D.bf16(xq, dev)
    dq = torch.zeros((N, K), dtype=torch.bfloat16, device=dev)
    y = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    yq = torch.zeros((Mq, N), dtype=torch.bfloat16, device=dev)
    assert enc.set_function("affine_dequant_bf16", "affine_dequant_w8g32") == 1
    for i, t in enumerate((wd, sd, bd, dq)):
        enc.set_buffer(i, t)
    enc.set_constant(4, K)
    enc.set_constant(5, N)
    enc.dispatch((K // 4, N, 1), (32, 1, 1))
    assert enc.set_function("affine_qmv_bf16", "affine_qmv_w8g32") == 1
    for i, t in enumerate((wd, sd, bd, xd, y)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.dispatch((32 * M, N // 4, 1), (32, 2, 1))
    assert enc.set_function("affine_qmm_steel_bf16", "affine_qmm_steel_w8g32") == 1
    for i, t in enumerate((wd, sd, bd, xqd, yq)):
        enc.set_buffer(i, t)
    enc.set_constant(5, K)
    enc.set_constant(6, N)
    enc.set_constant(7, Mq)
    enc.dispatch(((N + 31) // 32, (Mq + 31) // 32, 1), (32, 2, 2))
    ok, why = enc.wait_ok()
    assert ok, why
    assert torch.equal(dq, vpq.dequant_w8g32(wd, sd, bd, K, N))
    assert torch.equal(y, vpq.qmv_w8g32(wd, sd, bd, xd, K, N, M))
    scratch = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    assert torch.equal(yq, vpq.qmm_dense_route_w8g32(wd, sd, bd, xqd, K, N, Mq, scratch))
    assert y.abs().sum() > 0 and yq.abs().sum() > 0
