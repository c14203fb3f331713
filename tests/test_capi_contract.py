"""The C-ABI library loads and exports exactly what include/vpq.h declares.
No GPU: only symbol resolution, argument validation that happens before any
device call, and the host-side size helpers."""
import ctypes
import os
import re

import pytest

import vpipe_amd
from vpipe_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "vpq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vpq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = vpipe_amd.load()
    names = _declared()
    assert len(names) >= 14
    for n in names:
        assert hasattr(L, n), n
    assert sorted(n for n, _, _ in capi.SYMBOLS) == names


def test_missing_library_is_loud(monkeypatch, tmp_path):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "_SO", str(tmp_path / "libvpq.so"))
    with pytest.raises(FileNotFoundError):
        capi.load()


def test_host_side_validation_and_sizes():
    L = vpipe_amd.load()
    assert L.vpq_version() >= 100
    # generative-models/quantize/affine-quantizer.h:37-40
    assert L.vpq_weight_bytes(96, 256) == 96 * 32 * 4
    assert L.vpq_scale_bytes(96, 256) == 96 * 4 * 2
    assert L.vpq_qmv_workspace_bytes(4096, 1024, 1) % 256 == 0
    assert L.vpq_qmv_workspace_bytes(4096, 1024, 17) == 0
    one = ctypes.c_void_p(4096)   # never dereferenced: every call below fails validation first
    null = ctypes.c_void_p(0)
    # NULL buffers
    assert L.vpq_dequant_w4g64_bf16(null, null, one, one, one, 64, 1) == -1
    assert L.vpq_qmv_w4g64_bf16(null, one, one, one, null, one, 64, 8, 1, null, null, 0, 0) == -1
    # K not a multiple of the group, M out of range, bad rank
    assert L.vpq_dequant_w4g64_bf16(null, one, one, one, one, 96, 1) == -2
    assert L.vpq_qmv_w4g64_bf16(null, one, one, one, one, one, 64, 8, 17, null, null, 0, 0) == -2
    assert L.vpq_qmv_w4g64_bf16(null, one, one, one, one, one, 64, 8, 0, null, null, 0, 0) == -2
    assert L.vpq_qmm_w4g64_bf16(null, one, one, one, one, one, 64, 8, 0, null, null, 0, 0.0, null) == -2
    assert L.vpq_qmm_w4g64_bf16(null, one, one, one, one, one, 64, 8, 4, one, one, 36, 1.0, one) == -2      # rank not a multiple of 8
    assert L.vpq_qmm_w4g64_bf16(null, one, one, one, one, one, 64, 8, 4, one, one, 528, 1.0, one) == -2     # above VPQ_LORA_MAX_RANK
    # misaligned codes / x
    assert L.vpq_dequant_w4g64_bf16(null, ctypes.c_void_p(4100), one, one, one, 64, 1) == -3
    assert L.vpq_qmv_w4g64_bf16(null, one, one, one, ctypes.c_void_p(4098), one, 64, 8, 1, null, null, 0, 0) == -3
    # LoRA without its scratch
    assert L.vpq_qmm_w4g64_bf16(null, one, one, one, one, one, 64, 8, 4, one, one, 32, 1.0, null) == -4
    # fused gate|up: odd N, a residual-free epilogue the streaming kernel lacks, a column window
    # that does not fit its stride, odd row bytes
    assert L.vpq_qmv_swiglu_w4g64_bf16(null, one, one, one, one, one, 64, 7, 1, 0) == -2
    assert L.vpq_qmv_swiglu_w4g64_bf16(null, one, one, one, one, one, 64, 8, 1, capi.VPQ_QMV_STREAM) == -2
    assert L.vpq_qmm_swiglu_w4g64_bf16(null, one, one, one, one, one, 64, 8, 4, 6, 4) == -2
    assert L.vpq_qmm_swiglu_w4g64_bf16(null, one, one, one, one, one, 64, 8, 4, 0, 2) == -2
    assert L.vpq_interleave_rows(null, one, one, one, 3, 4) == -2
    assert L.vpq_interleave_rows(null, one, null, one, 4, 4) == -1
    assert L.vpq_embed_gather_w4g64_bf16(null, null, one, one, one, one, 64, 1, 8) == -1
    assert L.vpq_embed_gather_w4g64_bf16(null, one, one, one, one, one, 64, 0, 8) == -2
    assert b"NULL" in L.vpq_status_string(-1)


def test_host_layer_and_its_test_driver_load():
    # the C++ host layer links against the C ABI; its C test driver exports the encoder protocol
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    host = os.path.join(root, "vpipe_amd", "libvpq_host.so")
    drv = os.path.join(root, "tests", "host", "libhost_driver.so")
    assert os.path.exists(host) and os.path.exists(drv), "run python -m vpipe_amd.build"
    vpipe_amd.load()
    ctypes.CDLL(host, mode=ctypes.RTLD_GLOBAL)
    D = ctypes.CDLL(drv)
    for name in ("hd_open", "hd_close", "hd_set_function", "hd_set_buffer", "hd_set_constant_i32", "hd_dispatch",
                 "hd_scope_begin", "hd_scope_end", "hd_dispatch_count", "hd_wait_ok", "hd_reason", "hd_quant_linear"):
        assert hasattr(D, name), name


def test_build_refuses_kernels_that_spill():
    """Kernels that issue loads from inline assembly may not have their registers moved by the compiler before the
    counted wait: the build's check of the compiler's resource remarks fails on spills, on accumulation registers
    in such a kernel and on register pressure near its limit, with one capped exemption."""
    from vpipe_amd import build

    def remark(name, scratch=0, vgprs=64, agprs=0, vspill=0):
        lines = ["Function Name: %s" % name, "    VGPRs: %d" % vgprs, "    AGPRs: %d" % agprs,
                 "    ScratchSize [bytes/lane]: %d" % scratch, "    VGPRs Spill: %d" % vspill]
        return "".join("x.hip:1:1: remark: %s [-Rpass-analysis=kernel-resource-usage]\n" % l for l in lines)

    flow = "_ZN3vpq17qmv_flow_kernel_1ILi1ELi2ELb1ELb0EEEvPKtPKjS2_S2_PvijiS2_"
    ring = "_ZN3vpq15qmv_ring_kernelILi8ELi2ELb1ELb1EEEvjjjjjjjjjjjjjj"
    exempt = "_ZN3vpq14qmm_big_kernelILi4ELb0ELi3EEEvNS_12_GLOBAL__N_19BigParamsE"
    build._check_registers("x.hip", remark(ring) + remark(flow, vgprs=158) + remark(exempt, scratch=60, vgprs=256, agprs=256, vspill=15))
    for bad in (remark(ring, scratch=8),                       # scratch memory in use
                remark("_ZN3vpq13dequant_kernelEv", vspill=2),  # any kernel: spilled vector registers
                remark(exempt, scratch=4096, vspill=15),        # the exemption is capped
                remark(flow, agprs=4),                          # accumulation registers as spill slots
                remark(ring, vgprs=250)):                       # no headroom left
        with pytest.raises(RuntimeError, match="register allocation not allowed"):
            build._check_registers("x.hip", bad)


def test_build_refuses_use_of_a_load_register_before_its_wait():
    """The build walks the assembly of the kernels with asm loads into registers: from the load to the counted wait
    that guarantees its arrival no instruction may name a destination register, on any static path."""
    from vpipe_amd import build
    name = "_ZN3vpq17qmv_flow_kernel_1ILi1ELi2ELb1ELb0EEEvPKtPKjS2_S2_PvijiS2_"

    def kernel(body):
        return "\t.text\n%s:\n%s\n\ts_endpgm\n.Lfunc_end0:\n" % (name, "\n".join("\t" + l for l in body))

    ok = ["global_load_dwordx4 v[4:7], v1, s[2:3]",       # A
          "global_load_dwordx4 v[8:11], v1, s[4:5]",      # B
          "global_load_lds_dwordx4 v[2:3], off",          # to LDS: no register destination, but counted
          "v_add_u32_e32 v1, 16, v1",                     # other registers are free
          "s_waitcnt vmcnt(2)",                           # A has two younger operations: complete
          "v_mov_b32_e32 v20, v4",
          "s_waitcnt vmcnt(1)",
          "v_mov_b32_e32 v21, v8"]
    build._check_inflight("x.hip", kernel(ok))
    # kernels outside the list are not walked
    build._check_inflight("x.hip", kernel(ok[:2] + ["v_mov_b32_e32 v20, v4"]).replace("qmv_flow_kernel", "other_kernel"))
    bad_cases = [
        ok[:4] + ["v_mov_b32_e32 v20, v5"],                                  # a copy before any wait
        ok[:4] + ["s_waitcnt vmcnt(2)", "v_mov_b32_e32 v20, v9"],            # B has one younger operation only
        ok[:2] + ["v_mov_b32_e32 v6, 0"],                                    # overwritten while the load is on its way
        ok[:2] + ["s_waitcnt lgkmcnt(0)", "ds_write_b128 v30, v[4:7]"],      # a wait on the other counter
        # in flight on one of two joining paths
        ["s_cbranch_scc1 .LBB0_2"] + ok[:1] + [".LBB0_2:", "v_mov_b32_e32 v20, v4"],
        # around a loop: the load of one trip is read at the top of the next
        [".LBB0_1:", "v_mov_b32_e32 v20, v4"] + ok[:1] + ["s_cbranch_scc1 .LBB0_1"],
    ]
    for body in bad_cases:
        with pytest.raises(RuntimeError, match="used before its wait"):
            build._check_inflight("x.hip", kernel(body))
    # the same join is fine once both paths have waited
    build._check_inflight("x.hip", kernel(["s_cbranch_scc1 .LBB0_2"] + ok[:1] + ["s_waitcnt vmcnt(0)", ".LBB0_2:",
                                                                                  "v_mov_b32_e32 v20, v4"]))


def test_bench_refuses_more_than_one_gpu():
    # one GPU only: no collectives, no sharding; the benchmark says so instead of starting ranks
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
