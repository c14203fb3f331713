"""Compile the HIP sources of the w4g64 quantized-linear library for gfx950.

    python -m vpipe_amd.build            # -> vpipe_amd/libvpq.so

hipcc cross-compiles without a GPU.  Objects are built in parallel and linked
into one shared library that exports the C ABI declared in include/vpq.h.
"""
import concurrent.futures
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libvpq.so")
SOURCES = ["vpq_api.hip", "vpq_dequant.hip", "vpq_qmv_simple.hip", "vpq_qmv_mfma.hip", "vpq_qmv_stream.hip", "vpq_qmv_ring.hip", "vpq_qmv_rows.hip", "vpq_qmv_flow.hip", "vpq_profile.hip", "vpq_argmax.hip", "vpq_sample.hip", "vpq_moe_sort.hip",
           "vpq_lora_a.hip", "vpq_qmm_tile.hip", "vpq_qmm_big.hip", "vpq_norm.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed fp32 VALU ops are switched off for every kernel (device pass only; the
# host pass prints a harmless "not a recognized feature" note).
# Kernel-argument preloading: the first words of a kernel's scalar arguments arrive in scalar registers when a
# wavefront starts (see VPQ_PRELOADED_WORDS in vpq_internal.h).
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-kernarg-preload-count=16"]


# No kernel may spill registers.  Several kernels issue loads from inline assembly whose destination is a register
# and wait for them later with counted waits (gload16 in vpq_qmv_flow.hip, the x loads of vpq_qmv_ring.hip): the
# compiler takes the destination as written at the asm statement, so if it moves that register before the wait --
# a spill to scratch memory, a spill into the accumulation registers, a copy made while splitting a live range
# under register pressure -- it moves garbage and hands the register to other uses while the load is still on its
# way to it (seen once: a later address came out of such a register and the launch faulted).  The build fails
# instead, on three signs of that pressure:
#   * any kernel that uses scratch memory or reports spilled vector registers.  One exception, capped at the size
#     it has today: the binary16 256 x 256 GEMM tile spills 16 registers in its store epilogue (after the K loop); that kernel has no
#     register-destination asm loads at all (everything arrives by direct-to-LDS loads);
#   * a kernel with register-destination asm loads that holds accumulation registers (these kernels keep their
#     MFMA results in ordinary registers or use no MFMA, so any AGPR would be a spill slot);
#   * such a kernel using more than ASM_LOAD_VGPR_BUDGET of the 256 vector registers its launch bounds allow:
#     with headroom left the register allocator has no reason to split a live range.
# tests/test_gpu_dequant_qmv.py checks every instantiation the planner can reach against the oracle bit for bit,
# so a copy that slipped through would show as a wrong bit there.
SCRATCH_ALLOWED = {"_ZN3vpq14qmm_big_kernelILi4ELb0ELi3EEE": 68}    # mangled-name prefix -> bytes per lane
ASM_LOAD_KERNELS = re.compile(r"qmv_flow_kernel|qmv_ring_kernel")
ASM_LOAD_VGPR_BUDGET = 224
ASM_LOAD_SOURCES = ("vpq_qmv_flow.hip", "vpq_qmv_ring.hip")    # their assembly is walked by _check_inflight


def _check_registers(src, remarks):
    bad = []
    for block in re.split(r"remark: [^\n]*Function Name: ", remarks)[1:]:
        name = block.split()[0]

        def field(key):
            m = re.search(key + r": (\d+)", block)
            return int(m.group(1)) if m else 0

        scratch, vspill = field(r"ScratchSize \[bytes/lane\]"), field("VGPRs Spill")
        allowed = max([v for k, v in SCRATCH_ALLOWED.items() if name.startswith(k)] + [0])
        if scratch > allowed or (vspill > 0 and allowed == 0):
            bad.append("%s: %d bytes of scratch per lane, %d spilled vector registers" % (name, scratch, vspill))
        if ASM_LOAD_KERNELS.search(name):
            if allowed:
                bad.append("%s: a kernel with asm loads into registers may not be on the spill exemption list" % name)
            if field("AGPRs") > 0:
                bad.append("%s: %d accumulation registers in a kernel with asm loads into registers" % (name, field("AGPRs")))
            if field("VGPRs") > ASM_LOAD_VGPR_BUDGET:
                bad.append("%s: %d vector registers (budget %d)" % (name, field("VGPRs"), ASM_LOAD_VGPR_BUDGET))
    if bad:
        raise RuntimeError("%s: register allocation not allowed (see build.py):\n  %s" % (src, "\n  ".join(bad)))


# The registers of an asm load in flight, checked on the compiler's own assembly output of the kernels that have
# such loads: from a `global_load_* vN, ...` with a register destination until the `s_waitcnt vmcnt(n)` that
# guarantees its arrival (vector-memory operations retire in issue order, so a load with k younger operations is
# complete after a wait for n <= k), no instruction may name one of its destination registers.  That is the whole
# contract of gload16 / touch, and it covers what the resource checks above cannot see: a copy of the register made
# by live-range splitting, a spill into another register, a reuse.  The walk is a forward data-flow over the basic
# blocks (in-flight register -> fewest younger operations on any path, merged by union / minimum), so it does not
# depend on how the compiler lays the blocks out.  It follows every static path, feasible or
# not, so the kernels keep a wavefront that issues no such load on a path of its own.
_VMEM = re.compile(r"^(global|buffer|flat|scratch)_(load|store|atomic)")
_VREG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
_LABEL = re.compile(r"^([.\w$]+):")


def _vregs(text):
    regs = set()
    for m in _VREG.finditer(text):
        if m.group(1) is not None:
            regs.add(int(m.group(1)))
        else:
            regs.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return regs


def _check_inflight(src, asm):
    """Raises if an instruction of a kernel in `asm` touches the destination of a load that may still be in flight."""
    bad = []
    lines = asm.splitlines()
    i = 0
    while i < len(lines):
        m = _LABEL.match(lines[i])
        if not (m and lines[i].startswith("_Z") and ASM_LOAD_KERNELS.search(m.group(1))):
            i += 1
            continue
        kernel = m.group(1)
        # basic blocks of this function: [label, instructions]; ends at .Lfunc_end
        blocks, cur = [], [kernel, []]
        i += 1
        while i < len(lines) and not lines[i].startswith(".Lfunc_end"):
            t = lines[i].split(";")[0].strip()
            i += 1
            if not t:
                continue
            lm = _LABEL.match(t)
            if lm:
                blocks.append(cur)
                cur = [lm.group(1), []]
            elif not t.startswith("."):
                cur[1].append(t)
                if t.startswith(("s_branch", "s_cbranch", "s_endpgm", "s_setpc")):
                    blocks.append(cur)
                    cur = [None, []]
        blocks.append(cur)
        index = {b[0]: n for n, b in enumerate(blocks) if b[0]}
        state_in = [None] * len(blocks)       # {register: fewest younger vector-memory operations}
        state_in[0] = {}
        work = [0]
        seen_bad = set()
        while work:
            n = work.pop()
            st = dict(state_in[n])
            succ = [n + 1] if n + 1 < len(blocks) else []
            for t in blocks[n][1]:
                op = t.split()[0]
                args = t[len(op):]
                if op == "s_waitcnt":
                    w = re.search(r"vmcnt\((\d+)\)", t)
                    if w:
                        st = {r: y for r, y in st.items() if y < int(w.group(1))}
                    continue
                hit = _vregs(args) & set(st)
                if hit and (kernel, t) not in seen_bad:
                    seen_bad.add((kernel, t))
                    bad.append("%s: `%s` names v%d while a load into it may be in flight" % (kernel[:60], t, min(hit)))
                if _VMEM.match(op):
                    st = {r: min(y + 1, 64) for r, y in st.items()}
                    if "_load" in op and "_lds_" not in op and not op.startswith("scratch"):
                        for r in _vregs(args.split(",")[0]):
                            st[r] = 0
                if op == "s_branch":
                    succ = []
                if op in ("s_endpgm", "s_setpc_b64"):
                    succ = []
                if op.startswith(("s_branch", "s_cbranch")):
                    tgt = t.split()[-1]
                    if tgt in index:
                        succ = succ + [index[tgt]]
            for sn in succ:
                old = state_in[sn]
                if old is None:
                    merged = dict(st)
                else:
                    merged = dict(old)
                    for r, y in st.items():
                        merged[r] = min(y, merged.get(r, y))
                if merged != old:
                    state_in[sn] = merged
                    work.append(sn)
    if bad:
        raise RuntimeError("%s: register of an asm load used before its wait (see build.py):\n  %s"
                           % (src, "\n  ".join(bad[:20])))


def _compile(src):
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "remark:" not in l)
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    _check_registers(src, r.stderr)
    if src in ASM_LOAD_SOURCES:
        a = subprocess.run([HIPCC] + FLAGS + ["-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", "-"],
                           capture_output=True, text=True)
        if a.returncode != 0:
            raise RuntimeError("hipcc -S failed for %s:\n%s" % (src, a.stderr[-2000:]))
        _check_inflight(src, a.stdout)
    err = "\n".join(l for l in r.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "remark:" not in l and "-Rpass-analysis" not in l)
    return obj, err


def build(verbose=False):
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    build_host()
    return OUT


HOST_OUT = os.path.join(HERE, "libvpq_host.so")
ROOT = os.path.dirname(HERE)
DRIVER_SRC = os.path.join(ROOT, "tests", "host", "host_driver.cc")
DRIVER_OUT = os.path.join(ROOT, "tests", "host", "libhost_driver.so")


def _host_cc(args):
    r = subprocess.run([HIPCC, "-O2", "-std=c++17", "-fPIC", "-Wall", "-shared", "-D__HIP_PLATFORM_AMD__"] + args,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host build failed:\n" + r.stderr)


def build_host():
    """The C++ host layer (no device code) and, when the tests are present, their C driver over it."""
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "host")]
    _host_cc(inc + [os.path.join(HERE, "host", "vpq_host.cc"), os.path.join(HERE, "host", "vpq_weights.cc"), "-o", HOST_OUT, "-L" + HERE, "-lvpq",
                    "-Wl,-rpath,$ORIGIN"])
    if os.path.exists(DRIVER_SRC):
        _host_cc(inc + [DRIVER_SRC, "-o", DRIVER_OUT, "-L" + HERE, "-lvpq_host", "-lvpq",
                        "-Wl,-rpath,$ORIGIN/../../vpipe_amd"])
    return HOST_OUT


if __name__ == "__main__":
    print(build(verbose=True))
