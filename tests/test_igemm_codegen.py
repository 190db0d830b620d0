"""Properties of the compiled gfx950 code of igemm.hip that its correctness or
speed rely on and that a compiler change could silently break:

  * no igemm kernel uses scratch memory (spilled accumulators cost an order of
    magnitude);
  * in igemm_wreg_kernel the weight fragments are requested by inline assembly
    into registers the compiler knows nothing about while the request is in
    flight: each fragment keeps one register quad, and between the pipeline
    fill and the wait that follows the K loop only the MFMAs and those requests
    themselves may name these registers, on any path (a compiler-inserted copy
    or reuse there would read or clobber data that has not landed yet);
  * those requests take their address from a scalar register pair, which a
    vector-memory instruction must not read within five wait states of a VECTOR
    instruction writing it (v_readfirstlane, v_cmp); the compiler does not look
    into the inline assembly for that, so the distance is checked here.
"""
import os
import re
import shutil
import subprocess

import pytest

import __graft_entry__ as entry

HIPCC = "/opt/rocm/bin/hipcc"
SRC = os.path.join(entry.ROOT, "heterogeneity-aware-lowering-and-optimization_amd", "csrc", "kernels", "igemm.hip")
FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-O3", "-std=c++17",
         "-fPIC", "-ffp-contract=off", "--cuda-device-only", "-S", "-Rpass-analysis=kernel-resource-usage"]


@pytest.fixture(scope="module")
def compiled(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    d = tmp_path_factory.mktemp("igemm_asm")
    out = os.path.join(d, "igemm.s")
    r = subprocess.run([HIPCC] + FLAGS + [SRC, "-o", out], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    asm = open(out).read()
    shutil.rmtree(d, ignore_errors=True)
    return asm, r.stderr


def test_no_scratch(compiled):
    _, remarks = compiled
    blocks = re.split(r"remark: [^\n]*Function Name: ", remarks)[1:]
    seen = 0
    for b in blocks:
        name = b.split("\n")[0]
        if "igemm" not in name:
            continue
        seen += 1
        scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b).group(1))
        assert scratch == 0, (name, scratch)
    assert seen >= 40


def kernel_bodies(asm, prefix):
    for name in re.findall(r"^(%s\w+):" % prefix, asm, re.M):
        a = asm.index(name + ":")
        b = asm.index(".Lfunc_end", a)
        body = [l.split(";")[0].strip() for l in asm[a:b].split("\n")]
        yield name, [l for l in body if l and (not l.startswith(".") or l.startswith(".LBB"))]


def test_weight_fragment_registers_untouched_in_flight(compiled):
    asm, _ = compiled
    # (the lane's 32-bit offset in a vector register, the fragment's wavefront-uniform address in scalar ones)
    req = re.compile(r"global_load_dwordx4 v\[(\d+):(\d+)\], (?:v\d+, s\[\d+:\d+\]|v\[\d+:\d+\], off) offset:(0|1024|2048|3072)$")
    checked = 0
    for name, body in kernel_bodies(asm, "_ZN4ohip17igemm_wreg_kernel"):
        quads = {(int(m.group(1)), int(m.group(2))) for m in map(req.match, body) if m}
        # Two sets of four fragments per 32-channel slice (the last two template
        # arguments: one or two slices per wavefront, one or two K groups per
        # workgroup), each tied to one register quad for the whole K loop (also in
        # stages the optimizer peels off the loop).
        targs = re.search(r"Li(\d)ELi(\d)EEEvNS_11IgemmParamsEi$", name)
        slices, k_groups = int(targs.group(1)), int(targs.group(2))
        assert slices in (1, 2) and k_groups in (1, 2), name
        assert len(quads) == 8 * slices, (name, quads)
        owned = {x for a, b in quads for x in range(a, b + 1)}
        assert len(owned) == 32 * slices, (name, quads)
        mfma = [i for i, l in enumerate(body) if "v_mfma" in l]
        first = min(i for i, l in enumerate(body) if req.match(l))
        drain = min(i for i, l in enumerate(body) if i > mfma[-1] and l.startswith("s_waitcnt vmcnt(0)"))
        assert first < mfma[0]
        # From the first request to the wait behind the loop these registers
        # belong to the requests and to the MFMAs that consume them, whatever
        # path the control flow takes: any other instruction naming one of them
        # would read data that may not have landed, or be overwritten by it.
        for i in range(first, drain):
            l = body[i]
            if req.match(l) or l.startswith(".LBB"):
                continue
            regs = []
            for r in re.finditer(r"v\[(\d+):(\d+)\]|\bv(\d+)\b", l):
                regs += list(range(int(r.group(1)), int(r.group(2)) + 1)) if r.group(1) else [int(r.group(3))]
            hit = [x for x in regs if x in owned]
            if "v_mfma" in l:
                # as the A operand only (v_mfma dst, a, b, c): never as destination or accumulator
                ops = [o.strip() for o in l.split(None, 1)[1].split(",")]
                for o in (ops[0], ops[3]):
                    m = re.match(r"[av]\[(\d+):(\d+)\]", o)
                    assert not (o.startswith("v") and m and any(x in owned for x in range(int(m.group(1)), int(m.group(2)) + 1))), (name, i, l)
                continue
            assert not hit, (name, i, l)
        checked += 1
    assert checked >= 12


def test_scalar_addresses_of_fragment_requests_are_settled(compiled):
    asm, _ = compiled
    req = re.compile(r"global_load_dwordx4 v\[\d+:\d+\], v\d+, s\[(\d+):(\d+)\]")
    vwrite = re.compile(r"(v_readfirstlane_b32|v_readlane_b32|v_cmp\w*)\s+s\[?(\d+)(?::(\d+))?")
    loads = 0
    for name, body in kernel_bodies(asm, "_ZN4ohip17igemm_wreg_kernel"):
        real = [l for l in body if not l.startswith(".LBB")]
        for i, l in enumerate(real):
            m = req.match(l)
            if not m:
                continue
            loads += 1
            lo, hi = int(m.group(1)), int(m.group(2))
            for back in real[max(0, i - 8):i]:
                w = vwrite.match(back)
                if w:
                    a = int(w.group(2))
                    b = int(w.group(3)) if w.group(3) else a
                    assert b < lo or a > hi, (name, back, l)
    assert loads >= 200
