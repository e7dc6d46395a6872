"""The small-M kernel relies on a property of the generated code: between the wait for the shortlist
ids and the last load of the prologue there is no other wait on vector loads, so activations,
weights and bias are all requested before the wave blocks for the first time (a single early wait
costs a memory round trip per call).  The compiler decides where waits go, and small source changes
have moved them; this test compiles the device code to assembly and checks every fully fused
instantiation (MODE 1) and every pre-quantized one (MODE 0)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "marian-dev_amd", "csrc")
HIPCC = "/opt/rocm/bin/hipcc"
KNOWN_HIP = "7.2"


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    # What these tests look at is the compiler's choice (where waits go, what spills), so they
    # hold for the compiler they were written against and say so instead of failing on another.
    version = subprocess.run([HIPCC, "--version"], capture_output=True, text=True).stdout
    m = re.search(r"HIP version:\s*(\d+\.\d+)", version)
    if not m or m.group(1) != KNOWN_HIP:
        pytest.skip("written against the code generation of HIP %s, found %s" % (KNOWN_HIP, m.group(1) if m else "?"))
    flags = None
    for line in open(os.path.join(CSRC, "Makefile")).read().replace("\\\n", " ").splitlines():
        if line.startswith("HIPFLAGS"):
            flags = line.split("=", 1)[1].replace("$(ARCH)", "gfx950").split()
    assert flags, "HIPFLAGS not found in the Makefile"
    flags = [f for f in flags if f not in ("-fPIC", "-shared")]
    out = tmp_path_factory.mktemp("asm") / "c_abi.s"
    cmd = [HIPCC] + flags + ["-S", "--cuda-device-only", "-o", str(out), "c_abi.hip"]
    r = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return open(out).read().split("\n")


def kernels(lines):
    for i, l in enumerate(lines):
        m = re.match(r"^(_ZN10marian_hip20gemm_stream32_kernelILi(\d)ELi(\d)ELi(\d)ELi(\d)ELi(\d)ELi(\d)ELi(\d+)E\w*):", l)
        if m:
            end = next(j for j in range(i, len(lines)) if "s_endpgm" in lines[j])
            yield m.group(1), tuple(int(x) for x in m.groups()[1:]), lines[i:end]


def test_no_wait_between_ids_and_last_prologue_load(assembly):
    checked = 0
    for name, (mt32, wn, kw, pw, mode, ng, rows), body in kernels(assembly):
        if mode == 2:      # quantize-on-stage: the abs-max partials are waited for first, by design
            continue
        first_barrier = next(i for i, l in enumerate(body) if "s_barrier" in l)
        loads = [i for i, l in enumerate(body[:first_barrier]) if "global_load" in l]
        waits = [i for i, l in enumerate(body[:first_barrier]) if re.search(r"s_waitcnt.*vmcnt", l)]
        assert loads and waits, name
        # waits[0] is the one for the shortlist ids (vmcnt(0) with nothing else in flight)
        early = [w for w in waits[1:] if w < loads[-1]]
        assert not early, "%s: wait on vector loads at line %d, before the last prologue load at %d" % (
            name, early[0], loads[-1])
        checked += 1
    assert checked >= 30, "expected the fused and pre-quantized instantiations, found %d" % checked


def test_no_scratch_memory_in_stream32_kernels(assembly):
    """Register arrays indexed through a lambda that is not inlined end up in scratch memory (a
    forty-fold slowdown was measured); every instantiation must report a zero private segment."""
    text = "\n".join(assembly)
    found = 0
    for m in re.finditer(r"\.name:\s+(_ZN10marian_hip20gemm_stream32_kernel\w+)\n(.*?)\.wavefront_size", text, re.S):
        meta = dict(re.findall(r"\.(vgpr_spill_count|private_segment_fixed_size):\s+(\d+)", m.group(2)))
        assert int(meta["private_segment_fixed_size"]) == 0 and int(meta["vgpr_spill_count"]) == 0, (m.group(1), meta)
        found += 1
    assert found >= 40


def test_no_scratch_memory_in_the_large_m_kernels_the_dispatch_picks(assembly):
    """The eight-wave 256x256 tile uses nearly all of its registers: a few more and it spills (a
    three-fold slowdown was measured).  Every paired-fragment instantiation and the tile-pair
    kernel must report a zero private segment."""
    text = "\n".join(assembly)
    found = 0
    for m in re.finditer(r"\.name:\s+(_ZN10marian_hip(?:18gemm_mfma32_kernelILi\d+ELi\d+ELi\dELi\dELi\dELb1E|24gemm_mfma32_split_kernel|16gemm_pair_kernel)\w+)\n(.*?)\.wavefront_size", text, re.S):
        meta = dict(re.findall(r"\.(vgpr_spill_count|private_segment_fixed_size):\s+(\d+)", m.group(2)))
        assert int(meta["private_segment_fixed_size"]) == 0 and int(meta["vgpr_spill_count"]) == 0, (m.group(1), meta)
        found += 1
    assert found >= 22


def test_no_wait_between_the_stores_of_the_large_m_epilogue(assembly):
    """Stores count as vector memory operations, so a wait for all of them between two stores of the
    write-out makes every store wait for the one before (measured: 41 k instead of 17 k clocks for
    a 256x256 tile).  The compiler put such waits behind the lane-wise branches of the edge form,
    ahead of every use of the bias value, until the kernel used those values once before the stores."""
    checked = 0
    for i, l in enumerate(assembly):
        m = re.match(r"^(_ZN10marian_hip(?:18gemm_mfma32_kernelILi\d+ELi\d+ELi\dELi\dELi\dELb1E|24gemm_mfma32_split_kernel)\w*):", l)
        if not m:
            continue
        end = next(j for j in range(i, len(assembly)) if "s_endpgm" in assembly[j])
        body = assembly[i:end]
        stores = [j for j, t in enumerate(body) if re.search(r"global_store_dword\s", t)]
        assert len(stores) >= 64, m.group(1)
        span = body[stores[0]:stores[-1] + 1]
        if "split_kernel" in m.group(1):
            # The loop of the split form's loading waves (waits for K blocks, no stores) may be laid
            # out between two blocks of stores; it is not part of the write-out.  Here the rule is
            # per basic block: a block with a store holds no wait on vector memory (the first
            # store's block: none behind that store).
            waits, block_has_store, block_waits = [], False, []
            for t in span + [".LBB_end:"]:
                if re.match(r"^\.LBB\w+:", t):
                    if block_has_store:
                        waits += block_waits
                    block_has_store, block_waits = False, []
                elif re.search(r"global_store_dword\s", t):
                    block_has_store = True
                elif re.search(r"s_waitcnt.*vmcnt", t):
                    block_waits.append(t.strip())
        else:
            waits = [t.strip() for t in span if re.search(r"s_waitcnt.*vmcnt", t)]
        assert not waits, (m.group(1), len(waits), waits[:3])
        checked += 1
    assert checked >= 22
