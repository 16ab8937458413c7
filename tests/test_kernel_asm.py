"""Build-time checks on the code the compiler makes of the GEMM kernel (no GPU needed).

The kernel issues its MFMAs from inline assembly, which the compiler treats as
opaque: it neither knows their latency nor inserts the wait states the hardware
needs between an MFMA and a read of its accumulator.  The source therefore keeps
the accumulators in the matrix-core register file and reads them itself behind an
explicit delay.  These checks make a build fail if the compiler ever places an
accumulator access of its own close behind an MFMA, and keep the register budget
that lets the consumer's wavefronts run beside the GEMM's.
"""
import os
import re
import subprocess

import pytest

from flashoverlap_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MIN_WAIT_STATES = 16   # the longest MFMA of this family needs fewer before its result may be read


@pytest.fixture(scope="module")
def gemm_asm(tmp_path_factory):
    hipcc = os.path.join(build.ROCM, "bin", "hipcc")
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    out = tmp_path_factory.mktemp("asm") / "fo_gemm.s"
    flags = [f for f in build.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [hipcc, *flags, "--cuda-device-only", "-S", os.path.join(build.CSRC, "fo_gemm.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    return out.read_text()


def _kernels(text):
    """name -> (instruction lines, metadata dict) for every gemm_kernel instantiation."""
    bodies, name = {}, None
    for line in text.splitlines():
        m = re.match(r"^(_ZN2fo11gemm_kernel\S+):", line)
        if m:
            name = m.group(1)
            bodies[name] = []
            continue
        if name:
            if line.startswith(".Lfunc_end"):
                name = None
                continue
            code = line.split(";")[0].strip()
            if code:
                bodies[name].append(code)
    meta = {}
    for m in re.finditer(r"\.name:\s+(_ZN2fo11gemm_kernel\S+)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)\n\s+\.vgpr_spill_count:\s+(\d+)",
                         text):
        meta[m.group(1)] = {"vgpr": int(m.group(2)), "spill": int(m.group(3))}
    return bodies, meta


AGPR = re.compile(r"\ba(\d+|\[\d+:\d+\])")


def test_no_accumulator_access_close_behind_an_mfma(gemm_asm):
    bodies, _ = _kernels(gemm_asm)
    assert len(bodies) == 40            # 2 types x 2 macro tiles x (plain 2 + plain any-shape 2 + signal 3 + scatter 3)
    for name, ins in bodies.items():
        assert sum(i.startswith("v_mfma") for i in ins) > 0
        waited = None                   # wait states since the last MFMA of this straight-line stretch
        for i in ins:
            if i.endswith(":") or i.startswith(("s_branch", "s_cbranch", "s_endpgm")):
                waited = None           # a new stretch: what ran before it is not known here
                continue
            if i.startswith("v_mfma"):
                waited = 0
                continue
            if waited is not None:
                if AGPR.search(i):
                    assert waited >= MIN_WAIT_STATES, f"{name}: '{i}' only {waited} wait states behind an MFMA"
                m = re.match(r"s_nop (\d+)", i)
                waited += int(m.group(1)) + 1 if m else 1


def test_no_mfma_close_behind_an_accumulator_write(gemm_asm):
    """The other direction: the zeroed accumulators must have landed before the first MFMA adds to them."""
    bodies, _ = _kernels(gemm_asm)
    for name, ins in bodies.items():
        since_write = None
        for i in ins:
            if i.endswith(":") or i.startswith(("s_branch", "s_cbranch", "s_endpgm")):
                since_write = None
                continue
            if i.startswith(("v_accvgpr_write", "v_accvgpr_mov")):
                since_write = 0
                continue
            if since_write is not None:
                if i.startswith("v_mfma"):
                    assert since_write >= 4, f"{name}: an MFMA {since_write} wait states behind an accumulator write"
                m = re.match(r"s_nop (\d+)", i)
                since_write += int(m.group(1)) + 1 if m else 1


def test_register_budget_and_no_spills(gemm_asm):
    _, meta = _kernels(gemm_asm)
    assert len(meta) == 40
    for name, m in meta.items():
        assert m["spill"] == 0, f"{name} spills {m['spill']} registers"
        # 512 registers per SIMD lane: what the GEMM leaves free is all the consumer's wavefronts
        # (at most 72 registers each) have while they run beside it
        assert m["vgpr"] <= 440, f"{name} takes {m['vgpr']} of 512 registers"


def _vregs(operand):
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"v(\d+)", operand)
    return {int(m.group(1))} if m else set()


def test_no_vector_write_to_the_data_of_a_store_just_issued(gemm_asm):
    """A store of more than 8 bytes reads its data registers for a cycle or two after issue; a vector
    instruction that writes one of them right behind it is a hazard.  The compiler keeps its own
    instructions apart, but the accumulator reads are assembly statements it cannot see into, and it
    may give them the registers of a store just issued (in an experimental kernel that drained
    accumulators between stores this corrupted single rows now and then)."""
    bodies, _ = _kernels(gemm_asm)
    stores = 0
    for name, ins in bodies.items():
        for at, code in enumerate(ins):
            if not re.match(r"(buffer|global)_store_dwordx[34]", code):
                continue
            stores += 1
            ops = [o.strip().rstrip(",") for o in code.split()[1:]]
            data = _vregs(ops[0]) if code.startswith("buffer") else _vregs(ops[1])
            waited = 0
            for nxt in ins[at + 1:at + 3]:
                if waited >= 1:
                    break
                m = re.match(r"s_nop (\d+)", nxt)
                if m:
                    waited += int(m.group(1)) + 1
                    continue
                if nxt.startswith("v_"):
                    assert not (_vregs(nxt.split()[1].rstrip(",")) & data), f"{name}: '{nxt}' right behind '{code}'"
                waited += 1
    assert stores > 0


def test_consumer_copy_variants_differ_in_their_stores(tmp_path):
    """The two store policies of the consumer copy are separate kernels: written as one kernel
    with a run-time branch the compiler folded both into ordinary stores and the knob did nothing."""
    hipcc = os.path.join(build.ROCM, "bin", "hipcc")
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    out = tmp_path / "fo_sync.s"
    flags = [f for f in build.HIPCC_FLAGS if f != "-fPIC"]
    subprocess.run([hipcc, *flags, "--cuda-device-only", "-S", os.path.join(build.CSRC, "fo_sync.hip"), "-o", str(out)],
                   check=True, capture_output=True, timeout=600)
    stores = {}
    name = None
    for line in out.read_text().splitlines():
        m = re.match(r"^(_ZN2fo\d+(?:consume_kernel|wait_consume_kernel)ILb([01])E\S*):", line)
        if m:
            name = m.group(1)
            stores[name] = [m.group(2) == "1", 0, 0]
            continue
        if name and line.startswith(".Lfunc_end"):
            name = None
        if name and ("global_store_dwordx4" in line or "buffer_store_dwordx4" in line):
            stores[name][1 if re.search(r"\bnt\b", line.split(";")[0]) else 2] += 1
    assert len(stores) == 4
    for name, (stream, nt, plain) in stores.items():
        assert (nt > 0 and plain == 0) if stream else (plain > 0 and nt == 0), (name, nt, plain)
    # The persistent consumer's wavefronts share SIMDs with the GEMM's, which take up to 440 of the 512
    # registers: with more than 72 a resident consumer would keep the GEMM's workgroups from being placed.
    text = out.read_text()
    found = re.findall(r"\.name:\s+(_ZN2fo\d+wait_consume_kernel\S+)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)\n\s+\.vgpr_spill_count:\s+(\d+)", text)
    assert len(found) == 2
    for name, vgpr, spill in found:
        assert int(vgpr) <= 72 and int(spill) == 0, (name, vgpr, spill)
