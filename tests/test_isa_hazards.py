"""CPU-only check of the generated gfx950 code of the attention kernel.

The kernel's MFMAs are inline assembly, so the compiler knows neither their latency nor the wait states a vector
instruction needs before it may read an MFMA result (the hardware does not interlock that read).  The source keeps
such reads far behind the MFMAs by construction, or puts the wait states into the MFMA's own assembly statement
(at_mfma_acc_settled in csrc/sp_attn.hip).  What the source cannot see is the register allocator: to satisfy a tied
operand it may copy a result register with a vector move right behind the MFMA -- that happened in the pivot
instantiation and gave wrong row sums now and then.  This test compiles the file to assembly and measures, for every
vector / memory instruction that reads a register an MFMA wrote, how many wait states lie between the two."""

import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "shareprefill_amd", "csrc")
MIN_WAIT_STATES = 12  # an 8-pass MFMA needs 11 before a vector instruction reads its result
WINDOW = 40


def _regs(tok):
    tok = tok.strip().rstrip(",")
    m = re.match(r"v\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"-?\|?v(\d+)\|?$", tok)
    return {int(m.group(1))} if m else set()


def closest_reads(lines):
    """-> sorted [(wait states, mfma, reader)] for reads of MFMA results within WINDOW wait states.  Instructions are
    taken in program order (labels ignored); an s_nop N counts N + 1, an MFMA 4, anything else 1."""
    ins = [l.strip() for l in lines
           if l.strip() and not l.strip().startswith((";", ".")) and not l.strip().endswith(":")]
    found, pending = [], []
    for l in ins:
        op = l.split()[0]
        toks = [t for t in re.split(r"[ ,]+", l)[1:] if t]
        if op.startswith("v_mfma"):
            for p in pending:
                p[1] += 4
            dst = _regs(toks[0])
            pending = [p for p in pending if not (p[0] & dst)]  # accumulating in place: the hardware orders MFMAs
            pending.append([dst, 0, l])
            continue
        wait = int(toks[0]) + 1 if op == "s_nop" else 1
        is_store = op.startswith(("global_store", "ds_write", "buffer_store", "flat_store"))
        reads = set()
        if op.startswith(("v_", "ds_", "global_", "buffer_", "flat_")):
            for t in (toks if is_store else toks[1:]):
                reads |= _regs(t)
        for p in pending:
            if p[0] & reads:
                found.append((p[1], p[2], l))
        if op.startswith("v_") and toks:
            d = _regs(toks[0])
            pending = [p for p in pending if not (p[0] & d)]
        for p in pending:
            p[1] += wait
        pending = [p for p in pending if p[1] < WINDOW]
    return sorted(found)


def test_the_scanner_sees_a_copy_placed_right_behind_an_mfma():
    good = ["v_mfma_f32_16x16x32_bf16 v[8:11], v[0:3], v[4:7], v[8:11]", "s_nop 15", "v_mov_b32_e32 v20, v8"]
    bad = ["v_mfma_f32_16x16x32_bf16 v[8:11], v[0:3], v[4:7], v[8:11]", "s_nop 0", "v_mov_b64_e32 v[20:21], v[10:11]",
           "s_nop 15", "v_sub_f32_e32 v1, v20, v2"]
    assert closest_reads(good)[0][0] == 16
    assert closest_reads(bad)[0][0] == 1
    # an MFMA that accumulates into the same registers is ordered by the hardware and is no reader
    chain = ["v_mfma_f32_16x16x32_bf16 v[8:11], v[0:3], v[4:7], v[8:11]"] * 3
    assert closest_reads(chain) == []


def test_no_vector_instruction_reads_an_mfma_result_too_early():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    out = os.path.join(CSRC, "sp_attn.isa_check.s")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-S", "--cuda-device-only",
           os.path.join(CSRC, "sp_attn.hip"), "-o", out]
    try:
        subprocess.run(cmd, check=True, capture_output=True)
        text = open(out).read()
    finally:
        if os.path.exists(out):
            os.remove(out)
    kernels = {}
    for m in re.finditer(r"^(_Z\S*sp_attn_fwd_kernel\S*):.*\n", text, re.M):
        start = m.end()
        kernels[m.group(1)] = text[start:text.index(".Lfunc_end", start)].split("\n")
    assert len(kernels) == 5, "the forward kernel has five instantiations (pivot x half-channel, and small blocks)"
    for name, body in kernels.items():
        assert sum("v_mfma_f32_16x16x32_bf16" in l for l in body) > 100
        reads = closest_reads(body)
        assert not reads or reads[0][0] >= MIN_WAIT_STATES, (
            f"{name}: '{reads[0][2]}' reads the result of '{reads[0][1]}' only {reads[0][0]} wait states behind it")
