"""What the compiler made of the attention kernel, checked on its assembly.

The fast pass of swa_attn_fwd_kernel issues its matrix instructions as inline
assembly, which the compiler's hazard recogniser does not look into.  Two
properties of the generated code are therefore promises the source makes by
construction, and they are checked here on every build:

* A vector-ALU instruction that writes a register must be at least two wait
  states away from a matrix instruction that reads it as A, B or C operand
  (the distance the compiler itself keeps for its own matrix instructions; a
  constant formed right in front of an asm MFMA is read too early, which a
  stand-alone probe on the GPU showed as a wrong product).  This catches the
  register allocator gluing a fragment together with moves, or rematerialising
  a constant, right in front of an asm MFMA.
* The streaming loop touches no scratch memory (no register spilled there) and
  the kernel fits two waves per SIMD (at most 256 registers per lane).
"""
import os
import re
import subprocess

import pytest

from streamdiffusionv2_amd import build_ext

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MIN_WAIT_STATES = 2


@pytest.fixture(scope="module")
def assembly():
    out = os.path.join(ROOT, "build", "isa_check")
    os.makedirs(out, exist_ok=True)
    path = os.path.join(out, "swa_attn_fwd.s")
    cmd = [build_ext.hipcc_path(), *build_ext.HIPCC_FLAGS, f"-I{os.path.join(ROOT, 'include')}", f"-I{build_ext.CSRC}",
           "-S", "--cuda-device-only", str(build_ext.CSRC / "swa_attn_fwd.hip"), "-o", path]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return open(path).read().split("\n")


def kernel_bodies(lines):
    """{mangled name: lines} of every swa_attn_fwd_kernel instantiation."""
    starts = [i for i, l in enumerate(lines) if re.match(r"^_Z\S*swa_attn_fwd_kernel\S*:", l)]
    bodies = {}
    for st in starts:
        end = next(i for i in range(st, len(lines)) if lines[i].strip().startswith(".Lfunc_end"))
        bodies[lines[st].split(":")[0]] = lines[st:end]
    return bodies


def registers(operand):
    """Set of (file, index) a register operand names: v12, a[0:15], v[4:5]; empty for anything else."""
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", operand)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.fullmatch(r"([va])(\d+)", operand)
    if m:
        return {(m.group(1), int(m.group(2)))}
    return set()


def instructions(body):
    """(mnemonic, operands) of the real instructions, in order."""
    out = []
    for line in body:
        text = line.split(";")[0].strip()
        if not text or text.endswith(":") or text.startswith("."):
            continue
        parts = text.split(None, 1)
        ops = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
        out.append((parts[0], ops))
    return out


def writes_vgpr(mnemonic):
    # vector ALU results; loads are ordered by s_waitcnt and matrix results by the pipe itself
    return mnemonic.startswith("v_") and not mnemonic.startswith("v_mfma") and not mnemonic.startswith("v_cmp")


def test_two_instantiations_exist(assembly):
    assert len(kernel_bodies(assembly)) == 2


def early_reads(ins):
    """Matrix instructions that read a register a vector-ALU instruction wrote
    fewer than MIN_WAIT_STATES wait states earlier, and the number of matrix
    instructions seen."""
    problems, n_mfma = [], 0
    for i, (mn, ops) in enumerate(ins):
        if not mn.startswith("v_mfma"):
            continue
        n_mfma += 1
        sources = set()
        for o in ops[1:4]:
            sources |= registers(o)
        waited = 0
        j = i - 1
        while j >= 0 and waited < MIN_WAIT_STATES:
            pm, pops = ins[j]
            if pm == "s_nop":
                waited += int(pops[0], 0) + 1
            else:
                if writes_vgpr(pm) and pops and registers(pops[0]) & sources:
                    problems.append(f"{pm} {', '.join(pops)} -> {mn} {', '.join(ops)} after {waited} wait states")
                waited += 1
            j -= 1
    return problems, n_mfma


def test_the_check_sees_a_known_bad_sequence():
    bad = ["\tv_mov_b32_e32 v9, v8", "\tv_mfma_f32_4x4x4_16b_bf16 v[2:5], v[8:9], v[6:7], v[2:5]"]
    assert len(early_reads(instructions(bad))[0]) == 1
    spaced = [bad[0], "\ts_nop 1", bad[1]]
    assert early_reads(instructions(spaced))[0] == []
    accumulator = ["\tv_mov_b32_e32 v5, 0", "\tv_exp_f32_e32 v20, v21", bad[1]]
    assert len(early_reads(instructions(accumulator))[0]) == 1


def test_no_vector_write_right_before_a_matrix_read(assembly):
    for name, body in kernel_bodies(assembly).items():
        problems, n_mfma = early_reads(instructions(body))
        assert n_mfma >= 96, f"{name}: only {n_mfma} matrix instructions found"
        assert not problems, name + "\n" + "\n".join(problems[:10])


def test_streaming_loop_has_no_spills(assembly):
    for name, body in kernel_bodies(assembly).items():
        loop = next(i for i, l in enumerate(body) if "Loop Header" in l)
        drained = next(i for i, l in enumerate(body) if "matrix pipe drained, site 0" in l)
        assert drained > loop
        hot = body[loop:drained]
        assert sum("v_mfma_f32_32x32x16_bf16" in l for l in hot) >= 64
        spills = [l.strip() for l in hot if re.search(r"\bscratch_(load|store)", l)]
        assert not spills, f"{name}: scratch access in the streaming loop: {spills[:3]}"


def test_register_budget(assembly):
    text = "\n".join(assembly)
    counts = [int(x) for x in re.findall(r"\.vgpr_count:\s+(\d+)", text)]
    assert len(counts) == 2 and max(counts) <= 256, counts
