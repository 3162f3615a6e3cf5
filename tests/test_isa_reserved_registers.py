"""k_mm5_q4k keeps its prefetched weight sets in v[232:255], registers the compiler is told not to allocate
(amdgpu_num_vgpr(232)); the loads into them are issued from inline assembly the compiler cannot see. If the
compiler ever used one of those registers for a value of its own - the attribute is a request it may exceed under
register pressure - a load in flight would overwrite that value, or the value the loaded weights, and the kernel
would read through garbage addresses. This test compiles the file to gfx950 assembly (no GPU needed) and checks
that, in every instantiation of the kernel, nothing but the kernel's own global_load_dwordx4 writes v232..v255
and that the kernel does not spill."""
import re
import subprocess
from pathlib import Path

import pytest

from retrograd_amd import build as B

ROOT = Path(__file__).resolve().parent.parent
RESERVED = range(232, 256)


def _written_registers(line):
    """Destination VGPRs of one instruction line (first operand)."""
    m = re.match(r"\s*(\S+)\s+(?:v\[(\d+):(\d+)\]|v(\d+)\b)", line)
    if not m:
        return None, []
    op = m.group(1)
    if m.group(2):
        return op, list(range(int(m.group(2)), int(m.group(3)) + 1))
    return op, [int(m.group(4))]


def test_the_compiler_never_writes_the_registers_the_weight_prefetch_owns(tmp_path):
    out = tmp_path / "mm_lds.s"
    cmd = [B.hipcc(), *[f for f in B.HIP_FLAGS if f != "-fPIC"], "-x", "hip", "-S", "--cuda-device-only",
           str(B.CSRC / "mm_lds.hip"), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    text = out.read_text().split("\n")
    starts = [i for i, l in enumerate(text) if re.match(r"^_ZN2rk9k_mm5_q4kENS_6MMArgsE:", l)]
    assert len(starts) == 1, "k_mm5_q4k is expected in the assembly"
    for s in starts:
        end = next(i for i in range(s, len(text)) if text[i].startswith(".Lfunc_end"))
        body = text[s:end]
        stores_from_reserved = 0
        for line in body:
            code = line.split(";")[0]
            if not code.strip() or code.strip().endswith(":") or code.strip().startswith("."):
                continue
            assert "scratch_" not in code, "k_mm5_q4k spills: " + code.strip()
            op, regs = _written_registers(code)
            if op is None or op.startswith(("global_store", "buffer_store", "ds_write", "ds_store", "s_", "v_cmp")):
                continue            # first operand of a store / compare is not a VGPR destination
            hit = [r for r in regs if r in RESERVED]
            if hit:
                assert op == "global_load_dwordx4", "the compiler writes a reserved register: " + code.strip()
                stores_from_reserved += 1
        assert stores_from_reserved >= 6, "the inline-assembly weight loads are expected in the kernel"
        meta = "\n".join(body)          # the kernel descriptor directives sit between the code and .Lfunc_end
        m = re.search(r"\.amdhsa_next_free_vgpr (\d+)", meta)
        assert m and int(m.group(1)) == 256
        m = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", meta)
        assert m and int(m.group(1)) == 0


# Kernels whose inner loops are sized to the register file: a spill there costs the kernel its speed without failing
# any numerical test (seen once: a refactoring of the expert kernels' step loop into a lambda spilled 21-45
# registers in the Q4_K / Q5_K / Q6_K variants). The private segment of these must stay empty.
NO_SPILL = {
    "moe.hip": [r"k_moe_gate_upILi\d+ELi2E", r"k_moe_downILi\d+ELi[12]E"],
    "mm_lds.hip": [r"k_mm2_q4kILi\dELi2ELb[01]E", r"k_mm2_q8_0ILi\dELi2E", r"k_mm2_q6kILi\dELi2E"],
    "kernels.hip": [r"k_attention_decodeILi\d+ELi8E", r"k_rmsnorm_act8ILi\dE"],
    # sixteen waves a workgroup leave a lane 128 registers; the two-token form of this kernel did not fit them
    "gemv.hip": [r"k_gemv_f32ILi\d+ELi1E"],
}


@pytest.mark.parametrize("source", sorted(NO_SPILL))
def test_the_register_bound_kernels_do_not_spill(tmp_path, source):
    out = tmp_path / (source + ".s")
    cmd = [B.hipcc(), *[f for f in B.HIP_FLAGS if f != "-fPIC"], "-x", "hip", "-S", "--cuda-device-only",
           str(B.CSRC / source), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    text = out.read_text()
    # the kernel descriptor of every kernel: .amdhsa_kernel <name> ... .amdhsa_private_segment_fixed_size N
    found = 0
    for m in re.finditer(r"\.amdhsa_kernel (\S+)(.*?)\.end_amdhsa_kernel", text, re.S):
        name, desc = m.group(1), m.group(2)
        if not any(re.search(p, name) for p in NO_SPILL[source]):
            continue
        found += 1
        size = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", desc)
        assert size and int(size.group(1)) == 0, "%s spills (%s bytes of scratch per lane)" % (name, size.group(1) if size else "?")
    assert found >= len(NO_SPILL[source]), "the kernels named here are expected in " + source
