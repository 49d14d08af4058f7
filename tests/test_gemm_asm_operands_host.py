"""The hand-scheduled GEMM loops take addresses and counts as inline-asm operands that stay live for the whole loop.
The compiler must never place one of them in a register the loop writes (that build reads outside its buffers), and
every register a loop names must be declared to the compiler.  Checked on the device assembly hipcc produces here."""
import importlib.util
import os
import shutil

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "g-core-gh_amd", "csrc")


def _load():
    spec = importlib.util.spec_from_file_location("check_asm_operands", os.path.join(CSRC, "check_asm_operands.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_every_loop_register_is_declared():
    C = _load()
    declared = C.declared_registers(os.path.join(CSRC, "gemm_fp8_big.hip"))
    loops = sorted(f for f in os.listdir(CSRC) if f.endswith("_loop.inc"))
    assert loops and set(loops) == set(declared)
    for f in loops:
        _, literal = C.load_template(os.path.join(CSRC, f))
        assert len(literal) > 100 and not literal - declared[f], (f, sorted(literal - declared[f]))


def test_template_matcher_reads_operands_back():
    C = _load()
    import re, tempfile
    with tempfile.NamedTemporaryFile("w", suffix="_loop.inc", delete=False) as f:
        f.write('"s_mov_b64 s[40:41], %[abase]\\n"\n"global_load_lds_dwordx4 %[aoff0], s[40:41]\\n"\n"Lx%=:\\n"\n"v_mov_b32 v128, 0\\n"\n')
    try:
        patterns, literal = C.load_template(f.name)
    finally:
        os.unlink(f.name)
    assert literal == {("s", 40), ("s", 41), ("v", 128)}
    body = ["\ts_mov_b64 s[40:41], s[12:13]", "\tglobal_load_lds_dwordx4 v128, s[40:41]", "Lx17:", "\tv_mov_b32 v128, 0"]
    got = {}
    for p, line in zip(patterns, body):
        m = p.match(line)
        assert m, line
        got.update(m.groupdict())
    assert got == {"abase__0": "s[12:13]", "aoff0__0": "v128"}
    assert C._regs("v128") & literal                       # the clash the audit reports


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_no_operand_lands_in_a_loop_register(capsys):
    assert _load().audit(quiet=True) == 0, capsys.readouterr().out


def test_accumulation_registers_outside_asm_are_reported():
    C = _load()
    text = "\n".join(["_Z13gemm_asm_quadv:", "\tv_mov_b32 v1, 0", "\t;;#ASMSTART", "\tv_accvgpr_write_b32 a0, 0", "\t;;#ASMEND",
                      "\tv_accvgpr_write_b32 a17, v3 ; 4-byte Folded Spill", "\t.amdhsa_accum_offset 256", "_Z5otherv:",
                      "\tv_accvgpr_read_b32 v0, a3"])
    assert C.accumulation_registers_outside_asm(text, "gemm_asm_quad") == ["_Z13gemm_asm_quadv: v_accvgpr_write_b32 a17, v3"]


def test_build_refuses_decode_kernels_that_spill():
    """The decode kernels count their memory requests by hand; a spilled register's store and reload go through the same
    counter.  build.py reads the compiler's resource remarks for gemm_thin.hip and refuses to link when one of those
    kernels uses scratch: here the reader of those remarks, on a made-up excerpt."""
    spec = importlib.util.spec_from_file_location("lowp_build", os.path.join(os.path.dirname(CSRC), "build.py"))
    B = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(B)
    line = "gemm_thin.hip:525:1: remark: {} [-Rpass-analysis=kernel-resource-usage]"
    def kernel(name, scratch):
        return [line.format(f"Function Name: {name}"), line.format("    VGPRs: 128"),
                line.format(f"    ScratchSize [bytes/lane]: {scratch}"), line.format("    VGPRs Spill: 0")]
    remarks = "\n".join(kernel("_ZN12_GLOBAL__N_114gemm_thin_rowsILi0ELi7ELi9ELi2ELb0EEEvPKh", 0)
                        + kernel("_ZN12_GLOBAL__N_115gemm_thin_ring2ILi2ELi7ELi4ELi3ELi3ELb1EEEvPKh", 24)
                        + kernel("_ZN12_GLOBAL__N_19some_otherEvPKh", 64))
    pattern = B.SPILL_AUDIT["gemm_thin.hip"]
    assert B._kernels_with_scratch(remarks, pattern) == [("_ZN12_GLOBAL__N_115gemm_thin_ring2ILi2ELi7ELi4ELi3ELi3ELb1EEEvPKh", 24)]
    assert B._kernels_with_scratch(remarks.replace(": 24", ": 0"), pattern) == []
