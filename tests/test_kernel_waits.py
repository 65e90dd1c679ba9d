"""What the hand-counted waits of the kernels with written-out MFMAs and LDS reads promise, checked in the
compiler's output (no GPU: hipcc cross-compiles to assembly).

attention_wide_bf16.hip once left two LDS reads without a taker (the prologue's last V fragment, and the
fragments the last pass asks for the pass that never comes): the compiler gave their registers to other values
while the reads were out, and under load on LDS (a second block on the compute unit) the fragments arrived on top of
those values.  tests/asm_audit.py finds that pattern, an MFMA result read too early, and a counted wait on direct
loads that leaves a needed load in flight."""
import os
import shutil
import subprocess

import pytest

import asm_audit
from allpaca_amd.kernels import build

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
pytestmark = pytest.mark.skipif(not os.path.isfile(HIPCC), reason="hipcc is needed to compile to assembly")

SOURCES = {  # source -> LDS stages its counted waits rotate through
    "attention_wide_bf16.hip": 4,
    "gemm_direct_bf16.hip": 4,
    "gemm_wide_bf16.hip": 0,
}


def assembly(tmp_path, name):
    src = os.path.join(build.CSRC, name)
    out = tmp_path / (name + ".s")
    cmd = [HIPCC, *build.flags_for(src), "-I", build.CSRC, "-S", "--cuda-device-only", src, "-o", str(out)]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert p.returncode == 0, p.stdout
    return asm_audit.parse(str(out))


@pytest.mark.parametrize("name", sorted(SOURCES))
def test_no_register_is_touched_before_its_read_or_mfma_is_done(tmp_path, name):
    functions = assembly(tmp_path, name)
    assert functions
    counted = 0
    for fn, items in functions.items():
        found = asm_audit.audit(fn, items, verbose=False)
        assert not found, f"{fn}: " + "; ".join(f"{p[1]} {p[2]}" for p in list(found.values())[:4])
        if SOURCES[name]:
            for a, b, left, behind in asm_audit.direct_load_counts(items, SOURCES[name]):
                counted += 1
                assert behind >= left, (f"{fn}: the wait in loop {a}-{b} leaves {left} loads in flight, but only "
                                        f"{behind} were issued behind the last direct load of the stage read next")
    if SOURCES[name]:
        assert counted, "no loop with a counted wait on direct loads was found: the rule checks nothing"


LATE_FRAGMENT = """
_Zkernel:
	ds_read_b128 v[4:7], v1 offset:0
	ds_read_b128 v[8:11], v1 offset:1024
	s_waitcnt lgkmcnt(1)
	v_mfma_f32_32x32x16_bf16 v[16:31], v[4:7], v[12:15], 0
	v_mov_b32_e32 v8, 0
	s_endpgm
.Lfunc_end0:
"""
EARLY_RESULT = """
_Zkernel:
	v_mfma_f32_32x32x16_bf16 v[16:31], v[4:7], v[12:15], 0
	v_mfma_f32_32x32x16_bf16 a[0:15], v[4:7], v[12:15], a[0:15]
	v_add_f32_e32 v1, v16, v16
	s_nop 3
	v_accvgpr_read_b32 v2, a3
	s_nop 15
	v_accvgpr_read_b32 v2, a4
	s_endpgm
.Lfunc_end0:
"""


def test_the_audit_finds_what_it_is_for(tmp_path):
    def found(text):
        path = tmp_path / "t.s"
        path.write_text(text)
        (items,) = asm_audit.parse(str(path)).values()
        return asm_audit.audit("t", items, verbose=False)

    late = found(LATE_FRAGMENT)
    assert len(late) == 1 and "v_mov_b32_e32 v8" in list(late.values())[0][2]
    early = [p[2] for p in found(EARLY_RESULT).values()]
    # v16 is read 8 wait states behind its MFMA (the second MFMA goes out when the first has made its 8 passes): too
    # early by the table's 11; a3 four more behind that is too early for the second MFMA; a4 after s_nop 15 is not
    assert any("v_add_f32_e32 v1, v16" in t for t in early)
    assert any("a3" in t for t in early) and not any("a4" in t for t in early)
