"""The kernels that issue MFMAs without wait states (inline asm, outside the compiler's hazard handling) keep
another MFMA between a vector write of an operand register and the MFMA that reads it.  The checker compiles
them to assembly and verifies that on every MFMA; its scanner is tested on small listings first."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def checker():
    spec = importlib.util.spec_from_file_location("check_mfma_hazards",
                                                  os.path.join(ROOT, "jax-gptq_amd", "check_mfma_hazards.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


MFMA = "v_mfma_f32_16x16x32_f16 a[0:3], v[10:13], v[20:23], a[0:3]"


def test_scanner_flags_a_write_directly_in_front(checker):
    n, found = checker.scan("\n".join(["v_pk_fma_f16 v23, v1, s0, v2", MFMA]))
    assert n == 1 and len(found) == 1
    n, found = checker.scan("\n".join(["v_perm_b32 v12, 0, v1, v2", "s_waitcnt lgkmcnt(0)", MFMA]))
    assert len(found) == 1                                   # one instruction between: one wait state


def test_scanner_accepts_wait_states_and_mfmas_between(checker):
    other = "v_mfma_f32_16x16x32_f16 a[4:7], v[30:33], v[40:43], a[4:7]"
    for between in (["s_nop 1"], [other], ["v_mov_b32_e32 v99, 0", "s_waitcnt vmcnt(0)"]):
        n, found = checker.scan("\n".join(["v_pk_fma_f16 v23, v1, s0, v2", *between, MFMA]))
        assert found == [], between
    # a write of some other register in front is no hazard; comments and labels are skipped
    n, found = checker.scan("\n".join(["v_pk_fma_f16 v24, v1, s0, v2", "; comment", ".LBB0_1:", MFMA]))
    assert n == 1 and found == []


def test_scanner_follows_a_loop_back_edge(checker):
    """A vector write of an operand register at the end of a loop body, an MFMA at the loop's head: the two are
    adjacent across the back edge only."""
    loop = ["s_mov_b32 s0, 0", ".LBB0_1:", MFMA, "s_add_i32 s0, s0, 1", "s_cmp_lt_i32 s0, 8",
            "v_pk_fma_f16 v21, v1, s0, v2", "s_cbranch_scc1 .LBB0_1", "s_endpgm"]
    n, found = checker.scan("\n".join(loop))
    assert n == 1 and len(found) == 1
    # wait states at the head of the loop, or an MFMA as the last instruction of the body, clear it
    ok1 = loop[:2] + ["s_nop 1"] + loop[2:]
    other = "v_mfma_f32_16x16x32_f16 a[4:7], v[30:33], v[40:43], a[4:7]"
    ok2 = loop[:6] + [other] + loop[6:]
    for listing in (ok1, ok2):
        n, found = checker.scan("\n".join(listing))
        assert found == [], listing
    # nothing falls through an unconditional branch: the write in front of it reaches the label's code only
    skip = ["v_pk_fma_f16 v21, v1, s0, v2", "s_branch .LBB0_2", ".LBB0_3:", MFMA, ".LBB0_2:", "s_endpgm"]
    n, found = checker.scan("\n".join(skip))
    assert n == 1 and found == []


@pytest.mark.timeout(600)
def test_compiled_kernels_have_no_operand_hazard(checker):
    assert checker.check(verbose=False) == 0
