"""The build-time check for the MFMA pairing that gfx950 needs wait states for and the compiler does not add
(jaxrwkv_amd/mfma_hazard.py): the scanner on hand-written sequences, and the assembly of every kernel as built."""
import glob
import os

import pytest

from jaxrwkv_amd import build as b
from jaxrwkv_amd import mfma_hazard as mh

K32 = "\tv_mfma_f32_16x16x32_f16 v[50:53], v[26:29], v[58:61], v[54:57]\n"
K16 = "\tv_mfma_f32_16x16x16_f16 v[50:53], v[40:41], v[20:21], v[50:53]\n"
FILL = "\ts_add_i32 s47, s8, 0\n\tv_add3_u32 v66, s47, v103, v105\n\tv_readfirstlane_b32 s44, v117\n"


def test_the_sequence_that_failed_on_the_gpu_is_reported():
    found = mh.scan(K32 + FILL + K16)
    assert [(w, a, c) for w, a, c, _ in found] == [(3, "v_mfma_f32_16x16x32_f16", "v_mfma_f32_16x16x16_f16")]
    with pytest.raises(RuntimeError, match="fewer than 8 wait states"):
        mh.check(K32 + FILL + K16, "example")


def test_wait_states_count_nops_and_a_fence_passes():
    assert mh.scan(K32 + FILL + "\ts_nop 1\n" + K16)[0][0] == 5
    mh.check(K32 + FILL + "\t;;#ASMSTART\n\ts_nop 7\n\t;;#ASMEND\n" + K16, "example")


def test_same_opcode_chains_and_overwritten_results_are_not_reported():
    same = K32 + "\tv_mfma_f32_16x16x32_f16 v[50:53], v[30:33], v[58:61], v[50:53]\n"
    assert mh.scan(same) == []
    overwritten = K32 + "\tv_mov_b32_e32 v51, 0\n" + K16            # no longer the MFMA's result as a whole
    assert mh.scan(overwritten) == []


def test_a_label_between_the_two_makes_the_distance_unknown():
    found = mh.scan(K32 + FILL * 4 + ".LBB0_7:\n" + K16)
    assert found[0][0] is None and mh.violations(K32 + FILL * 4 + ".LBB0_7:\n" + K16)


def test_every_built_kernel_keeps_mixed_opcode_accumulations_apart():
    """The assembly that `jaxrwkv_amd.build` leaves next to the objects; built here when it is missing or stale."""
    objdir = os.path.join(b.HERE, "build")
    stale = [s for s in b.SOURCES
             if not os.path.exists(os.path.join(objdir, s[:-4] + ".s"))
             or os.path.getmtime(os.path.join(objdir, s[:-4] + ".s")) < max(
                 os.path.getmtime(p) for p in glob.glob(os.path.join(b.CSRC, "*.h")) + [os.path.join(b.CSRC, s)])]
    if stale:
        if not os.path.exists(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")):
            pytest.skip("no hipcc to produce the assembly")
        b.build(verbose=False)
    mixed = 0
    for s in b.SOURCES:
        with open(os.path.join(objdir, s[:-4] + ".s")) as f:
            text = f.read()
        mh.check(text, s)
        mixed += len(mh.scan(text))
    assert mixed >= 2, "the WKV7 forward consumer has two such accumulations: the scanner no longer sees them"
