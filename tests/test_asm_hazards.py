"""The direct-to-LDS tiles issue their LDS fragment reads from inline asm, which the compiler cannot
see are still in flight.  This test compiles those files to assembly with the library's own flags
and checks, instruction by instruction, that nothing touches a register such a read is still
filling (tests/asm_inflight.py).  A kernel that fails this check can fault: a late write-back into
a register the compiler has reused for an index corrupts an address.
"""
import concurrent.futures
import os
import subprocess

import pytest

import asm_inflight
from cuasr_amd import build as B

FILES = ["direct_f32.hip", "direct_i32.hip", "direct_u32.hip", "direct_f64.hip", "mfma_direct_f32.hip", "mfma_direct_f64.hip",
         "mfma_direct_narrow.hip", "fwgemm.hip"]


def _listing(src, out_dir):
    out = os.path.join(out_dir, src[:-4] + ".s")
    extra = [f for k, v in B.PER_FILE.items() if src.startswith(k) for f in v]
    cmd = [B.HIPCC] + B.FLAGS + extra + ["-S", "--cuda-device-only", os.path.join(B.CSRC, src), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    with open(out) as f:
        return f.read()


# ---- the checker itself, on listings small enough to read ------------------------------------

GOOD = """
_Zgood:
	;;#ASMSTART
	ds_read_b64 v[4:5], v20 offset:0
	;;#ASMEND
	;;#ASMSTART
	ds_read_b64 v[6:7], v20 offset:256
	;;#ASMEND
	v_add_f32_e32 v30, v31, v32
	s_waitcnt lgkmcnt(1)
	v_add_f32_e32 v30, v4, v5
	s_waitcnt lgkmcnt(0)
	v_add_f32_e32 v30, v6, v7
	s_endpgm
"""

# the second read is still in flight when v6 is reused as scratch
REUSED = GOOD.replace("v_add_f32_e32 v30, v31, v32", "v_lshrrev_b32_e32 v6, 4, v0")
# waits for the older read only, then consumes the younger one
EARLY = GOOD.replace("s_waitcnt lgkmcnt(0)\n", "")
# a loop whose last iteration leaves a read in flight that nothing after the loop waits for
UNDRAINED = """
_Zloop:
.LBB0_1:
	s_waitcnt lgkmcnt(0)
	v_add_f32_e32 v30, v4, v5
	;;#ASMSTART
	ds_read_b64 v[4:5], v20 offset:0
	;;#ASMEND
	s_cbranch_scc1 .LBB0_1
	v_and_b32_e32 v4, 15, v0
	s_endpgm
"""
DRAINED = UNDRAINED.replace("\tv_and_b32_e32 v4", "\ts_waitcnt lgkmcnt(0)\n\tv_and_b32_e32 v4")
# a read issued on one side of a branch is in flight where the two paths meet
BRANCH = """
_Zbranch:
	s_cbranch_scc1 .LBB0_2
	;;#ASMSTART
	ds_read_b64 v[4:5], v20 offset:0
	;;#ASMEND
	s_branch .LBB0_3
.LBB0_2:
	v_mov_b32_e32 v4, 0
.LBB0_3:
	v_add_f32_e32 v30, v4, v4
	s_endpgm
"""
# the compiler's own reads (outside the asm markers) only count for the wait arithmetic
COMPILER_READ = """
_Zown:
	;;#ASMSTART
	ds_read_b64 v[4:5], v20 offset:0
	;;#ASMEND
	ds_read_b64 v[8:9], v21
	s_waitcnt lgkmcnt(1)
	v_add_f32_e32 v30, v4, v5
	v_mov_b32_e32 v8, 0
	s_endpgm
"""


@pytest.mark.parametrize("name,text,bad", [
    ("good", GOOD, 0), ("reused", REUSED, 1), ("early", EARLY, 1), ("undrained", UNDRAINED, 1),
    ("drained", DRAINED, 0), ("branch", BRANCH, 1), ("compiler_read", COMPILER_READ, 0)])
def test_checker_on_small_listings(name, text, bad):
    res = asm_inflight.check_listing(text, "")
    assert len(res) == 1
    findings = next(iter(res.values()))
    assert len(findings) == bad, findings


def test_wait_for_more_than_is_in_flight():
    text = GOOD.replace("s_waitcnt lgkmcnt(1)", "s_waitcnt lgkmcnt(5)\n\ts_waitcnt lgkmcnt(1)")
    assert next(iter(asm_inflight.check_listing(text, "").values())) == []


# ---- the library's kernels ---------------------------------------------------------------------

def test_no_instruction_touches_a_register_an_asm_lds_read_is_filling(tmp_path):
    with concurrent.futures.ThreadPoolExecutor(len(FILES)) as ex:
        texts = list(ex.map(lambda s: _listing(s, str(tmp_path)), FILES))
    kernels = 0
    for src, text in zip(FILES, texts):
        # every kernel of the direct_*.hip files: the plain tiles and the stream-K form, which inlines the tile's
        # segment twice inside run-time loops and so gets a register allocation of its own
        res = asm_inflight.check_listing(text, "mfma_narrow_kernel" if src.startswith("mfma_direct_narrow") else "gemm_mfma_direct" if src.startswith("mfma") else "fwgemm_direct_kernel" if src.startswith("fwgemm") else "_kernel")
        assert res, f"{src}: no kernels found in the listing"
        if src in ("direct_f32.hip", "direct_i32.hip", "direct_u32.hip"):
            assert any("streamk_kernel" in k for k in res), f"{src}: no stream-K kernel was checked"
            assert any("srgemm_kernel" in k for k in res), f"{src}: no plain tile was checked"
        kernels += len(res)
        bad = {k: v[:3] for k, v in res.items() if v}
        assert not bad, f"{src}: {len(bad)} kernels touch in-flight registers, e.g. {next(iter(bad.items()))}"
        # the check must have seen asm-issued reads, or it checked nothing
        assert text.count("ds_read") > 0 and ";;#ASMSTART" in text
    assert kernels >= 100
