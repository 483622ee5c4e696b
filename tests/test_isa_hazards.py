"""The attention kernels' score MFMAs are inline assembly: the compiler neither knows that a read of
their result needs wait states nor keeps its own register copies away from them.  This test emits
the gfx950 assembly of those translation units (hipcc cross-compiles, no GPU needed) with the
library's own flags and checks every VGPR-destination MFMA for a too-early access (isa_hazards.py)."""
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

import isa_hazards as H
from diffgemma_amd import build

UNITS = {"attn_mfma.hip": 100, "attn_wsplit.hip": 50}   # file -> at least this many assembly MFMAs expected


def _emit(src, out_dir):
    out = out_dir / (src + ".s")
    cmd = [build.hipcc_path(), *build.HIP_FLAGS, "-S", "--cuda-device-only", str(build.CSRC / src), "-o", str(out)]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    return out.read_text()


@pytest.fixture(scope="module")
def asm(tmp_path_factory):
    if shutil.which("hipcc") is None and not build.hipcc_path():
        pytest.skip("no hipcc")
    d = tmp_path_factory.mktemp("isa")
    with ThreadPoolExecutor(len(UNITS)) as ex:
        return dict(zip(UNITS, ex.map(lambda s: _emit(s, d), UNITS)))


@pytest.mark.parametrize("unit", sorted(UNITS))
def test_no_access_to_a_score_mfma_result_inside_its_wait_states(asm, unit):
    text = asm[unit]
    assert H.count_vgpr_mfmas(text) >= UNITS[unit], "the checker no longer sees the assembly MFMAs"
    findings = H.check(text)
    assert not findings, "\n".join(str(f) for f in findings[:10])


def test_the_checker_sees_a_copy_behind_an_mfma():
    # what a compiler-made copy of the accumulator between two score MFMAs looks like
    bad = """
kernel_a:
	v_mfma_f32_32x32x16_bf16 v[18:33], v[4:7], v[74:77], v[18:33]
	s_nop 0
	v_mov_b64_e32 v[2:3], v[18:19]
	v_mfma_f32_32x32x16_bf16 v[2:17], v[86:89], v[78:81], v[2:17]
	s_nop 15
	s_nop 7
	v_max_f32_e32 v4, v2, v3
	s_endpgm
"""
    f = H.check(bad)
    assert len(f) == 1 and "v_mov_b64" in f[0].reader
    # enough distance, directly or through a branch, is accepted; too little behind a branch is not
    ok = bad.replace("s_nop 0\n", "s_nop 15\n\ts_nop 3\n")
    assert not H.check(ok)
    branchy = """
kernel_b:
	v_mfma_f32_32x32x16_bf16 v[2:17], v[86:89], v[78:81], v[2:17]
	s_cbranch_scc1 .LBB0_2
	s_nop 15
	s_nop 7
	v_max_f32_e32 v4, v2, v3
	s_endpgm
.LBB0_2:
	v_add_f32_e32 v40, v17, v17
	s_endpgm
"""
    f = H.check(branchy)
    assert len(f) == 1 and "v_add_f32" in f[0].reader
    # accumulation registers are walked too: the compiler pads its own reads, an assembly read it does not
    acc = "k:\n\tv_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[4:7], a[0:15]\n{}\tv_accvgpr_read_b32 v9, a0\n\ts_endpgm\n"
    assert len(H.check(acc.format("\ts_nop 3\n"))) == 1
    assert not H.check(acc.format("\ts_nop 11\n"))
    # another MFMA in between occupies the matrix pipe for its eight passes
    assert not H.check(acc.format("\tv_mfma_f32_32x32x16_bf16 a[16:31], v[0:3], v[4:7], a[16:31]\n\ts_nop 3\n"))
