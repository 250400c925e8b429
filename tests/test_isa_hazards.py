"""The generated code of the kernels whose MFMAs are inline assembly keeps the wait states between
an MFMA and the first ordinary access to its result (see tests/isa_lint.py).  Compiles
csrc/qgemm_dma.hip (about a minute and a half) and csrc/conv.hip to assembly, no GPU needed."""
import os
import shutil
import subprocess

import pytest

from tests import isa_lint

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def test_lint_finds_a_read_right_behind_an_assembly_mfma(tmp_path):
    listing = tmp_path / "sample.s"
    listing.write_text("""
_Z6samplev:
	;;#ASMSTART
	v_mfma_i32_16x16x64_i8 a[0:3], v[0:3], v[4:7], a[0:3]
	;;#ASMEND
	s_nop 3
	v_accvgpr_read_b32 v8, a1
	;;#ASMSTART
	v_mfma_f32_32x32x64_f8f6f4 a[16:31], v[0:7], v[8:15], a[16:31]
	;;#ASMEND
	s_nop 7
	s_nop 7
	s_nop 2
	scratch_store_dwordx4 off, a[28:31], off
	v_mfma_i32_16x16x64_i8 a[4:7], v[0:3], v[4:7], a[4:7]
	v_accvgpr_read_b32 v9, a5
""")
    seen, hazards = isa_lint.scan(str(listing))
    # the int8 read comes 4 + 1 wait states behind (7 needed); the fp8 store 19 behind (19 needed: fine);
    # the last MFMA is the compiler's own (outside an assembly region) and not this scan's business
    assert seen == 2
    assert len(hazards) == 1 and "a1" in hazards[0]


def test_lint_finds_a_copy_of_a_loaded_register_in_front_of_its_wait(tmp_path):
    listing = tmp_path / "loads.s"
    listing.write_text("""
_Z5loadsv:
	;;#ASMSTART
	global_load_ushort v9, v1, s[2:3] nt
	;;#ASMEND
	;;#ASMSTART
	global_load_dwordx4 v[4:7], v0, s[2:3] offset:128 nt
	;;#ASMEND
	v_add_u32_e32 v8, 1, v0
	v_mov_b32_e32 v10, v9
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_and_b32_e32 v11, 15, v9
	v_mov_b32_e32 v12, v5
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_mov_b32_e32 v13, v5
	s_endpgm
""")
    seen, hazards = isa_lint.scan_assembly_loads(str(listing))
    # v9 is copied before its wait (vmcnt(1) covers it: one load behind it) and read properly after;
    # v5 is read once before vmcnt(0) and once after
    assert seen == 2
    assert len(hazards) == 2 and "v9" in hazards[0] and "v5" in hazards[1]


_LISTINGS = {}


def _listing(tmp_path, source):
    # one compilation per source and test session (qgemm_dma.hip takes a minute and a half)
    if source in _LISTINGS and os.path.exists(_LISTINGS[source]):
        return _LISTINGS[source]
    out = tmp_path / (source + ".s")
    cmd = [HIPCC, "-O3", "-std=c++17", "--offload-arch=gfx950", "-I" + os.path.join(ROOT, "include"),
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only",
           "-o", str(out), os.path.join(ROOT, "amdmigraphx_amd", "csrc", source)]
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=900)
    _LISTINGS[source] = str(out)
    return str(out)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_direct_convolution_kernel_keeps_its_wait_states(tmp_path):
    seen, hazards = isa_lint.scan(_listing(tmp_path, "conv.hip"), only="conv_direct")
    # 16 MFMAs per K step body, 24 int8 instantiations (4 result types, vector stores or not, 3 ring
    # depths); the fp8 ones use the compiler's own MFMAs
    assert seen >= 16 * 24
    assert hazards == [], hazards[:5]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_reordered_int4_gemv_reads_no_load_before_its_wait(tmp_path):
    seen, hazards = isa_lint.scan_assembly_loads(_listing(tmp_path, "w4a16_prepacked.hip"), only="w4p_gemv_kernel")
    # per kernel: the activation loads and, in each of the two bodies, five loads per block
    assert seen >= 24 * (1 + 2 * 5)
    assert hazards == [], hazards[:5]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_four_wave_kernels_keep_their_wait_states(tmp_path):
    seen, hazards = isa_lint.scan(_listing(tmp_path, "qgemm_dma.hip"))
    # 64 (int8) or 16 (fp8) MFMAs per slab body, several bodies per kernel, 28 kernels
    assert seen > 5000
    assert hazards == [], hazards[:5]


def test_lint_finds_a_load_right_behind_an_assembly_m0_write(tmp_path):
    listing = tmp_path / "m0.s"
    listing.write_text("""
_Z2m0v:
	;;#ASMSTART
	s_add_i32 m0, s4, 0x1000
	global_load_lds_dwordx4 v1, s[0:1]
	v_mfma_i32_16x16x64_i8 a[0:3], v[0:3], v[4:7], a[0:3]
	s_add_i32 m0, s4, 0x2000
	v_mfma_i32_16x16x64_i8 a[4:7], v[0:3], v[4:7], a[4:7]
	global_load_lds_dwordx4 v2, s[0:1]
	;;#ASMEND
	s_mov_b32 m0, s5
	global_load_lds_dwordx4 v3, s[0:1]
""")
    seen, hazards = isa_lint.scan_m0_writes(str(listing))
    # the first load follows its M0 write directly, the second has an MFMA between; the last pair is
    # the compiler's own code (outside an assembly region): the compiler knows that hazard
    assert seen == 2
    assert len(hazards) == 1 and "line 5" in hazards[0]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_four_wave_kernels_keep_a_wait_state_behind_their_m0_writes(tmp_path):
    seen, hazards = isa_lint.scan_m0_writes(_listing(tmp_path, "qgemm_dma.hip"))
    # 8 M0 writes per slab of a twelve-slab trip, in each of the 30 four-wave kernels
    assert seen >= 30 * 96
    assert hazards == [], hazards[:5]
