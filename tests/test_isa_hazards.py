"""The generated gfx950 assembly of the GEMM kernels is free of the wait-state hazards that the
compiler does not check inside asm statements, and the streaming kernels issue their loads back to
back (see isa_check.py).  CPU only: hipcc cross-compiles."""
import importlib.util
import os
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_spec = importlib.util.spec_from_file_location(
    "mi355q_isa_check", os.path.join(ROOT, "tests", "isa_check.py"))
isa_check = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(isa_check)


def test_scanner_flags_scalar_register_written_too_late():
    text = """
	v_readfirstlane_b32 s30, v68
	v_lshl_add_u32 v68, v189, 3, v172
	;;#ASMSTART
	s_mov_b32 m0, s5
	s_nop 0
	buffer_load_dwordx4 v1, s[28:31], 0 offen lds
	;;#ASMEND
"""
    found = isa_check.scan(text)
    assert len(found) == 1 and "s[30]" in found[0]


def test_scanner_accepts_enough_wait_states():
    late_enough = """
	v_readfirstlane_b32 s30, v68
	v_add_u32_e32 v1, v2, v3
	v_add_u32_e32 v1, v2, v3
	v_add_u32_e32 v1, v2, v3
	;;#ASMSTART
	s_mov_b32 m0, s5
	s_nop 0
	buffer_load_dwordx4 v1, s[28:31], 0 offen lds
	;;#ASMEND
"""
    nop_inside = """
	v_readfirstlane_b32 s30, v68
	;;#ASMSTART
	s_mov_b32 m0, s5
	s_nop 4
	buffer_load_dword v1, s[28:31], 0 offen lds
	;;#ASMEND
"""
    other_register = """
	v_readfirstlane_b32 s40, v68
	;;#ASMSTART
	s_mov_b32 m0, s5
	s_nop 0
	buffer_load_dwordx4 v1, s[28:31], 0 offen lds
	;;#ASMEND
"""
    scalar_write = """
	s_add_u32 s28, s28, s2
	;;#ASMSTART
	s_mov_b32 m0, s5
	s_nop 0
	buffer_load_dwordx4 v1, s[28:31], 0 offen lds
	;;#ASMEND
"""
    for text in (late_enough, nop_inside, other_register, scalar_write):
        assert isa_check.scan(text) == []


def test_scanner_flags_m0_used_at_once():
    text = """
	;;#ASMSTART
	s_mov_b32 m0, s5
	buffer_load_dwordx4 v1, s[28:31], 0 offen lds
	;;#ASMEND
"""
    assert any("M0" in f for f in isa_check.scan(text))


@pytest.mark.timeout(900)
def test_gemm_kernels_have_no_uncovered_hazard():
    sources = ["gemm_inst_kk.hip", "gemm_inst_km.hip", "gemm_inst_mk.hip", "gemm_inst_mm.hip", "w4_gemm.hip", "sdpa_kernels.hip"]
    with ThreadPoolExecutor(max_workers=6) as ex:
        texts = list(ex.map(isa_check.compile_to_isa, sources))
    sharing = 0
    for src, text in zip(sources, texts):
        assert text.count("#ASMSTART") > 100, f"{src}: the asm statements are gone?"
        assert isa_check.scan(text) == [], src
        shared, findings = isa_check.m0_sharing(text)
        assert findings == [], src
        sharing += shared
        # no kernel spills registers (a spill in a K loop shows as tens of MB of HBM traffic per launch), but for
        # two forms of the attention kernel that keep a few loop-invariant values there
        spills = isa_check.scratch_bytes(text)
        if src == "sdpa_kernels.hip":
            assert all("fp8_sdpa_fwd_kernel" in k and v <= 40 for k, v in spills.items()) and len(spills) <= 4, spills
        else:
            assert spills == {}, (src, spills)
    assert sharing > 0, "the kernels whose loads share a write of m0 are gone?"


def test_m0_sharing_scanner():
    good = """
	;;#ASMSTART
	s_mov_b32 m0, s5
	s_nop 0
	buffer_load_dwordx4 v1, s[28:31], 0 offen lds
	;;#ASMEND
	v_mfma_f32_16x16x128_f8f6f4 a[0:3], v[2:9], v[10:17], a[0:3]
	;;#ASMSTART
	buffer_load_dwordx4 v2, s[28:31], 0 offen offset:1024 lds
	;;#ASMEND
"""
    assert isa_check.m0_sharing(good) == (1, [])
    across_a_label = good.replace("\tv_mfma", ".LBB0_3:\n\tv_mfma")
    assert isa_check.m0_sharing(across_a_label)[1]
    compiler_write = good.replace("\tv_mfma", "\ts_mov_b32 m0, s9\n\tv_mfma")
    assert isa_check.m0_sharing(compiler_write)[1]


@pytest.mark.timeout(600)
def test_attention_block_loop_does_not_wait_for_its_own_prefetch():
    """The compiler places the wait for a load at its first use.  The query fragments of the attention kernels
    are loaded once and first used by the first MFMA of the block loop: left alone, that is a vmcnt(0) in every
    pass, which also waits for the K / V blocks the pass has just requested (global -> LDS loads share the
    counter).  The kernels name the fragments in front of the loop; here the basic block that ends in the first
    MFMA must hold no wait on vmcnt."""
    import re
    text = isa_check.compile_to_isa("sdpa_kernels.hip")
    seen = 0
    for name, body in re.findall(r"^(_ZN6mi355q\w+):.*?\n(.*?)s_endpgm", text, flags=re.S | re.M):
        if "fp8_sdpa_fwd_kernel" not in name and "fp8_sdpa_decode_kernel" not in name:
            continue
        lines = body.split("\n")
        first = next(k for k, line in enumerate(lines) if "v_mfma" in line)
        start = first
        while start > 0 and not lines[start].startswith(".LBB"):
            start -= 1
        assert not any("vmcnt" in line for line in lines[start:first]), name
        seen += 1
    assert seen >= 16


def test_memory_order_reads_a_kernel():
    text = """
_Z3foov:                                ; @_Z3foov
	global_load_dwordx4 v[2:5], v[0:1], off
	s_waitcnt vmcnt(0)
	global_load_dwordx4 v[6:9], v[0:1], off offset:16
	s_waitcnt vmcnt(1) lgkmcnt(0)
	buffer_store_dwordx2 v[2:3], v10, s[4:7], 0 offen
	s_endpgm
.Lfunc_end0:
"""
    assert isa_check.memory_order(text) == {"_Z3foov": "LWLwS"}


@pytest.mark.timeout(600)
def test_streaming_kernels_issue_their_loads_back_to_back():
    """Every bandwidth-tuned streaming kernel issues all its independent loads before its first
    full wait (a full wait before each load is what a divergent branch around it produces)."""
    order = isa_check.memory_order(isa_check.compile_to_isa("cast_kernels.hip"))
    seen = 0
    for name, seq in order.items():
        if "cast_to_fp8_vec8" in name or "cast_from_fp8_vec" in name:
            loads = 4                                   # U
        elif "quantize_rows_kernel" in name:            # VPT is the last template argument
            loads = int(name.split("ELi")[-1].split("E")[0]) * (2 if "silu_mul" in name else 1)
        else:
            continue
        seen += 1
        first_full_wait = seq.find("W") if "W" in seq else len(seq)
        assert seq[:first_full_wait].count("L") >= loads, (name, seq)
    assert seen >= 60


def test_exchange_order_reads_a_kernel():
    text = """
_Z3barv:                                ; @_Z3barv
	global_store_dwordx2 v[0:1], v[2:3], off sc1
	s_waitcnt vmcnt(0)
	s_barrier
	global_atomic_add v4, v[0:1], v5, off sc0
	s_waitcnt vmcnt(0)
	s_barrier
	s_barrier
	global_load_dwordx2 v[6:7], v[0:1], off sc1
	buffer_wbl2 sc1
	s_endpgm
.Lfunc_end0:
"""
    assert isa_check.exchange_order(text) == {"_Z3barv": "SWBAWBLF"}


@pytest.mark.timeout(900)
def test_partial_results_are_exchanged_by_device_scope_accesses_in_order():
    """Workgroups that split one reduction (the K parts of the 4-bit GEMMs, the key splits of the decoding attention
    kernel) hand their partial results over without a fence: device-scope relaxed atomic stores (sc1: written through
    to where every XCD sees them), a wait until they are acknowledged, a workgroup barrier, the ticket; whoever draws
    the last ticket passes a barrier and reads with device-scope loads (sc1).  The generated code has to keep that
    order and those bits, and must hold no cache-wide write-back or invalidate."""
    import re
    with ThreadPoolExecutor(max_workers=2) as ex:
        texts = list(ex.map(isa_check.compile_to_isa, ["w4_gemm.hip", "sdpa_kernels.hip"]))
    for src, text, least in zip(["w4_gemm.hip", "sdpa_kernels.hip"], texts, [12, 2]):
        orders = isa_check.exchange_order(text)
        assert len(orders) >= least, src
        for name, seq in orders.items():
            assert "F" not in seq, name
            assert seq.count("A") == 1, name
            # partial results stored, acknowledged, barrier, ticket (and its return to zero by the last one), barrier, read
            assert re.search(r"S+WBAW?S?BL+", seq), (name, seq)
