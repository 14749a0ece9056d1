"""The build-time scan for register spills that lose lanes (int_flashattention_amd/spill_check.py) on hand-made assembly:
the two placements it must report and the ones it must leave alone."""
import importlib.util
import os

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("spill_check", os.path.join(HERE, "..", "int-flashattention_amd", "spill_check.py"))
spill_check = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(spill_check)

HEAD = "_ZN5intfa4kernEv:\n\ts_load_dwordx2 s[0:1], s[4:5], 0x0\n"
SPILL = "\tscratch_store_dword off, v1, off offset:4 ; 4-byte Folded Spill\n"
RELOAD = "\tscratch_load_dword v1, off, off offset:4 ; 4-byte Folded Reload\n"


def test_spill_before_the_exec_restore_of_a_join_block_is_reported():
    asm = (HEAD + "\ts_and_saveexec_b64 s[2:3], vcc\n\ts_cbranch_execz .LBB0_2\n; %bb.1:\n\tglobal_load_dword v5, v[2:3], off\n"
           ".LBB0_2:\n" + SPILL + "\ts_or_b64 exec, exec, s[2:3]\n\tv_add_f32_e32 v0, v0, v1\n\ts_endpgm\n")
    found = spill_check.scan(asm)
    assert found and all("_ZN5intfa4kernEv" in f for f in found)
    assert any("before exec is restored" in f for f in found)


def test_reload_before_the_exec_restore_of_a_join_block_is_reported():
    asm = (HEAD + "\ts_and_saveexec_b64 s[2:3], vcc\n\ts_cbranch_execz .LBB0_2\n; %bb.1:\n\tv_mov_b32_e32 v5, 0\n"
           ".LBB0_2:\n" + RELOAD + "\ts_or_b64 exec, exec, s[2:3]\n\ts_endpgm\n")
    assert any("before exec is restored" in f for f in spill_check.scan(asm))


def test_spill_store_inside_a_masked_region_is_reported_and_a_reload_there_is_not():
    store = HEAD + "\ts_and_saveexec_b64 s[2:3], vcc\n" + SPILL + "\ts_or_b64 exec, exec, s[2:3]\n\ts_endpgm\n"
    assert any("while exec is narrowed" in f for f in spill_check.scan(store))
    # a value reloaded for the active lanes and used by them is how the compiler serves a masked region
    reload = (HEAD + "\ts_and_saveexec_b64 s[2:3], vcc\n\ts_cbranch_execz .LBB0_2\n; %bb.1:\n" + RELOAD +
              "\tglobal_store_dword v[2:3], v1, off\n.LBB0_2:\n\ts_or_b64 exec, exec, s[2:3]\n\ts_endpgm\n")
    assert spill_check.scan(reload) == []


def test_spills_with_the_full_mask_and_scalar_branches_pass():
    asm = (HEAD + SPILL + "\ts_cmp_lg_u32 s6, 0\n\ts_cbranch_scc1 .LBB0_2\n; %bb.1:\n" + SPILL + RELOAD +
           ".LBB0_2:\n" + RELOAD + "\tv_add_f32_e32 v0, v0, v1\n\ts_endpgm\n")
    assert spill_check.scan(asm) == []
    # the mask restored before the spill code of the join block
    ok = (HEAD + "\ts_and_saveexec_b64 s[2:3], vcc\n\ts_cbranch_execz .LBB0_2\n; %bb.1:\n\tv_mov_b32_e32 v5, 0\n"
          ".LBB0_2:\n\ts_or_b64 exec, exec, s[2:3]\n" + SPILL + RELOAD + "\ts_endpgm\n")
    assert spill_check.scan(ok) == []


def test_a_mask_narrowed_ahead_of_the_program_end_does_not_reach_the_code_behind_it():
    """A guarded store and `s_endpgm` close one path; the block behind it is entered by branches with their own mask."""
    asm = (HEAD + "\ts_cbranch_scc1 .LBB0_3\n; %bb.1:\n\ts_and_b64 exec, exec, s[2:3]\n\ts_cbranch_execz .LBB0_2\n; %bb.4:\n"
           "\tglobal_store_dword v[2:3], v1, off\n.LBB0_2:\n\ts_endpgm\n.LBB0_3:\n" + SPILL + RELOAD + "\ts_endpgm\n")
    assert spill_check.scan(asm) == []
    # ... while the same store on the fall-through side of the narrowing is still reported
    bad = HEAD + "\ts_and_b64 exec, exec, s[2:3]\n" + SPILL + "\ts_endpgm\n"
    assert any("while exec is narrowed" in f for f in spill_check.scan(bad))
