"""The build's check of the code generated around hand-scheduled loads: it passes on what a
good build looks like and names each kind of break."""
import os

import pytest

from ferrum_amd import build, isa_check

GOOD = """
	.text
_Z6kernelv:
	s_load_dwordx2 s[0:1], s[4:5], 0x0
	;;#ASMSTART
	global_load_dwordx2 v[4:5], v[2:3], off
	;;#ASMEND
	v_add_u32_e32 v9, v8, v7
	;;#ASMSTART
	s_mov_b32 m0, s3
	global_load_lds_dwordx4 v[2:3], off
	;;#ASMEND
	s_add_u32 s2, s2, 1
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mov_b32_e32 v6, v4
	global_load_dword v10, v[2:3], off
	s_endpgm
.Lfunc_end0:
	.amdhsa_kernel _Z6kernelv
		.amdhsa_private_segment_fixed_size 0
	.end_amdhsa_kernel
"""


def test_a_clean_kernel_passes():
    assert isa_check.violations(GOOD) == []


@pytest.mark.parametrize("old,new,message", [
    # a copy of the destination before the wait
    ("v_add_u32_e32 v9, v8, v7", "v_mov_b32_e32 v9, v5", "touches registers loaded"),
    # a load of the compiler's own between the counted loads and the wait
    ("s_add_u32 s2, s2, 1", "global_load_dword v11, v[2:3], off", "hand-counted wait"),
    # the compiler keeps something of its own in M0
    ("s_add_u32 s2, s2, 1", "s_mov_b32 m0, s9", "M0 is used outside"),
    ("s_add_u32 s2, s2, 1", "ds_gws_init v0 gds", None),
    # spill space in a kernel with such loads
    (".amdhsa_private_segment_fixed_size 0", ".amdhsa_private_segment_fixed_size 64", "bytes of scratch"),
    # a register load that no hand-placed wait follows
    ("s_waitcnt vmcnt(1)", "s_nop 0", "no hand-placed s_waitcnt"),
])
def test_each_break_is_named(old, new, message):
    assert old in GOOD
    found = isa_check.violations(GOOD.replace(old, new, 1), "x.hip")
    if message is None:
        assert found == []      # an instruction that does not touch M0 or the registers is no break
    else:
        assert any(message in v for v in found), found
        assert all(v.startswith("x.hip:") for v in found)


def test_requests_with_a_scalar_base_are_hand_loads_too():
    # `global_load_lds_dwordx4 vOFFSET, s[BASE]`: one vector register of lane offsets, the base in scalar registers
    scalar = GOOD.replace("global_load_lds_dwordx4 v[2:3], off", "global_load_lds_dwordx4 v14, s[8:9]", 1)
    assert scalar != GOOD and isa_check.violations(scalar) == []
    broken = scalar.replace("s_add_u32 s2, s2, 1", "global_load_dword v11, v[2:3], off", 1)
    assert any("hand-counted wait" in v for v in isa_check.violations(broken, "x.hip"))
    broken = scalar.replace("s_add_u32 s2, s2, 1", "s_mov_b32 m0, s9", 1)
    assert any("M0 is used outside" in v for v in isa_check.violations(broken, "x.hip"))


def test_a_store_may_stand_behind_a_request_into_lds_but_not_behind_a_register_load():
    # vmcnt counts stores too and everything retires in order: a store among the later operations only
    # lengthens the wait for a request into LDS.  Behind a load into registers it stays a break (the
    # scan cannot tell which of the two waits the author counted).
    store = "global_store_dwordx4 v[20:21], v[22:25], off"
    lds_only = GOOD.replace("global_load_dwordx2 v[4:5], v[2:3], off", "s_nop 0", 1)
    assert isa_check.violations(lds_only.replace("s_add_u32 s2, s2, 1", store, 1)) == []
    both = isa_check.violations(GOOD.replace("s_add_u32 s2, s2, 1", store, 1), "x.hip")
    assert any("hand-counted wait" in v for v in both), both
    # a load of the compiler's behind the same request is still named
    load = lds_only.replace("s_add_u32 s2, s2, 1", "global_load_dword v11, v[2:3], off", 1)
    assert any("hand-counted wait" in v for v in isa_check.violations(load, "x.hip"))


def test_the_release_is_read_from_hipcc_version_text():
    assert isa_check.hipcc_release("HIP version: 7.2.26015-fc0010cf6a\nAMD clang version 22") == "7.2.26015"
    assert isa_check.hipcc_release("nothing") == ""


def test_the_built_library_came_through_the_check():
    # the assembly texts the last build checked lie beside its objects; they pass, and they
    # do contain the statements the check is about
    texts = [os.path.join(build.OBJ_DIR, os.path.splitext(s)[0] + ".s") for s in isa_check.CHECKED_SOURCES]
    if not all(os.path.exists(t) for t in texts):
        pytest.skip("no build in this tree yet")
    for path in texts:
        with open(path) as f:
            asm = f.read()
        assert isa_check.violations(asm, os.path.basename(path)) == []
        assert "global_load_lds_dwordx4" in asm
