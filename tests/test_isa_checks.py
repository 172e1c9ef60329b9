"""The two checks of xlstm_amd/isa_check.py: on small listings that show what they look for, and on the assembly the
compiler really makes of the kernels (no GPU needed: hipcc cross-compiles)."""
import os

from xlstm_amd import isa_check

HAZARD = """
_Z6kernelv:
	v_readlane_b32 s44, v83, 26
	v_mul_lo_u32 v62, v65, s0
	v_readlane_b32 s45, v83, 27
	;;#ASMSTART
	global_load_ubyte v68, v62, s[44:45]
	;;#ASMEND
	s_endpgm
"""

HAZARD_FIXED = HAZARD.replace("\tglobal_load_ubyte", "\ts_nop 4\n\tglobal_load_ubyte")

COPY_IN_FLIGHT = """
_Z6kernelv:
	;;#ASMSTART
	global_load_dwordx2 v[4:5], v60, s[2:3]
	;;#ASMEND
	v_mov_b64_e32 v[26:27], v[4:5]
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	ds_write_b64 v67, v[26:27]
	s_endpgm
"""

COPY_AFTER_WAIT = """
_Z6kernelv:
	;;#ASMSTART
	global_load_dwordx2 v[4:5], v60, s[2:3]
	;;#ASMEND
	;;#ASMSTART
	global_load_dwordx2 v[6:7], v60, s[2:3]
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mov_b64_e32 v[26:27], v[4:5]
	s_endpgm
"""

TO_LDS = """
_Z6kernelv:
	;;#ASMSTART
	s_nop 4
	s_mov_b32 m0, s35
	s_nop 0
	buffer_load_dwordx4 v39, s[12:15], 0 offen lds
	;;#ASMEND
	v_mov_b32_e32 v39, 0
	s_endpgm
"""


def test_a_freshly_written_scalar_register_read_by_hand_issued_memory_instruction_is_found():
    assert len(isa_check.scalar_read_hazards(HAZARD)) == 2  # s44 (3 wait states behind) and s45 (1 behind)
    assert isa_check.scalar_read_hazards(HAZARD_FIXED) == []


def test_a_copy_of_a_register_with_a_hand_issued_load_in_flight_is_found():
    assert len(isa_check.inflight_register_uses(COPY_IN_FLIGHT)) == 1
    # vmcnt(1) with one younger load: the first load has landed, the second has not
    assert isa_check.inflight_register_uses(COPY_AFTER_WAIT) == []
    assert len(isa_check.inflight_register_uses(COPY_AFTER_WAIT.replace("v[26:27], v[4:5]", "v[26:27], v[6:7]"))) == 1
    # a load that goes straight to LDS has no destination register (v39 is its address)
    assert isa_check.inflight_register_uses(TO_LDS) == []


_LISTING = {}


def _compiled_listing(tmp_path):
    if "text" not in _LISTING:  # (one compilation for the tests of this file)
        _LISTING["text"] = isa_check.emit_assembly(os.path.join(tmp_path, "device.s"))
    return _LISTING["text"]


def test_the_kernels_as_compiled_have_neither(tmp_path):
    listing = _compiled_listing(tmp_path)
    assert listing.count("ASMSTART") > 50  # (the listing really is the kernels')
    assert isa_check.check(listing) == []


def test_the_backward_kernel_with_feeder_waves_keeps_its_registers_and_polls_with_scalar_offsets(tmp_path):
    """Two properties of slstm_bwd_split_kernel that its speed rests on and that only the assembly shows: the variants
    with feeder waves (twelve waves: 168 registers a lane) do not spill, and the polls of the exchange ring take their
    slot offset from a scalar register (with the offset in a vector register the compiler wraps every poll in a loop
    over the distinct values of the lanes)."""
    import re

    listing = _compiled_listing(tmp_path)
    meta = listing[listing.index("amdhsa.kernels:"):]
    seen = 0
    for entry in re.split(r"\n  - ", meta)[1:]:
        name = re.search(r"\.name:\s+(\S+)", entry)
        # (template arguments: bf16, S, feeder waves, gate deltas in bf16)
        if not name or not re.search(r"slstm_bwd_split_kernelILb[01]ELi\d+ELb1ELb[01]EEEvNS_14BwdSplitParamsE$", name.group(1)):
            continue
        seen += 1
        assert int(re.search(r"\.vgpr_count:\s*(\d+)", entry).group(1)) <= 168, name.group(1)
        assert int(re.search(r"\.private_segment_fixed_size:\s*(\d+)", entry).group(1)) == 0, name.group(1)
        body = listing[listing.index(name.group(1) + ":"):]
        body = body[: body.index(".end_amdhsa_kernel")].split("\n")
        polls = [i for i, line in enumerate(body) if "buffer_load_dwordx4" in line and "sc1" in line]
        assert polls, name.group(1)
        for i in polls:
            assert not any("v_readfirstlane" in line for line in body[max(0, i - 6): i]), (name.group(1), body[i - 6: i + 1])
    assert seen == 8  # bf16 at head dims 64, 128, 256 with the gate deltas in float32 and in bf16; float32 at 64, 128
