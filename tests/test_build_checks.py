"""The build's check of hand-waited loads: registers written by marked ring loads must be the registers the
marked ring waits pass through, per function of the generated code (backpack_amd/build.py)."""
import os

from backpack_amd import build as b

GOOD = """
	.text
_ZN2kq6kernelE:                          ; @_ZN2kq6kernelE
	global_load_dwordx4 v[52:55], v[2:3], off ; ringld
	global_load_dwordx2 v[60:61], v[4:5], off ; ringld
	global_load_ushort v70, v[4:5], off ; ringld
.LBB0_2:
	s_waitcnt vmcnt(4) ; ringwait v[52:55] v[60:61] v70
	v_and_b32_e32 v1, 15, v52
	s_endpgm
_ZN2kq5otherE:
	v_mov_b32_e32 v1, v2
	s_endpgm
"""
# the load writes v[52:55]; the value was copied to v[84:87] before the wait
MOVED = GOOD.replace("ringwait v[52:55]", "ringwait v[84:87]")
# a load into a register no wait names (handed to another function's wait after a copy)
ORPHAN = GOOD.replace("	global_load_ushort v70,", "	global_load_dwordx4 v[20:23], v[2:3], off ; ringld\n	global_load_ushort v70,")


def _check(tmp_path, text):
    p = tmp_path / "k.s"
    p.write_text(text)
    return b.check_ring_registers(str(p))


def test_matching_registers_pass(tmp_path):
    assert _check(tmp_path, GOOD) == []


def test_moved_register_is_reported(tmp_path):
    probs = _check(tmp_path, MOVED)
    assert len(probs) == 1 and "_ZN2kq6kernelE" in probs[0] and "52" in probs[0] and "84" in probs[0]


def test_load_without_wait_is_reported(tmp_path):
    probs = _check(tmp_path, ORPHAN)
    assert len(probs) == 1 and "20" in probs[0]


# the stricter reading, top to bottom, for sources whose rings live in straight-line code
TOUCHED = GOOD.replace(".LBB0_2:\n", ".LBB0_2:\n\tv_mov_b32_e32 v90, v61\n")                      # a copy of a register in flight
SWAPPED = GOOD.replace("ringwait v[52:55] v[60:61] v70", "ringwait v[52:55] v[60:61] v71")          # a wait on another register
RELOADED = GOOD.replace(".LBB0_2:\n", ".LBB0_2:\n\tglobal_load_ushort v70, v[4:5], off ; ringld\n")  # refilled before its wait


def _order(tmp_path, text):
    p = tmp_path / "k.s"
    p.write_text(text)
    return b.check_ring_order(str(p))


def test_straight_line_reading_passes_good_code(tmp_path):
    assert _order(tmp_path, GOOD) == []


def test_straight_line_reading_reports_touch_wrong_wait_and_early_refill(tmp_path):
    probs = _order(tmp_path, TOUCHED)
    assert len(probs) == 1 and "61" in probs[0] and "v_mov_b32_e32" in probs[0]
    probs = _order(tmp_path, SWAPPED)
    assert len(probs) == 1 and "71" in probs[0]
    probs = _order(tmp_path, RELOADED)
    assert len(probs) == 1 and "70" in probs[0] and "again" in probs[0]
    # (the per-function comparison of sets sees the wrong wait as well, but neither the copy nor the early refill)
    assert _check(tmp_path, TOUCHED) == [] and _check(tmp_path, RELOADED) == []


def test_generated_code_of_the_library_was_checked():
    """The build leaves the device code of the guarded sources as text; every kernel in it that has marked
    loads has marked waits on the same registers."""
    for name in ("kq_stream.s", "kq_chain.s"):
        path = os.path.join(b.OBJ, name)
        if not os.path.exists(path):      # a tree that was built elsewhere carries the library only
            continue
        assert "; ringld" in open(path).read()
        assert b.check_ring_registers(path) == []
    path = os.path.join(b.OBJ, "kq_mgemv.s")
    if os.path.exists(path):
        assert "; ringld" in open(path).read()
        assert b.check_ring_registers(path) == [] and b.check_ring_order(path) == []
