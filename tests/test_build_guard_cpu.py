"""The build's check on kernels that wait for inline-assembly loads by count
(`warpconvnet_amd/_build.py::_check_loads_not_copied`), fed hand-written listings: what it must
accept, what it must reject, and that it refuses a listing it cannot read."""
import pytest

from warpconvnet_amd import _build


def _listing(body: str, name: str = "_Z13conv_fwd_packv") -> str:
    return f"\t.text\n{name}:\n{body}\n\ts_endpgm\n"


LOAD = "\t;;#ASMSTART\n\tglobal_load_dword {dst}, v1, s[0:1]{off}\n\t;;#ASMEND\n"


def _load(dst, off=""):
    return LOAD.format(dst=dst, off=off)


CLEAN_LOOP = (
    "\ts_mov_b32 s4, 0\n"
    ".LBB0_1:\n"
    + _load("v5") + _load("v6", " offset:4") +
    "\ts_waitcnt vmcnt(1)\n"            # one load issued since v5's: v5 has landed
    "\tv_add_u32_e32 v7, v5, v2\n"
    "\ts_waitcnt vmcnt(0)\n"
    "\tv_add_u32_e32 v8, v6, v2\n"
    "\ts_add_i32 s4, s4, 1\n"
    "\ts_cmp_lt_i32 s4, 10\n"
    "\ts_cbranch_scc1 .LBB0_1\n"
)

# the load into v6 is still in flight when the branch goes back; the loop head copies v6 before
# any wait (what the compiler once did to a pair-list register: wrong sums, no fault)
COPY_AT_LOOP_HEAD = (
    ".LBB0_1:\n"
    "\tv_mov_b32_e32 v9, v6\n"
    "\ts_waitcnt vmcnt(0)\n"
    "\tv_add_u32_e32 v7, v9, v2\n"
    + _load("v6") +
    "\ts_cmp_lt_i32 s4, 10\n"
    "\ts_cbranch_scc1 .LBB0_1\n"
    "\ts_waitcnt vmcnt(0)\n"
)

# vmcnt(2) with only one load issued since: v5 need not have landed
WAIT_ONE_TOO_HIGH = (
    ".LBB0_1:\n"
    + _load("v5") + _load("v6", " offset:4") +
    "\ts_waitcnt vmcnt(2)\n"
    "\tv_add_u32_e32 v7, v5, v2\n"
    "\ts_waitcnt vmcnt(0)\n"
    "\tv_add_u32_e32 v8, v6, v2\n"
    "\ts_cbranch_scc1 .LBB0_1\n"
)

# one of two paths to the use has no wait
READ_ON_A_FORWARD_JUMP = (
    ".LBB0_1:\n"
    + _load("v5") +
    "\ts_cbranch_vccz .LBB0_3\n"
    "\ts_waitcnt vmcnt(0)\n"
    "\tv_add_u32_e32 v7, v5, v2\n"
    "\ts_branch .LBB0_4\n"
    ".LBB0_3:\n"
    "\tv_add_u32_e32 v7, v5, v2\n"
    ".LBB0_4:\n"
    "\ts_waitcnt vmcnt(0)\n"
    "\ts_cbranch_scc1 .LBB0_1\n"
)

# the destination takes its next load before the first was waited for and used: overwritten in flight
RELOADED_TOO_EARLY_IS_NOT_A_USE = (
    ".LBB0_1:\n"
    + _load("v5") + _load("v5") +
    "\ts_waitcnt vmcnt(0)\n"
    "\tv_add_u32_e32 v7, v5, v2\n"
    "\ts_cbranch_scc1 .LBB0_1\n"
)


def test_clean_loop_is_accepted():
    _build._check_loads_not_copied("probe.hip", _listing(CLEAN_LOOP))
    # a load's destination given to its next load ends the walk for the first one: not a use
    _build._check_loads_not_copied("probe.hip", _listing(RELOADED_TOO_EARLY_IS_NOT_A_USE))


@pytest.mark.parametrize("body,where", [
    (COPY_AT_LOOP_HEAD, "v_mov_b32_e32 v9, v6"),
    (WAIT_ONE_TOO_HIGH, "v_add_u32_e32 v7, v5, v2"),
    (READ_ON_A_FORWARD_JUMP, "v_add_u32_e32 v7, v5, v2"),
], ids=["copy_at_loop_head", "wait_count_one_too_high", "read_on_a_forward_jump"])
def test_touching_a_load_in_flight_is_rejected(body, where):
    with pytest.raises(RuntimeError) as err:
        _build._check_loads_not_copied("probe.hip", _listing(body))
    assert where in str(err.value)


def test_register_ranges_and_wide_loads():
    body = (
        ".LBB0_1:\n"
        "\t;;#ASMSTART\n\tglobal_load_dwordx4 v[10:13], v1, s[0:1]\n\t;;#ASMEND\n"
        "\tv_mov_b32_e32 v20, v12\n"       # inside the 4-register destination
        "\ts_waitcnt vmcnt(0)\n"
        "\ts_cbranch_scc1 .LBB0_1\n"
    )
    with pytest.raises(RuntimeError):
        _build._check_loads_not_copied("probe.hip", _listing(body))
    assert _build._vgprs_in("v[10:13], v1, s[0:1]") == {10, 11, 12, 13, 1}


def test_a_listing_the_check_cannot_read_is_refused():
    """A kernel known to keep loads in flight in which no written-out load, or no loop around
    them, is recognised (the compiler spelling its markers or labels differently, say) fails
    the build instead of passing unchecked."""
    unreadable = CLEAN_LOOP.replace("#ASMSTART", "#APP").replace("#ASMEND", "#NO_APP")
    with pytest.raises(RuntimeError, match="0 written-out loads"):
        _build._check_loads_not_copied("probe.hip", _listing(unreadable))
    no_loop = CLEAN_LOOP.replace("\ts_cbranch_scc1 .LBB0_1\n", "")
    with pytest.raises(RuntimeError, match="not found"):
        _build._check_loads_not_copied("probe.hip", _listing(no_loop))
    # kernels of other names are not held to this
    _build._check_loads_not_copied("probe.hip", _listing(unreadable, name="_Z5otherv"))


def test_no_scratch_rule_reads_the_resource_remarks():
    ok = ("x.hip:1:1: remark: Function Name: k [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]\n")
    _build._check_no_scratch("wcn_conv_pack_f16.hip", ok)
    with pytest.raises(RuntimeError, match="scratch"):
        _build._check_no_scratch("wcn_conv_pack_f16.hip", ok.replace("VGPRs Spill: 0", "VGPRs Spill: 3"))
    with pytest.raises(RuntimeError, match="no resource-usage remarks"):
        _build._check_no_scratch("wcn_conv_pack_f16.hip", "")
    _build._check_no_scratch("wcn_table.hip", "")  # other sources are not held to the rule
