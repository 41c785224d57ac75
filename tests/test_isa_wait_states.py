"""The wait-state scan that the library's build runs over the device assembly of its asm-issued copies
(flaggems_amd/csrc/isa_check.py): known-answer cases on hand-written assembly, so that a scan that stops seeing
the hazard (a regex that no longer matches, an off-by-one in the count) fails here and not on a GPU."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_spec = importlib.util.spec_from_file_location("fg_isa_check", os.path.join(ROOT, "flaggems_amd", "csrc", "isa_check.py"))
isa_check = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(isa_check)


def kernel(body, name="k0"):
    return "%s:                ; @%s\n; %%bb.0:\n%s\n\ts_endpgm\n.Lfunc_end0:\n" % (name, name, body)


COPY = "\tglobal_load_lds_dwordx4 v47, s[6:7] offset:1024"


@pytest.mark.parametrize("between,expect", [(0, 1), (1, 1), (4, 1), (5, 0), (9, 0)])
def test_readfirstlane_then_copy_needs_five_wait_states(between, expect):
    body = "\tv_readfirstlane_b32 s6, v36\n" + "\tv_add_u32_e32 v1, v2, v3\n" * between + COPY
    assert len(isa_check.scan(kernel(body))) == expect


def test_both_halves_of_the_base_are_seen():
    body = "\tv_readfirstlane_b32 s6, v36\n\tv_readfirstlane_b32 s7, v37\n" + COPY
    hits = isa_check.scan(kernel(body))
    assert len(hits) == 2 and all("global_load_lds" in h[2] for h in hits)


@pytest.mark.parametrize("nop,expect", [(3, 1), (4, 0)])
def test_s_nop_counts_as_its_argument_plus_one(nop, expect):
    body = "\tv_readlane_b32 s7, v3, 5\n\ts_nop %d\n%s" % (nop, COPY)
    assert len(isa_check.scan(kernel(body))) == expect


def test_scalar_arithmetic_on_the_base_is_no_hazard():
    body = "\ts_add_u32 s6, s6, 0x80\n\ts_addc_u32 s7, s7, 0\n" + COPY
    assert isa_check.scan(kernel(body)) == []


def test_other_registers_do_not_count():
    body = "\tv_readfirstlane_b32 s8, v36\n" + COPY + "\n\tglobal_load_dwordx4 v[0:3], v8, s[10:11]"
    assert isa_check.scan(kernel(body)) == []


def test_compare_into_scalar_pair_then_store_with_that_base():
    body = "\tv_cmp_lt_u32_e64 s[6:7], v1, v2\n\tglobal_store_dword v0, v1, s[6:7]"
    assert len(isa_check.scan(kernel(body))) == 1


def test_m0_needs_one_wait_state_before_an_lds_direct_load():
    assert len(isa_check.scan(kernel("\ts_mov_b32 m0, s9\n" + COPY))) == 1
    assert isa_check.scan(kernel("\ts_mov_b32 m0, s9\n\ts_nop 0\n" + COPY)) == []
    # an ordinary load does not read M0
    assert isa_check.scan(kernel("\ts_mov_b32 m0, s9\n\tglobal_load_dwordx4 v[0:3], v8, s[6:7]")) == []


def test_every_function_and_every_exit_is_scanned():
    early = "\ts_cbranch_scc1 .LBB0_2\n\ts_endpgm\n.LBB0_2:\n\tv_readfirstlane_b32 s6, v36\n" + COPY
    text = kernel("\ts_nop 0", "k0") + kernel(early, "k1")
    hits = isa_check.scan(text)
    assert [h[0] for h in hits] == ["k1"]


def test_state_does_not_leak_between_functions():
    text = kernel("\tv_readfirstlane_b32 s6, v36", "k0") + kernel(COPY, "k1")
    assert isa_check.scan(text) == []


MFMA = "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[10:13], v[20:23], a[0:3]"


@pytest.mark.parametrize("between,expect", [(0, 1), (10, 1), (11, 0)])
def test_accumulator_read_after_a_matrix_instruction(between, expect):
    body = MFMA + "\n" + "\tv_add_u32_e32 v1, v2, v3\n" * between + "\tv_accvgpr_read_b32 v5, a2"
    assert len(isa_check.scan(kernel(body))) == expect


def test_two_s_nop_15_clear_the_accumulators():
    body = MFMA + "\n\ts_nop 15\n\ts_nop 15\n\tv_accvgpr_read_b32 v5, a0\n\tv_accvgpr_write_b32 a3, v1"
    assert isa_check.scan(kernel(body)) == []


def test_chained_matrix_instructions_and_other_accumulators_are_fine():
    other = "\tv_mfma_f32_16x16x32_bf16 a[4:7], v[10:13], v[20:23], a[4:7]"
    body = MFMA + "\n" + MFMA + "\n" + other + "\n\tv_accvgpr_read_b32 v5, a9"
    assert isa_check.scan(kernel(body)) == []


# ---- LDS reads against the LDS counter ------------------------------------------------------------------------
READS = "\tds_read_b128 v[0:3], v40\n\tds_read_b128 v[4:7], v40 offset:1024\n\tds_read_b64_tr_b16 v[8:9], v41\n"
USE0 = "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[20:23], a[0:3]"


@pytest.mark.parametrize("wait,expect", [(0, 0), (2, 0), (3, 1)])
def test_a_counted_wait_retires_the_oldest_reads_only(wait, expect):
    body = READS + "\ts_waitcnt lgkmcnt(%d)\n" % wait + USE0
    assert len(isa_check.scan_lds_reads(kernel(body))) == expect


def test_use_of_a_younger_read_needs_a_smaller_count():
    use2 = "\tv_pk_mul_f16 v30, v8, v9"
    assert len(isa_check.scan_lds_reads(kernel(READS + "\ts_waitcnt lgkmcnt(1)\n" + use2))) == 1
    assert isa_check.scan_lds_reads(kernel(READS + "\ts_waitcnt vmcnt(3) lgkmcnt(0)\n" + use2)) == []
    # a wait on the vector-memory counter alone retires nothing here
    assert len(isa_check.scan_lds_reads(kernel(READS + "\ts_waitcnt vmcnt(0)\n" + USE0))) == 1


def test_overwriting_a_register_with_a_read_in_flight_is_reported():
    body = "\tds_read_b128 v[0:3], v40\n\tv_mov_b32_e32 v2, 0\n\ts_waitcnt lgkmcnt(0)"
    assert len(isa_check.scan_lds_reads(kernel(body))) == 1


def test_the_address_register_may_be_reused_at_once():
    body = "\tds_read_b128 v[0:3], v40\n\tv_add_u32_e32 v40, 16, v40\n\ts_waitcnt lgkmcnt(0)\n" + USE0
    assert isa_check.scan_lds_reads(kernel(body)) == []


def test_lds_writes_and_scalar_loads_count_too():
    body = "\tds_read_b128 v[0:3], v40\n\tds_write_b32 v41, v42\n\ts_waitcnt lgkmcnt(1)\n" + USE0
    assert isa_check.scan_lds_reads(kernel(body)) == []
    # a scalar load in flight returns out of order: lgkmcnt(1) proves nothing about the read
    body = "\tds_read_b128 v[0:3], v40\n\ts_load_dwordx2 s[4:5], s[0:1], 0x0\n\ts_waitcnt lgkmcnt(1)\n" + USE0
    assert len(isa_check.scan_lds_reads(kernel(body))) == 1


def test_the_counter_is_followed_around_a_loop():
    """The read issued at the bottom of the loop body is still in flight at its top on the way round; the use at the
    top is fine on entry (nothing outstanding) and stale on the back edge unless the body waits first."""
    loop = ("\ts_mov_b32 s4, 8\n.LBB0_1:\n%s" + USE0 + "\n\tds_read_b128 v[0:3], v40\n\ts_sub_u32 s4, s4, 1\n"
            "\ts_cmp_lg_u32 s4, 0\n\ts_cbranch_scc1 .LBB0_1\n\ts_waitcnt lgkmcnt(0)")
    assert len(isa_check.scan_lds_reads(kernel(loop % ""))) == 1
    assert isa_check.scan_lds_reads(kernel(loop % "\ts_waitcnt lgkmcnt(0)\n")) == []


def test_both_arms_of_a_branch_are_followed():
    body = ("\tds_read_b128 v[0:3], v40\n\ts_cbranch_scc1 .LBB0_2\n\ts_waitcnt lgkmcnt(0)\n.LBB0_2:\n" + USE0)
    assert len(isa_check.scan_lds_reads(kernel(body))) == 1   # the taken arm skips the wait


def test_packed_fp32_arithmetic_is_reported():
    assert len(isa_check.scan_packed_f32(kernel("\tv_pk_fma_f32 v[0:1], v[2:3], v[4:5], v[6:7]"))) == 1
    assert isa_check.scan_packed_f32(kernel("\tv_pk_mul_f16 v0, v1, v2\n\tv_fma_f32 v0, v1, v2, v3")) == []


def _build_module():
    spec = importlib.util.spec_from_file_location("fg_build_for_test", os.path.join(ROOT, "flaggems_amd", "csrc", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_the_build_refuses_an_object_whose_assembly_fails_the_scan(tmp_path, monkeypatch):
    build = _build_module()
    obj = tmp_path / "x.hip.o"
    asm = tmp_path / "x-hip-amdgcn-amd-amdhsa-gfx950.s"
    leftover = tmp_path / "x-hip-amdgcn-amd-amdhsa-gfx950.hipi"
    other = tmp_path / "y.hip.o"
    for f in (obj, leftover, other):
        f.write_text("")
    asm.write_text(kernel("\tv_readfirstlane_b32 s6, v36\n" + COPY))
    with pytest.raises(RuntimeError, match="fails 1 check"):
        build._check_wait_states("x.hip", str(obj), str(tmp_path))
    assert not obj.exists() and other.exists()        # nothing stale left to link
    # a clean assembly: the object stays, the bulky intermediates go, the assembly is kept for inspection
    obj.write_text("")
    leftover.write_text("")
    asm.write_text(kernel("\tv_readfirstlane_b32 s6, v36\n\ts_nop 4\n" + COPY))
    build._check_wait_states("x.hip", str(obj), str(tmp_path))
    assert obj.exists() and asm.exists() and not leftover.exists() and other.exists()
    # no assembly at all is an error too: the check must not be skipped silently
    asm.unlink()
    with pytest.raises(RuntimeError, match="no device assembly"):
        build._check_wait_states("x.hip", str(obj), str(tmp_path))


def test_expected_compiler_remarks_are_dropped_from_the_build_log():
    build = _build_module()
    text = "\n".join([
        "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)",
        "In file included from x.hip:5:",
        "/a/gemm_dma.h:290:20: warning: inline asm clobber list contains reserved registers: m0 [-Winline-asm]",
        "  290 |       asm volatile(...);",
        "      |                    ^",
        "/a/gemm_dma.h:290:20: note: Reserved registers on the clobber list may not be preserved across the asm statement",
        "In file included from x.hip:6:",
        "/a/foo.h:12:3: warning: unused variable 'x' [-Wunused-variable]",
        "   12 |   int x;",
        "800 warnings generated.",
    ])
    kept = build._quiet(text).splitlines()
    assert kept == ["In file included from x.hip:6:", "/a/foo.h:12:3: warning: unused variable 'x' [-Wunused-variable]",
                    "   12 |   int x;"]


def test_scratch_accesses_are_reported_inside_loops_only():
    spill = "\tscratch_store_dword off, v5, off offset:4\n"
    straight = kernel(spill + "\tv_mov_b32_e32 v1, v2")
    assert isa_check.scan_scratch_in_loops(straight) == []
    loop = kernel("\ts_mov_b32 s4, 8\n.LBB0_1:\n" + spill + "\ts_sub_u32 s4, s4, 1\n\ts_cmp_lg_u32 s4, 0\n"
                  "\ts_cbranch_scc1 .LBB0_1\n\tscratch_load_dword v5, off, off offset:4")
    hits = isa_check.scan_scratch_in_loops(loop)
    assert len(hits) == 1 and hits[0][1] == 1          # the reload behind the loop does not count
    # a loop of several blocks (the access sits in a block that only the back edge closes)
    nested = kernel("\ts_mov_b32 s4, 8\n.LBB0_1:\n\ts_cbranch_scc0 .LBB0_3\n.LBB0_2:\n" + spill +
                    ".LBB0_3:\n\ts_sub_u32 s4, s4, 1\n\ts_cmp_lg_u32 s4, 0\n\ts_cbranch_scc1 .LBB0_1")
    assert len(isa_check.scan_scratch_in_loops(nested)) == 1
    # allowed by name
    assert isa_check.scan_scratch_in_loops(loop, allowed={"k0": "test"}) == []


# ---- vector-memory loads against the VM counter (scan_vmem_loads) ------------------------------------------------
LOAD = "\tglobal_load_dwordx4 v[8:11], v[20:21], off"
STORE = "\tglobal_store_dwordx4 v[20:21], v[30:33], off"


@pytest.mark.parametrize("younger,wait,expect", [(0, 0, 0), (2, 2, 0), (2, 3, 1), (2, 1, 0), (5, 63, 1)])
def test_a_vm_wait_retires_all_but_the_youngest(younger, wait, expect):
    """A load, `younger` stores behind it, a wait for all but `wait` operations, then a use of the loaded register."""
    body = LOAD + "\n" + (STORE + "\n") * younger + "\ts_waitcnt vmcnt(%d)\n\tv_add_u32_e32 v1, v8, v3" % wait
    assert len(isa_check.scan_vmem_loads(kernel(body))) == expect


def test_a_use_without_any_wait_and_an_overwrite_are_reported():
    assert len(isa_check.scan_vmem_loads(kernel(LOAD + "\n\tv_mov_b32_e32 v40, v11"))) == 1
    assert len(isa_check.scan_vmem_loads(kernel(LOAD + "\n\tv_mov_b32_e32 v9, v40"))) == 1    # written under the load
    assert len(isa_check.scan_vmem_loads(kernel(LOAD + "\n\tv_mov_b32_e32 v20, v40"))) == 0   # the address is free at once
    assert len(isa_check.scan_vmem_loads(kernel(LOAD + "\n\tds_bpermute_b32 v50, v51, v10"))) == 1


def test_loads_return_in_order_lds_direct_loads_and_stores_count():
    again = "\tglobal_load_dwordx4 v[8:11], v[22:23], off"
    assert isa_check.scan_vmem_loads(kernel(LOAD + "\n" + again + "\n\ts_waitcnt vmcnt(0)\n\tv_mov_b32_e32 v1, v8")) == []
    body = LOAD + "\n" + COPY + "\n" + STORE + "\n\ts_waitcnt vmcnt(2)\n\tv_mov_b32_e32 v1, v8"
    assert isa_check.scan_vmem_loads(kernel(body)) == []
    body = LOAD + "\n" + COPY + "\n" + STORE + "\n\ts_waitcnt vmcnt(3)\n\tv_mov_b32_e32 v1, v8"
    assert len(isa_check.scan_vmem_loads(kernel(body))) == 1
    # a wait that names only the LDS counter retires nothing here; a bare immediate carries the count in bits 3:0, 15:14
    assert len(isa_check.scan_vmem_loads(kernel(LOAD + "\n\ts_waitcnt lgkmcnt(0)\n\tv_mov_b32_e32 v1, v8"))) == 1
    assert isa_check.scan_vmem_loads(kernel(LOAD + "\n\ts_waitcnt 0x0f70\n\tv_mov_b32_e32 v1, v8")) == []
    assert len(isa_check.scan_vmem_loads(kernel(LOAD + "\n\ts_waitcnt 0x0f71\n\tv_mov_b32_e32 v1, v8"))) == 1


def test_the_vm_counter_is_followed_around_a_loop_and_through_both_arms():
    # a ring of two registers: the load of one trip is used in the next, behind a wait that leaves one load in flight
    ring = ("\tglobal_load_dwordx4 v[8:11], v[20:21], off\n.LBB0_1:\n\tglobal_load_dwordx4 v[12:15], v[20:21], off\n"
            "\ts_waitcnt vmcnt(%d)\n\tv_mov_b32_e32 v1, v8\n\tglobal_load_dwordx4 v[8:11], v[20:21], off\n"
            "\ts_waitcnt vmcnt(%d)\n\tv_mov_b32_e32 v1, v12\n\ts_cbranch_scc1 .LBB0_1")
    assert isa_check.scan_vmem_loads(kernel(ring % (1, 1))) == []
    assert len(isa_check.scan_vmem_loads(kernel(ring % (2, 1)))) == 1
    assert len(isa_check.scan_vmem_loads(kernel(ring % (1, 2)))) == 1
    arms = (LOAD + "\n\ts_cbranch_scc1 .LBB0_2\n\ts_waitcnt vmcnt(0)\n\ts_branch .LBB0_3\n.LBB0_2:\n" + STORE +
            "\n.LBB0_3:\n\tv_mov_b32_e32 v1, v8")
    assert len(isa_check.scan_vmem_loads(kernel(arms))) == 1        # one arm does not wait
    assert isa_check.scan_vmem_loads(kernel(arms.replace(STORE, "\ts_waitcnt vmcnt(0)"))) == []
