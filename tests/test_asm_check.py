"""The build-time checker of hand-issued LDS reads (csrc/check_asm_reads.py) on small pieces of
assembly text: it must accept the intended pattern and flag each way the pattern can break."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_spec = importlib.util.spec_from_file_location("check_asm_reads", os.path.join(ROOT, "bfuse-project_amd", "csrc", "check_asm_reads.py"))
chk = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(chk)

READ_A = "\t;;#ASMSTART\n\tds_read_b128 v[20:23], v14 offset:0\n\t;;#ASMEND\n"
READ_B = "\t;;#ASMSTART\n\tds_read_b64 v[24:25], v15 offset:0x800\n\t;;#ASMEND\n"
WAIT = "\t;;#ASMSTART\n\ts_waitcnt lgkmcnt({n})\n\t;;#ASMEND\n"


def _run(tmp_path, body):
    p = tmp_path / "k.s"
    p.write_text("kern:\n" + body + "\ts_endpgm\n")
    return chk.check(str(p))


def test_the_intended_pattern_is_accepted(tmp_path):
    body = (READ_A + READ_B + "\tv_mfma_f32_16x16x4_f32 a[0:3], v2, v3, a[0:3]\n" + WAIT.format(n=1) +
            "\tv_mfma_f32_16x16x32_bf16 a[4:7], v[20:23], v[30:33], a[4:7]\n" + WAIT.format(n=0) +
            "\tv_mov_b32_e32 v40, v24\n")
    findings, n = _run(tmp_path, body)
    assert n == 2 and findings == []


def test_a_copy_before_the_wait_is_flagged(tmp_path):
    findings, _ = _run(tmp_path, READ_A + "\tv_mov_b32_e32 v40, v21\n" + WAIT.format(n=0))
    assert len(findings) == 1 and "names v21" in findings[0]


def test_a_spill_or_an_overwrite_before_the_wait_is_flagged(tmp_path):
    findings, _ = _run(tmp_path, READ_A + "\tscratch_store_dword off, v22, off offset:8\n" + WAIT.format(n=0))
    assert len(findings) == 1
    findings, _ = _run(tmp_path, READ_A + "\tv_add_u32_e32 v20, v1, v2\n" + WAIT.format(n=0))
    assert len(findings) == 1 and "names v20" in findings[0]
    findings, _ = _run(tmp_path, READ_A + "\tv_accvgpr_write_b32 a3, v23\n" + WAIT.format(n=0))
    assert len(findings) == 1


def test_a_partial_wait_retires_only_the_older_reads(tmp_path):
    # lgkmcnt(1) after two reads: the first has landed, the second has not
    findings, _ = _run(tmp_path, READ_A + READ_B + WAIT.format(n=1) + "\tv_mov_b32_e32 v40, v20\n" + WAIT.format(n=0))
    assert findings == []
    findings, _ = _run(tmp_path, READ_A + READ_B + WAIT.format(n=1) + "\tv_mov_b32_e32 v40, v25\n" + WAIT.format(n=0))
    assert len(findings) == 1 and "names v25" in findings[0]


def test_a_scalar_load_in_flight_at_a_partial_wait_is_flagged(tmp_path):
    findings, _ = _run(tmp_path, "\ts_load_dwordx2 s[4:5], s[0:1], 0x10\n" + READ_A + READ_B + WAIT.format(n=1) + WAIT.format(n=0))
    assert len(findings) == 1 and "scalar-memory load" in findings[0]
    # a full wait between them makes it sound
    findings, _ = _run(tmp_path, "\ts_load_dwordx2 s[4:5], s[0:1], 0x10\n\ts_waitcnt lgkmcnt(0)\n" + READ_A + READ_B + WAIT.format(n=1) + WAIT.format(n=0))
    assert findings == []


def test_reads_never_waited_for_and_reads_across_a_backward_branch_are_flagged(tmp_path):
    findings, _ = _run(tmp_path, READ_A)
    assert len(findings) == 1 and "never waited for" in findings[0]
    findings, _ = _run(tmp_path, ".LBB0_1:\n" + READ_A + "\ts_cbranch_scc1 .LBB0_1\n" + WAIT.format(n=0))
    assert len(findings) == 1 and "backward branch" in findings[0]


def test_a_loop_may_carry_reads_round_its_branch_in_the_registers_it_was_entered_with(tmp_path):
    use_a = WAIT.format(n=0) + "\tv_mfma_f32_16x16x32_bf16 a[4:7], v[20:23], v[30:33], a[4:7]\n"
    # software pipelining: the first read of the next step is in flight at the loop head, each time
    findings, _ = _run(tmp_path, READ_A + ".LBB0_1:\n" + use_a + READ_A + "\ts_cbranch_scc1 .LBB0_1\n" + use_a)
    assert findings == []
    # the branch is taken with the read in other registers than the loop head expects
    findings, _ = _run(tmp_path, READ_A + ".LBB0_1:\n" + use_a + READ_B + "\ts_cbranch_scc1 .LBB0_1\n" + use_a)
    assert len(findings) == 1 and "backward branch" in findings[0]
    # ... or with nothing in flight where the loop head was entered with a read
    findings, _ = _run(tmp_path, READ_A + ".LBB0_1:\n" + use_a + "\ts_cbranch_scc1 .LBB0_1\n")
    assert len(findings) == 1 and "backward branch" in findings[0]


def test_the_compilers_own_reads_are_not_tracked_but_take_a_counter_slot(tmp_path):
    # a compiler-issued ds_read after the asm read is the youngest: lgkmcnt(1) retires the asm read
    body = READ_A + "\tds_read_b32 v50, v51\n" + "\ts_waitcnt lgkmcnt(1)\n" + "\tv_mov_b32_e32 v40, v20\n" + "\ts_waitcnt lgkmcnt(0)\n"
    findings, n = _run(tmp_path, body)
    assert n == 1 and findings == []


def test_the_built_kernels_pass(tmp_path):
    import glob
    files = glob.glob(os.path.join(ROOT, "bfuse-project_amd", "csrc", "obj", "kernels_*-gfx950.s"))
    if not files:
        import pytest
        pytest.skip("device assembly not present (library not built in this tree)")
    total = 0
    for f in files:
        findings, n = chk.check(f)
        assert findings == [], findings[:3]
        total += n
    assert total > 1000          # the GEMMs' hand-issued reads were found and followed
