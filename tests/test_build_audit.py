"""The build's check of the generated assembly: an inline-asm LDS read whose registers are touched before the
wait that covers it must be reported (the compiler may copy such registers when a conditional read is merged
with the other path; nothing else would notice)."""
from fourierattention_amd.build import audit_async_lds_reads, audit_handover_stores

GOOD = """
_Zkernel_a:
\t;;#ASMSTART
\tds_read_b128 v[10:13], v1 offset:0
\t;;#ASMEND
\tv_add_f32_e32 v20, v21, v22
\t;;#ASMSTART
\ts_waitcnt lgkmcnt(0)
\t;;#ASMEND
\tv_mov_b32_e32 v30, v12
"""

# the copy the compiler makes when the read sits in one arm of a branch
BAD_COPY = """
_Zkernel_b:
\t;;#ASMSTART
\tds_read_b128 v[82:85], v1 offset:0xc00
\t;;#ASMEND
\ts_nop 0
\tv_mov_b32_e32 v93, v85
\t;;#ASMSTART
\ts_waitcnt lgkmcnt(0)
\t;;#ASMEND
"""

# a counted wait leaves the youngest reads in flight
PARTIAL = """
_Zkernel_c:
\t;;#ASMSTART
\tds_read_b128 v[10:13], v1
\t;;#ASMEND
\t;;#ASMSTART
\tds_read_b128 v[14:17], v1 offset:64
\t;;#ASMEND
\t;;#ASMSTART
\ts_waitcnt lgkmcnt(1)
\t;;#ASMEND
\tv_mul_f32_e32 v40, v10, v11
\tv_mul_f32_e32 v41, v14, v15
"""


def test_clean_sequence_passes():
    assert audit_async_lds_reads(GOOD) == []


def test_copy_before_wait_is_reported():
    found = audit_async_lds_reads(BAD_COPY)
    assert len(found) == 1 and "_Zkernel_b" in found[0] and "v_mov_b32_e32 v93, v85" in found[0]


def test_counted_wait_releases_only_the_older_reads():
    found = audit_async_lds_reads(PARTIAL)
    assert len(found) == 1 and "v41" in found[0] and "v40" not in found[0]


# a loop whose tail (with the wait) is laid out before its head and whose exit block follows the body: the exit is
# entered from the loop's latch, where nothing is outstanding, not by falling through from the reads above it
LOOP_EXIT_BEHIND_BODY = """
_Zkernel_d:
.LBB0_1:
\t;;#ASMSTART
\ts_waitcnt lgkmcnt(0)
\t;;#ASMEND
\tv_mul_f32_e32 v40, v28, v29
\ts_cbranch_scc1 .LBB0_3
.LBB0_2:
\t;;#ASMSTART
\tds_read_b128 v[28:31], v16 offset:0
\t;;#ASMEND
\ts_branch .LBB0_1
.LBB0_3:
\tv_accvgpr_read_b32 v29, a29
\ts_endpgm
"""

FALLS_THROUGH_A_CONDITIONAL_BRANCH = """
_Zkernel_e:
\t;;#ASMSTART
\tds_read_b128 v[28:31], v16 offset:0
\t;;#ASMEND
\ts_cbranch_scc1 .LBB0_3
\tv_mov_b32_e32 v5, v30
.LBB0_3:
\ts_endpgm
"""


def test_scan_restarts_behind_an_unconditional_branch_only():
    assert audit_async_lds_reads(LOOP_EXIT_BEHIND_BODY) == []
    found = audit_async_lds_reads(FALLS_THROUGH_A_CONDITIONAL_BRANCH)
    assert len(found) == 1 and "v_mov_b32_e32 v5, v30" in found[0]


def test_audit_fails_closed():
    """No assembly listing at all, or none of the inline-asm reads in a source that issues them, is a failure of
    the audit, not a pass."""
    from fourierattention_amd.build import ASYNC_LDS_SOURCES, audit_listings, count_async_lds_reads
    assert count_async_lds_reads(GOOD) == 1 and count_async_lds_reads(PARTIAL) >= 2
    assert audit_listings("fa_prefill", [GOOD]) == []
    # fa_decode also holds the kernels that hand data between workgroups: without any of their counting atomics in
    # the listing the audit has seen nothing and says so
    assert any("no counting atomic" in m for m in audit_listings("fa_decode", [GOOD]))
    assert any("no gfx950 assembly" in m for m in audit_listings("fa_decode", []))
    plain = "_Zkernel_z:\n\tv_add_f32_e32 v1, v2, v3\n\ts_endpgm\n"
    assert "fa_decode_mid_bf16" in ASYNC_LDS_SOURCES and "fa_stream" not in ASYNC_LDS_SOURCES
    assert any("no inline-asm LDS read" in m for m in audit_listings("fa_decode_mid_bf16", [plain]))
    assert audit_listings("fa_stream", [plain]) == []          # a source without such reads passes on a plain listing
    assert audit_listings("fa_stream", [BAD_COPY]) != []       # but a violation is reported wherever it shows up


# ---- hand-over between workgroups: stores, wait, counting atomic ----------------------------------------------------
HANDOVER_GOOD = """
_Z24decode_merge_rows_kernel13MergeRowsArgs:
\tglobal_store_dword v[2:3], v4, off sc1
\tglobal_store_dwordx4 v[6:7], v[8:11], off
\ts_waitcnt vmcnt(0) expcnt(0) lgkmcnt(0)
\ts_barrier
\ts_cbranch_execz .LBB0_2
; %bb.1:
\tglobal_atomic_add v1, v[2:3], v1, off sc0
.LBB0_2:
\ts_endpgm
"""

# a store that was moved behind the wait
HANDOVER_SUNK = """
_Z24decode_merge_rows_kernel13MergeRowsArgs:
\tglobal_store_dword v[2:3], v4, off sc1
\ts_waitcnt vmcnt(0) lgkmcnt(0)
\ts_barrier
\tglobal_store_dword v[12:13], v14, off sc1
\tglobal_atomic_add v1, v[2:3], v1, off sc0
"""

# a wait that does not cover vector memory
HANDOVER_WRONG_WAIT = """
_ZN7fa_mfma22decode_mid_mfma_kernelI6bf16_tLi8ELi2ELi4ELi2ELi0ELb1ELb0ELb0EEEvNS_9MidParamsIT_EE:
\tglobal_store_dwordx4 v[6:7], v[8:11], off
\ts_waitcnt lgkmcnt(0)
\ts_barrier
\tglobal_atomic_add v1, v[2:3], v1, off sc0
"""

# other kernels are not looked at (the general merge; an instance of the mid-row kernel that leaves the merge to a
# launch of its own: FUSE = false)
HANDOVER_OTHER = """
_Z19decode_merge_kernelPKf:
\tglobal_store_dword v[2:3], v4, off
\tglobal_atomic_add v1, v[2:3], v1, off sc0
_ZN7fa_mfma22decode_mid_mfma_kernelI6bf16_tLi8ELi2ELi4ELi2ELi0ELb0ELb0ELb0EEEvNS_9MidParamsIT_EE:
\tglobal_store_dword v[2:3], v4, off
\tglobal_atomic_add v1, v[2:3], v1, off sc0
"""


def test_handover_clean_sequence_passes():
    assert audit_handover_stores(HANDOVER_GOOD) == ([], 1)


def test_handover_store_behind_the_wait_is_reported():
    found, seen = audit_handover_stores(HANDOVER_SUNK)
    assert seen == 1 and len(found) == 1 and "global_store_dword v[12:13]" in found[0]


def test_handover_wait_must_cover_vector_memory():
    found, seen = audit_handover_stores(HANDOVER_WRONG_WAIT)
    assert seen == 1 and len(found) == 1 and "decode_mid_mfma_kernel" in found[0]


def test_handover_scan_only_covers_the_named_kernels():
    assert audit_handover_stores(HANDOVER_OTHER) == ([], 0)


def test_handover_audit_is_part_of_the_build_of_the_decode_kernels():
    from fourierattention_amd.build import audit_listings
    assert audit_listings("fa_decode", [GOOD + HANDOVER_GOOD]) == []
    assert any("global_store_dword v[12:13]" in m for m in audit_listings("fa_decode", [GOOD + HANDOVER_SUNK]))
    # a kernel with a counting atomic that the audit does not look at (new, or renamed out of its patterns) is reported
    found = audit_listings("fa_decode", [GOOD + HANDOVER_GOOD + HANDOVER_OTHER])
    assert len(found) == 2 and all("not among the kernels" in m for m in found)
    assert "decode_merge_kernel" in found[0] and "Lb0ELb0ELb0EEEv" in found[1]
