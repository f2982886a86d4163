"""The build-time check of the block-scaled kernel's generated assembly (cute-examples_amd/
check_async_loads.py) on hand-written instruction streams: it must accept scale registers that go
from the asynchronous load straight into scaled MFMAs and reject any other reader in between."""
import os
import sys

import pytest

PKG = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cute-examples_amd")
sys.path.insert(0, PKG)
import check_async_loads  # noqa: E402

HEAD = "_ZN5mi35512_GLOBAL__N_117gemm_tn_tile_ringINS_6MxE4M3ENS_4BF16ELb0ELi256ELi2EEEvNS_8GemmArgsE: ; @kernel\n"
TAIL = "\n\ts_endpgm\n.Lfunc_end24:\n"
LOAD = "\tbuffer_load_dwordx2 v[130:131], v190, s[40:43], s61 offen\n\tbuffer_load_dwordx2 v[132:133], v199, s[56:59], s61 offen\n"
MFMA = "\tv_mfma_scale_f32_16x16x128_f8f6f4 a[0:3], v[2:9], v[10:17], a[0:3], v132, v130 op_sel:[1,0,0] op_sel_hi:[0,1,0]\n"


def run(tmp_path, body):
    f = tmp_path / "k.s"
    f.write_text(HEAD + body + TAIL)
    return check_async_loads.check(str(f))


def test_accepts_load_then_mfma_then_reuse(tmp_path):
    body = LOAD + "\ts_waitcnt vmcnt(34)\n" + MFMA + MFMA + "\tv_add_u32_e32 v130, v179, v175\n\tds_read_b128 v[0:3], v130\n"
    assert run(tmp_path, body) == 4


@pytest.mark.parametrize("bad,msg", [
    ("\tv_mov_b32_e32 v200, v131\n", "is read while it belongs to a scale load"),              # a copy of in-flight data
    ("\tds_read_b128 v[0:3], v130\n", "is read while it belongs to a scale load"),
    ("\tbuffer_store_dword v133, v1, s[0:3], 0 offen\n", "is read while it belongs to a scale load"),
])
def test_rejects_other_readers_of_a_loaded_register(tmp_path, bad, msg):
    with pytest.raises(RuntimeError, match=msg):
        run(tmp_path, LOAD + bad + MFMA)


def test_rejects_a_scale_from_a_register_that_was_overwritten(tmp_path):
    with pytest.raises(RuntimeError, match="not fresh from a scale load"):
        run(tmp_path, LOAD + "\tv_mov_b32_e32 v130, v1\n" + MFMA)


def test_rejects_a_scale_register_as_data_operand(tmp_path):
    bad = "\tv_mfma_scale_f32_16x16x128_f8f6f4 a[0:3], v[126:133], v[10:17], a[0:3], v132, v130 op_sel_hi:[0,0,0]\n"
    with pytest.raises(RuntimeError, match="data operand"):
        run(tmp_path, LOAD + bad)


def test_rejects_a_file_without_the_kernel(tmp_path):
    f = tmp_path / "k.s"
    f.write_text("\ts_endpgm\n")
    with pytest.raises(RuntimeError, match="no block-scaled kernel"):
        check_async_loads.check(str(f))


# Lanes whose 16 bytes a ds_read_b128 fetches in the same cycle (64 banks x 4 bytes = 16 lanes per
# cycle).  Not consecutive lanes: this grouping is the one that reproduces every hardware counter
# reading taken on the kernels (SQ_LDS_BANK_CONFLICT per SQ_LDS_IDX_ACTIVE cycle): 0 for the 16-bit
# fragment reads, 0 for fp8 fragments read as chunks g and 4+g, one conflict cycle per access cycle
# (every access takes twice as long) for fp8 fragments read as chunks 2g and 2g+1, and an eight
# times slower read of 32 unswizzled rows.  Sixteen consecutive lanes would call all three fragment
# patterns conflict-free.
LDS_CYCLE_GROUPS = [[l + half for r in ranges for l in r] for half in (0, 32)
                    for ranges in ((range(0, 4), range(12, 16), range(20, 24), range(24, 28)),
                                   (range(4, 8), range(8, 12), range(16, 20), range(28, 32)))]


def lds_read_cycles(lane_addresses):
    """Cycles a ds_read_b128 with these 64 byte addresses takes under the model above (4 = no conflict)."""
    cycles = 0
    for group in LDS_CYCLE_GROUPS:
        per_bank = {}
        for l in group:
            for b in range(4):
                bank = (lane_addresses[l] // 4 + b) % 64
                per_bank[bank] = per_bank.get(bank, 0) + 1
        cycles += max(per_bank.values())
    return cycles


def test_lds_cycle_groups_partition_the_wave():
    assert sorted(l for g in LDS_CYCLE_GROUPS for l in g) == list(range(64))
    assert all(len(g) == 16 for g in LDS_CYCLE_GROUPS)


def test_lds_swizzle_is_a_bijection_and_conflict_free():
    """CPU model of the LDS layout of the tile kernels (the counterpart of the reference's swizzled
    shared-memory layouts, kernels/gemm_kernels/sm90a/gemm.cuh:420-451).  A row is 128 bytes = 8
    chunks of 16; chunk c of row r is stored at chunk c ^ swizzle(r).  Checked: the map is a
    bijection on a 256-row slot; what the direct-to-LDS copies write (lane l of a copy lands at
    16*l and fetches global chunk (l%8) ^ swizzle(row)) is exactly that layout; and every
    ds_read_b128 pattern the kernels issue takes the minimum of four cycles under a bank model that
    also reproduces the patterns measured to conflict."""
    import re
    src = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cute-examples_amd", "csrc",
                            "ring_common.h")).read()
    m = re.search(r"uint32_t swizzle\(uint32_t row\) \{ return \(row >> (\d+)\) & (\d+)u; \}", src)
    assert m, "the swizzle in ring_common.h changed: update this model"
    shift, mask = int(m.group(1)), int(m.group(2))
    swz = lambda r: (r >> shift) & mask

    def address(row, chunk):              # byte address of logical chunk `chunk` of row `row` inside a slot
        return row * 128 + ((chunk ^ swz(row)) * 16)

    rows = 256
    assert len({address(r, c) for r in range(rows) for c in range(8)}) == rows * 8
    assert all(0 <= address(r, c) < rows * 128 for r in range(rows) for c in range(8))

    # copies: one instruction covers 8 rows; lane l -> row l/8, LDS bytes [16 l, 16 l + 16) of those rows
    for first_row in range(0, rows, 8):
        for lane in range(64):
            row = first_row + lane // 8
            fetched_chunk = (lane % 8) ^ swz(row)
            assert address(row, fetched_chunk) == first_row * 128 + 16 * lane

    # Fragment reads of 16-row blocks: lane l reads row (block base + l%16); group g = l/16 picks the
    # logical chunk.  Expected cycles per read: what the hardware counters gave for each pattern.
    patterns16 = {
        "16-bit, slice s (in use)": (lambda s, g, e: s * 4 + g, 4),
        "fp8, chunks g and 4+g (in use, plain and block-scaled)": (lambda s, g, e: g + 4 * e, 4),
        "fp8, chunks 2g and 2g+1 (replaced: measured one conflict cycle per access cycle)": (lambda s, g, e: 2 * g + e, 8),
    }
    for name, (chunk_of, want) in patterns16.items():
        for base in range(0, rows, 16):
            for s in range(2):
                for e in range(2):
                    addrs = [address(base + l % 16, chunk_of(s, l // 16, e)) for l in range(64)]
                    assert lds_read_cycles(addrs) == want, (name, base, s, e)
    # Fragment reads of 32-row blocks (fp8 on 32x32x64 in the two-group kernel): lane l reads row
    # l%32, group l/32 picks chunks 4s + 2g + e.
    for base in range(0, rows, 32):
        for s in range(2):
            for e in range(2):
                addrs = [address(base + l % 32, 4 * s + 2 * (l // 32) + e) for l in range(64)]
                assert lds_read_cycles(addrs) == 4, ("32-row fp8", base, s, e)
    # The layout without the swizzle: 32 rows at one chunk measured 7.85 times slower than swizzled.
    plain32 = [(l % 32) * 128 + (l // 32) * 16 for l in range(64)]
    assert lds_read_cycles(plain32) == 32


def test_kernels_read_fp8_fragments_in_the_conflict_free_order():
    """The sources use chunks g and 4+g for every fragment of two chunks per lane."""
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cute-examples_amd", "csrc")
    ring = open(os.path.join(csrc, "gemm_tn_ring.h")).read()
    assert "if constexpr (kRowSliced) return ((uint32_t)(grp + 4 * e) ^ swz) << 4;" in ring
    stream = open(os.path.join(csrc, "gemm_tn_stream.hip")).read()
    assert "(p + ((grp ^ swz) * 16))" in stream and "(p + (((grp + 4) ^ swz) * 16))" in stream
    assert "grp * 2 + 1" not in stream


RING_HEAD = "_ZN5mi35512_GLOBAL__N_117gemm_tn_tile_ringINS_4BF16ES2_Lb0ELi256ELi2ELi256EEEvNS_8GemmArgsE: ; @kernel\n"
SET = "\ts_add_u32 m0, s12, 0x8000\n"
COPY = "\tbuffer_load_dwordx4 v175, s[40:43], s61 offen lds\n"
MFMA16 = "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]\n"


def run_lds(tmp_path, body):
    f = tmp_path / "r.s"
    f.write_text(RING_HEAD + body + TAIL)
    return check_async_loads.check_lds_base(str(f))


def test_lds_base_check_accepts_a_write_one_mfma_ahead(tmp_path):
    assert run_lds(tmp_path, SET + MFMA16 + COPY + MFMA16 + SET + COPY) == 2


@pytest.mark.parametrize("body,msg", [
    (SET + "\ts_mov_b32 m0, -1\n" + COPY, "written by something else"),
    (SET + SET + COPY, "two writes of M0"),
    (SET + COPY + COPY, "without its own write"),
    (SET + COPY + SET, "no copy uses"),
])
def test_lds_base_check_rejects(tmp_path, body, msg):
    with pytest.raises(RuntimeError, match=msg):
        run_lds(tmp_path, body)


# ---------------------------------------------------------------- store-data and MFMA-result distances

K_HEAD = "_ZN5mi3554demoEv: ; @kernel\n"
STORE = "\tbuffer_store_dwordx4 v[0:3], v150, s[20:23], s86 offen nt sc1\n"
FILL = "\tv_add_u32_e32 v100, v101, v102\n"
ASM_MFMA = "\t;;#ASMSTART\n\tv_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]\n\t;;#ASMEND\n"


def run_hazards(tmp_path, body):
    f = tmp_path / "h.s"
    f.write_text(K_HEAD + body + TAIL)
    return check_async_loads.check_hazard_distances(str(f))


def test_store_data_may_be_rewritten_after_the_window(tmp_path):
    w = check_async_loads.STORE_DATA_WINDOW
    assert run_hazards(tmp_path, STORE + FILL * w + "\tv_mov_b32_e32 v0, v9\n") == (1, 0)
    assert run_hazards(tmp_path, STORE + "\ts_nop %d\n" % (w - 1) + "\tv_mov_b32_e32 v3, v9\n") == (1, 0)
    # the address register and unrelated registers are free at once
    assert run_hazards(tmp_path, STORE + "\tv_mov_b32_e32 v150, v9\n\tv_mov_b32_e32 v4, v9\n") == (1, 0)


@pytest.mark.parametrize("body", [
    STORE + FILL * 3 + "\tv_accvgpr_read_b32 v0, a248\n",                                  # a plain write, too early
    STORE + "\ts_nop 7\n" + "\tv_cvt_pk_bf16_f32 v2, v4, v5\n",                               # eight idle cycles are not twelve
    STORE + FILL * 2 + "\tv_permlane16_swap_b32_e32 v9, v1\n",                              # the swap writes both operands
    STORE + FILL * 2 + "\ts_cbranch_scc1 .LBB0_2\n" + FILL * 20 + ".LBB0_2:\n\tv_mov_b32_e32 v1, v9\n",   # on the taken path
    STORE + FILL * 2 + "\ts_branch .LBB0_3\n.LBB0_3:\n\tds_read_b128 v[0:3], v123\n",
    "\tglobal_store_dwordx4 v[4:5], v[8:11], off\n" + FILL + "\tv_mov_b32_e32 v10, v9\n",   # data is the second operand there
    "\tbuffer_store_dwordx2 v[2:3], v0, s[20:23], 0 offen\n" + FILL * 4 + "\tv_mov_b32_e32 v2, v9\n",
])
def test_store_data_rewritten_too_early_is_rejected(tmp_path, body):
    with pytest.raises(RuntimeError, match="rewrites data of"):
        run_hazards(tmp_path, body)


def test_inline_mfma_results_are_left_alone_for_the_window(tmp_path):
    w = check_async_loads.MFMA_RESULT_WINDOW
    # accumulating in place into exactly the same registers is what the hardware is built for
    assert run_hazards(tmp_path, ASM_MFMA + ASM_MFMA + FILL * w + "\tv_accvgpr_read_b32 v0, a0\n") == (0, 2)
    with pytest.raises(RuntimeError, match="touches the result of"):
        run_hazards(tmp_path, ASM_MFMA + FILL * 5 + "\tv_accvgpr_read_b32 v0, a2\n")
    with pytest.raises(RuntimeError, match="touches the result of"):
        run_hazards(tmp_path, ASM_MFMA + FILL * 5 + "\tbuffer_store_dwordx4 a[0:3], v1, s[20:23], 0 offen\n")
    with pytest.raises(RuntimeError, match="touches the result of"):     # an overlapping, not identical, accumulator
        run_hazards(tmp_path, ASM_MFMA + "\t;;#ASMSTART\n\tv_mfma_f32_16x16x32_bf16 a[2:5], v[2:5], v[6:9], a[2:5]\n\t;;#ASMEND\n")
    # MFMAs the compiler emitted itself get their wait states from the compiler: not this check's business
    assert run_hazards(tmp_path, "\tv_mfma_f32_16x16x32_bf16 v[0:3], v[12:15], v[16:19], v[0:3]\n\tv_mov_b32_e32 v20, v0\n") == (0, 0)


def test_scratch_use_is_rejected(tmp_path):
    meta = "    .private_segment_fixed_size: %d\n    .vgpr_spill_count: %d\n"
    f = tmp_path / "m.s"
    f.write_text(meta % (0, 0) + meta % (0, 0))
    assert check_async_loads.check_no_scratch(str(f)) == 2
    f.write_text(meta % (0, 0) + meta % (1420, 1756))
    with pytest.raises(RuntimeError, match="uses scratch memory"):
        check_async_loads.check_no_scratch(str(f))


def test_fallback_build_of_the_block_scaled_kernel_passes_the_hazard_checks(tmp_path):
    """The block-scaled kernel's fallback build (MI355_MX_SYNC_SCALES: scale loads that wait for
    themselves, what build.py switches to when a compiler copies a scale register) compiles for
    gfx950 here, without a GPU, and its generated assembly passes the checks every build applies:
    store-data and MFMA-result distances, the copies' LDS base, no scratch.  In that object every
    scale load is followed by a wait for all outstanding vector-memory instructions."""
    import glob
    import importlib.util
    import shutil
    import subprocess
    spec = importlib.util.spec_from_file_location("_mi355_build_for_test", os.path.join(PKG, "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not (os.path.exists(hipcc) or shutil.which(hipcc)):
        pytest.skip("hipcc not found")
    src = build.CHECKED_SOURCE
    cmd = [hipcc] + build.HIPCC_FLAGS + ["-c", "-save-temps=obj", "-DMI355_MX_SYNC_SCALES", "-o",
                                         str(tmp_path / "mx_sync.o"), os.path.join(build.CSRC, src)]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    asm = glob.glob(str(tmp_path / "*-hip-amdgcn-*gfx950.s"))
    assert len(asm) == 1, asm
    stores, mfmas = check_async_loads.check_hazard_distances(asm[0])
    assert stores > 100 and mfmas > 1000
    assert check_async_loads.check_lds_base(asm[0]) > 100
    check_async_loads.check_no_scratch(asm[0])
    text = open(asm[0]).read().split("\n")
    loads = [i for i, l in enumerate(text) if l.strip().startswith("buffer_load_dwordx2")]
    assert len(loads) > 100
    for i in loads:
        assert text[i + 1].strip().startswith("s_waitcnt vmcnt(0)"), text[i:i + 2]
