"""The build-time check of the block-scaled kernel's generated assembly (cute-examples_amd/
check_async_loads.py) on hand-written instruction streams: it must accept scale registers that go
from the asynchronous load straight into scaled MFMAs and reject any other reader in between."""
import os
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cute-examples_amd"))
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


def test_lds_swizzle_is_a_bijection_and_conflict_free():
    """CPU model of the LDS layout of the tile kernels (the counterpart of the reference's swizzled
    shared-memory layouts, kernels/gemm_kernels/sm90a/gemm.cuh:420-451).  A row is 128 bytes = 8
    chunks of 16; chunk c of row r is stored at chunk c ^ swizzle(r).  Checked: the map is a
    bijection on a 256-row slot; what the direct-to-LDS copies write (lane l of a copy lands at
    16*l and fetches global chunk (l%8) ^ swizzle(row)) is exactly that layout; and every
    ds_read_b128 the kernels issue is conflict-free under the model that such a read is served 16
    lanes at a time from 64 four-byte banks (the hardware counter SQ_LDS_BANK_CONFLICT reads 0 on
    the real kernels)."""
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

    def conflict_free(lane_addresses):
        for q in range(0, 64, 16):        # 16 lanes x 16 bytes = all 64 banks once
            banks = set()
            for a in lane_addresses[q:q + 16]:
                for b in range(4):
                    banks.add((a // 4 + b) % 64)
            if len(banks) != 64:
                return False
        return True

    # fragment reads: lane l reads row (block base + l%16); group l/16 picks the logical chunk
    patterns = {
        "16-bit, slice s": lambda s, g, e: s * 4 + g,
        "fp8, two chunks per lane": lambda s, g, e: 2 * g + e,
        "block-scaled fp8": lambda s, g, e: g + 4 * e,
    }
    for name, chunk_of in patterns.items():
        for base in range(0, rows, 16):
            for s in range(2):
                for e in range(2):
                    addrs = [address(base + l % 16, chunk_of(s, l // 16, e)) for l in range(64)]
                    assert conflict_free(addrs), (name, base, s, e)
    # and the layout without the swizzle would conflict, so the check has teeth
    plain = [(l % 16) * 128 + (l // 16) * 16 for l in range(64)]
    assert not conflict_free(plain)


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
