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
