"""The C-ABI library on a machine without a GPU: it loads, exports every symbol the public
header declares, validates arguments before touching the device, and its tile map is a
bijection (the invariant of the reference's Scheduler, kernels/gemm_kernels/sm90a/gemm.cuh:184-211)."""
import ctypes
import subprocess

import pytest

from tests import abi_ctypes as ac


def test_exports_every_declared_symbol(abi):
    names = ac.declared_symbols()
    assert {"mi355_gemm_tn", "mi355_gemm_tn_scaled", "mi355_quantize_e4m3", "mi355_gemm_tn_mxfp8",
            "mi355_quantize_mxfp8", "mi355_mx_shuffle_scales"} <= set(names) and len(names) >= 15
    for n in names:
        assert hasattr(abi, n), n
    dyn = subprocess.run(["nm", "-D", "--defined-only", ac.LIB], capture_output=True, text=True).stdout
    for n in names:
        assert f" T {n}" in dyn, n


def test_fallback_library_loads_and_exports_the_same_symbols():
    """The second library of the build (the block-scaled kernel in its fallback form) is a full library."""
    fallback = ac.load(ac.LIB_SYNC_SCALES)
    dyn = subprocess.run(["nm", "-D", "--defined-only", ac.LIB_SYNC_SCALES], capture_output=True, text=True).stdout
    for n in ac.declared_symbols():
        assert hasattr(fallback, n) and f" T {n}" in dyn, n
    assert fallback.mi355_gemm_mx_check(256, 256, 128, 128, 128, 256, ac.BF16) == ac.OK


def test_version_and_strerror(abi):
    assert abi.mi355_gemm_version() >= 1
    for code in range(0, -8, -1):
        msg = abi.mi355_gemm_strerror(code)
        assert msg and b"unknown status" not in msg
    assert b"unknown status" in abi.mi355_gemm_strerror(-99)


@pytest.mark.parametrize("args,want", [
    ((256, 256, 64, 64, 64, 256, ac.BF16, ac.BF16, ac.AUTO), ac.OK),
    ((256, 256, 64, 64, 64, 256, 7, ac.BF16, ac.AUTO), ac.ERR_DTYPE),
    ((256, 256, 64, 64, 64, 256, ac.BF16, ac.E4M3, ac.AUTO), ac.ERR_DTYPE),
    ((256, 256, 64, 64, 64, 256, ac.BF16, ac.BF16, 9), ac.ERR_VARIANT),
    ((-1, 256, 64, 64, 64, 256, ac.BF16, ac.BF16, ac.AUTO), ac.ERR_SHAPE),
    ((256, 256, 64, 32, 64, 256, ac.BF16, ac.BF16, ac.AUTO), ac.ERR_SHAPE),   # lda < K
    ((256, 256, 64, 64, 64, 128, ac.BF16, ac.BF16, ac.AUTO), ac.ERR_SHAPE),   # ldc < N
    ((256, 256, 72, 72, 72, 256, ac.BF16, ac.BF16, ac.BASIC), ac.OK),         # ragged last k-step
    ((256, 256, 68, 72, 72, 256, ac.BF16, ac.BF16, ac.BASIC), ac.ERR_SHAPE),  # K bytes % 16
    ((256, 256, 68, 72, 72, 256, ac.BF16, ac.BF16, ac.AUTO), ac.OK),          # AUTO falls back
    ((16, 30, 7, 7, 7, 30, ac.F16, ac.F16, ac.SIMPLE), ac.OK),
    ((256, 256, 128, 128, 128, 256, ac.E4M3, ac.BF16, ac.BASIC), ac.OK),
    ((256, 256, 64, 64, 64, 256, ac.E4M3, ac.BF16, ac.BASIC), ac.OK),         # half a k-step of fp8
    ((256, 256, 24, 32, 32, 256, ac.E4M3, ac.BF16, ac.BASIC), ac.ERR_SHAPE),  # 24 fp8 bytes % 16
    ((64, 256, 128, 128, 128, 256, ac.BF16, ac.BF16, ac.SKINNY), ac.OK),
    ((257, 256, 128, 128, 128, 256, ac.BF16, ac.BF16, ac.SKINNY), ac.ERR_SHAPE),     # M > 256
    ((64, 256, 128, 128, 128, 256, ac.E4M3, ac.BF16, ac.SKINNY), ac.OK),             # fp8 streams too
    ((0, 0, 0, 0, 0, 0, ac.BF16, ac.BF16, ac.AUTO), ac.OK),
    # 32-bit offsets inside a tile: 256 rows of A or B below 2 GiB, 256 rows of fp32 partials too
    ((256, 256, 64, 1 << 22, 64, 256, ac.BF16, ac.BF16, ac.BASIC), ac.ERR_SHAPE),
    ((256, 256, 64, 1 << 22, 64, 256, ac.BF16, ac.BF16, ac.AUTO), ac.OK),
    ((256, 256, 64, 64, 64, 1 << 21, ac.BF16, ac.BF16, ac.BASIC), ac.ERR_SHAPE),
    ((256, 256, 64, 64, 64, (1 << 21) - 4, ac.BF16, ac.BF16, ac.BASIC), ac.OK),
    ((256, 256, 64, 64, 64, 1 << 21, ac.BF16, ac.BF16, ac.AUTO), ac.OK),
])
def test_check(abi, args, want):
    assert abi.mi355_gemm_check(*args) == want


def test_sizes_beyond_any_memory_are_refused_before_any_arithmetic_on_them(abi):
    """Extents above 2^40 and arrays above 2^50 elements come back as MI355_ERR_SHAPE (0 from the
    size queries) from every entry point: products of such sizes would leave 64 bits."""
    huge = [2**62, 2**63 - 1, 2**48 + 16, 2**41]
    for h in huge:
        assert abi.mi355_gemm_check(256, 256, h, h, h, 256, ac.BF16, ac.BF16, ac.AUTO) == ac.ERR_SHAPE
        assert abi.mi355_gemm_check(h, 256, 64, 64, 64, 256, ac.BF16, ac.BF16, ac.AUTO) == ac.ERR_SHAPE
        assert abi.mi355_gemm_check(256, 256, 64, 64, 64, h, ac.BF16, ac.BF16, ac.AUTO) == ac.ERR_SHAPE
        assert abi.mi355_gemm_select_variant(8253, 160, h, ac.F16) == ac.ERR_SHAPE
        assert abi.mi355_gemm_select_variant(h, h, 64, ac.F16) == ac.ERR_SHAPE
        assert ac.plan(abi, 256, h, 256, ac.E4M3)[0] == ac.ERR_SHAPE
        assert abi.mi355_gemm_workspace_bytes(16, h, 4096, ac.BF16, ac.AUTO) == 0
        assert abi.mi355_gemm_mx_check(256, 256, h, h, h, 256, ac.BF16) == ac.ERR_SHAPE
        assert abi.mi355_gemm_mx_workspace_bytes(h, 256, 128, 0) == 0
        assert abi.mi355_mx_shuffled_bytes(h, 128) == 0
        assert abi.mi355_quantize_e4m3(None, ac.BF16, max(h, 2**50 + 1), None, None, None) == ac.ERR_SHAPE
        assert abi.mi355_quantize_mxfp8(None, ac.BF16, 4, 128, h, None, None, 0, None) == ac.ERR_SHAPE
        a, b = ctypes.c_int64(), ctypes.c_int64()
        assert abi.mi355_gemm_tile_coord(5, h, h, ctypes.byref(a), ctypes.byref(b)) == ac.ERR_SHAPE
    # 2^25 x 2^25 x 2^25 is within the bound (2^50 elements per array): the queries answer
    assert abi.mi355_gemm_select_variant(2**25, 2**25, 2**25, ac.BF16) == ac.SIMPLE      # rows too long for the tiled kernels
    assert abi.mi355_gemm_select_variant(2**26, 2**25, 64, ac.BF16) == ac.ERR_SHAPE     # C would have 2^51 elements
    assert abi.mi355_gemm_tile_coord(5, 2**29, 2**29, ctypes.byref(a), ctypes.byref(b)) == ac.OK


def test_gemm_tn_rejects_before_any_device_access(abi):
    """Bad arguments and NULL pointers come back as codes without a GPU present."""
    f = abi.mi355_gemm_tn
    assert f(None, None, None, 256, 256, 64, 64, 64, 256, 0, 0, 1.0, 0, None, 0, None) == ac.ERR_NULL
    assert f(None, None, None, 256, 256, 64, 64, 64, 256, 5, 0, 1.0, 0, None, 0, None) == ac.ERR_DTYPE
    assert f(None, None, None, 256, 256, 64, 8, 64, 256, 0, 0, 1.0, 0, None, 0, None) == ac.ERR_SHAPE
    assert f(None, None, None, 0, 256, 64, 64, 64, 256, 0, 0, 1.0, 0, None, 0, None) == ac.OK  # empty


def test_quantize_rejects_before_any_device_access(abi):
    f = abi.mi355_quantize_e4m3
    assert f(None, ac.F32, 16, None, None, None) == ac.ERR_NULL
    assert f(None, ac.E4M3, 16, None, None, None) == ac.ERR_DTYPE
    assert f(None, ac.F32, -1, None, None, None) == ac.ERR_SHAPE
    assert f(17, ac.F32, 16, 8, 12, None) == ac.ERR_ALIGN


@pytest.mark.parametrize("args,want", [
    ((256, 256, 128, 128, 128, 256, ac.BF16), ac.OK),
    ((100, 260, 1024, 1024, 1040, 264, ac.F16), ac.OK),
    ((256, 256, 64, 64, 64, 256, ac.BF16), ac.ERR_SHAPE),            # K % 128
    ((256, 256, 128, 120, 128, 256, ac.BF16), ac.ERR_SHAPE),         # lda < K
    ((256, 258, 128, 128, 128, 258, ac.BF16), ac.ERR_SHAPE),         # N % 4
    ((256, 256, 128, 128, 128, 256, ac.E4M3), ac.ERR_DTYPE),
    ((0, 256, 128, 128, 128, 256, ac.BF16), ac.OK),
    ((1 << 20, 256, 1 << 17, 1 << 17, 1 << 17, 256, ac.BF16), ac.ERR_SHAPE),   # 4 GiB of scales for A
])
def test_mx_check(abi, args, want):
    assert abi.mi355_gemm_mx_check(*args) == want


def test_mx_sizes_and_rejections_before_any_device_access(abi):
    assert abi.mi355_mx_shuffled_bytes(256, 128) == 256 * 4
    assert abi.mi355_mx_shuffled_bytes(257, 1024) == 512 * 32       # rows padded to whole 256-row tiles
    assert abi.mi355_mx_shuffled_bytes(256, 96) == 0                 # K % 128
    assert abi.mi355_gemm_mx_workspace_bytes(300, 100, 256, 0) == (512 + 256) * 8
    assert abi.mi355_gemm_mx_workspace_bytes(300, 100, 256, 1) == 0
    # partial results of the planner's K split (32 tiles of 256x128 cut in seven) or tail split
    # (384 tiles of 256x256) behind the shuffled scales; the plan is the one for plain e4m3 among the
    # tiles the block-scaled kernel has (plain operands may get the nine-slot ring instead)
    assert ac.plan(abi, 256, 4096, 14336, ac.E4M3)[1:4] == (128, 128, 4)
    assert abi.mi355_gemm_mx_workspace_bytes(256, 4096, 14336, 1) == 7 * 256 * 4096 * 4
    assert abi.mi355_gemm_mx_workspace_bytes(256, 4096, 14336, 0) == 7 * 256 * 4096 * 4 + (256 + 4096) * 448
    assert abi.mi355_gemm_mx_workspace_bytes(6144, 4096, 4096, 1) == 2 * 128 * 256 * 256 * 4      # tail split: 128 tiles cut in two
    assert abi.mi355_gemm_mx_workspace_bytes(4096, 6144, 4096, 1) == 0                              # two launches instead
    assert abi.mi355_gemm_mx_workspace_bytes(512, 6144, 4096, 1) == 0      # 192 tiles of 128x128, unsplit
    f = abi.mi355_gemm_tn_mxfp8
    assert f(None, None, None, 256, 256, 128, 128, 128, 256, None, 4, None, 4, 0, ac.BF16, None, 0, None) == ac.ERR_NULL
    assert f(None, None, None, 256, 256, 100, 128, 128, 256, None, 4, None, 4, 0, ac.BF16, None, 0, None) == ac.ERR_SHAPE
    assert f(None, None, None, 0, 256, 128, 128, 128, 256, None, 4, None, 4, 0, ac.BF16, None, 0, None) == ac.OK
    assert f(16, 16, 16, 256, 256, 128, 128, 128, 256, 16, 2, 16, 4, 0, ac.BF16, 16, 1 << 20, None) == ac.ERR_SHAPE  # ld_scale < K/32
    assert f(16, 16, 16, 256, 256, 128, 128, 128, 256, 16, 4, 16, 4, 0, ac.BF16, 16, 100, None) == ac.ERR_WORKSPACE
    assert f(24, 16, 16, 256, 256, 128, 128, 128, 256, 16, 4, 16, 4, 1, ac.BF16, None, 0, None) == ac.ERR_ALIGN
    assert abi.mi355_mx_shuffle_scales(None, 256, 128, 4, None, None) == ac.ERR_NULL
    assert abi.mi355_mx_shuffle_scales(None, 256, 96, 4, None, None) == ac.ERR_SHAPE
    assert abi.mi355_quantize_mxfp8(None, ac.BF16, 4, 64, 64, None, None, 0, None) == ac.ERR_NULL
    assert abi.mi355_quantize_mxfp8(None, ac.E4M3, 4, 64, 64, None, None, 0, None) == ac.ERR_DTYPE
    assert abi.mi355_quantize_mxfp8(None, ac.BF16, 4, 48, 48, None, None, 0, None) == ac.ERR_SHAPE
    assert abi.mi355_quantize_mxfp8(None, ac.BF16, 4, 64, 64, None, None, 1, None) == ac.ERR_SHAPE   # shuffled: K % 128
    assert abi.mi355_quantize_mxfp8(16, ac.BF16, 4, 64, 68, 16, 16, 0, None) == ac.ERR_ALIGN


def test_workspace_bytes(abi):
    f = abi.mi355_gemm_workspace_bytes
    assert f(8192, 8192, 8192, ac.BF16, ac.AUTO) == 0
    assert f(8192, 8192, 8192, ac.BF16, ac.BASIC) == 0
    assert f(8192, 8192, 8192, ac.BF16, ac.PINGPONG) == 0
    assert f(256, 4096, 14336, ac.BF16, ac.BASIC) == 8 * 256 * 4096 * 4        # 32 tiles of 256x128 -> 8 K splits
    assert ac.plan(abi, 256, 4096, 14336, ac.BF16, ac.BASIC) == (ac.BASIC, 256, 128, 8, 0, 1)
    assert f(16, 512, 128, ac.BF16, ac.SKINNY) == 0              # too few k-steps to split
    need = f(16, 4096, 14336, ac.BF16, ac.AUTO)
    assert need > 0 and need % (16 * 4096 * 4) == 0 and need // (16 * 4096 * 4) <= 16
    assert f(16, 4096, 14336, ac.BF16, ac.PINGPONG) == 0
    assert f(16, 4096, 14336, ac.E4M3, ac.AUTO) == f(16, 4096, 14336, ac.E4M3, ac.SKINNY) > 0  # fp8 streams too
    assert f(16, 4096, 14336, ac.E4M3, ac.BASIC) > 0                                           # tiled kernel + K splits
    assert f(-1, 4096, 14336, ac.BF16, ac.AUTO) == 0 and f(16, 4096, 14336, 9, ac.AUTO) == 0
    # tail split: 384 tiles of 256 -> the 128 of the second round are cut in two along K
    assert f(4096, 6144, 4096, ac.BF16, ac.BASIC) == f(4096, 6144, 4096, ac.BF16, ac.AUTO) == 2 * 128 * 256 * 256 * 4
    assert f(4096, 6144, 1024, ac.BF16, ac.BASIC) == 0          # 16 k-steps: too short to cut
    assert f(4096, 7168, 4096, ac.BF16, ac.BASIC) == 0          # 448 tiles: the last round is 3/4 full
    assert f(4352, 4352, 4096, ac.BF16, ac.BASIC) == 4 * 33 * 256 * 256 * 4    # 289 tiles: 33 cut in four
    assert f(4352, 4352, 1024, ac.BF16, ac.BASIC) == 0          # too short to cut: runs on 128x128 tiles
    assert f(6144, 6144, 6144, ac.BF16, ac.BASIC) == 4 * 64 * 256 * 256 * 4    # two full rounds + 64 tiles cut in four
    assert f(4096, 14336, 4096, ac.BF16, ac.BASIC) == 0         # three full rounds: not worth it
    assert f(4096, 6144, 4096, ac.BF16, ac.PINGPONG) == 0


def test_plan(abi):
    """mi355_gemm_plan reports what a call would launch; the workspace query must agree with it."""
    assert ac.plan(abi, 8192, 8192, 8192, ac.BF16) == (ac.BASIC, 256, 256, 1, 0, 1)
    assert ac.plan(abi, 8192, 8192, 8192, ac.E4M3, ac.PINGPONG) == (ac.PINGPONG, 256, 256, 1, 0, 1)
    assert ac.plan(abi, 4096, 6144, 4096, ac.BF16) == (ac.BASIC, 256, 256, 1, 128, 2)       # tail split
    assert ac.plan(abi, 512, 14336, 4096, ac.BF16) == (ac.BASIC, 256, 128, 1, 0, 1)         # 224 rectangular tiles
    assert ac.plan(abi, 2048, 2048, 2048, ac.F16) == (ac.BASIC, 128, 128, 1, 0, 1)          # 256 small tiles
    assert ac.plan(abi, 512, 6144, 4096, ac.BF16) == (ac.BASIC, 128, 128, 1, 0, 1)          # 192 small tiles in one round
    assert ac.plan(abi, 256, 6144, 4096, ac.BF16) == (ac.BASIC, 256, 128, 4, 0, 1)          # 48 tiles cut in four
    v, rows, cols, splits, _, _ = ac.plan(abi, 16, 6144, 4096, ac.BF16)
    assert (v, rows, cols) == (ac.SKINNY, 16, 64) and splits >= 2
    # 224 tiles of 64 columns: (nearly) one per CU, so no K split (the kernel then runs a deeper ring)
    assert ac.plan(abi, 16, 14336, 4096, ac.BF16) == (ac.SKINNY, 16, 64, 1, 0, 1)
    assert ac.plan(abi, 64, 14336, 4096, ac.E4M3) == (ac.SKINNY, 64, 64, 1, 0, 1)
    assert ac.plan(abi, 16, 28672, 4096, ac.BF16)[3] == 1        # 448 tiles: two per CU at this height
    # 33...64 rows: tiles of 128 columns where they make one unsplit round, or with enough k-steps per split
    assert ac.plan(abi, 64, 28672, 4096, ac.BF16) == (ac.SKINNY, 64, 128, 1, 0, 1)
    assert ac.plan(abi, 48, 8192, 8192, ac.BF16) == (ac.SKINNY, 64, 128, 4, 0, 1)
    assert ac.plan(abi, 64, 8192, 2048, ac.BF16)[1:3] == (64, 64)     # 32 k-steps: too few
    assert ac.plan(abi, 64, 8192, 4096, ac.E4M3)[1:3] == (64, 64)     # the same in fp8
    assert ac.plan(abi, 64, 8192, 8192, ac.E4M3)[1:3] == (64, 128)
    assert ac.plan(abi, 64, 18432, 2048, ac.BF16)[1:3] == (64, 128)   # 288 narrow tiles would not fit one round
    assert ac.plan(abi, 64, 6144, 4096, ac.BF16)[1:3] == (64, 128)    # 48 wide tiles of 64 k-steps
    assert ac.plan(abi, 64, 3072, 8192, ac.BF16)[1:3] == (64, 128)    # 24 of 128 k-steps
    assert ac.plan(abi, 64, 3072, 4096, ac.BF16)[1:3] == (64, 64)
    assert ac.plan(abi, 64, 14336, 4096, ac.BF16)[1:3] == (64, 64)    # 224 narrow tiles: one unsplit round
    assert ac.plan(abi, 16, 17408, 4096, ac.BF16)[1:3] == (64, 128)
    assert ac.plan(abi, 32, 28672, 4096, ac.BF16)[1:3] == (32, 64)
    assert ac.plan(abi, 16, 24576, 4096, ac.BF16) == (ac.SKINNY, 64, 128, 1, 0, 1)   # the wide tile has 64 rows only
    # 65...128 rows against 4096...32768 columns: the tile kernel, one row of 128x128 tiles, K split
    assert ac.plan(abi, 128, 8192, 4096, ac.BF16) == (ac.BASIC, 128, 128, 4, 0, 1)
    assert ac.plan(abi, 100, 4100, 8200, ac.F16) == (ac.BASIC, 128, 128, 7, 0, 1)      # 33 tiles, 129 k-steps
    assert ac.plan(abi, 96, 2048, 4096, ac.BF16)[0] == ac.SKINNY                        # 16 tiles, 64 k-steps: streams
    assert ac.plan(abi, 96, 8192, 8192, ac.E4M3) == (ac.BASIC, 128, 128, 4, 0, 1)       # 64 tiles of 64 k-steps, in four parts
    assert ac.plan(abi, 96, 4096, 4096, ac.E4M3)[0] == ac.SKINNY                        # 32 tiles x 2 parts: too few items
    # one column of 128x128 tiles under many rows: the same ring
    assert ac.plan(abi, 32768, 128, 4096, ac.BF16) == (ac.BASIC, 128, 128, 1, 0, 1)
    assert ac.plan(abi, 8192, 96, 8192, ac.E4M3) == (ac.BASIC, 128, 128, 4, 0, 1)
    assert ac.plan(abi, 100, 30, 77, ac.BF16)[0] == ac.SIMPLE
    assert ac.plan(abi, 256, 256, 68, ac.BF16, ac.BASIC)[0] == ac.ERR_SHAPE
    assert ac.plan(abi, 256, 256, 64, 7)[0] == ac.ERR_DTYPE
    assert abi.mi355_gemm_plan(256, 256, 64, ac.BF16, ac.AUTO, None, None, None, None, None) == ac.BASIC
    for dt, es in ((ac.BF16, 2), (ac.E4M3, 1)):
        for (M, N, K) in [(512, 6144, 4096), (1024, 6144, 4096), (256, 4096, 14336), (768, 768, 8192), (4352, 4352, 4096),
                          (300, 1000, 2048), (6144, 6144, 6144), (64, 4096, 14336)]:
            v, rows, cols, splits, tail_tiles, tail_splits = ac.plan(abi, M, N, K, dt)
            want = splits * M * N * 4 if splits > 1 else tail_tiles * tail_splits * rows * cols * 4
            assert abi.mi355_gemm_workspace_bytes(M, N, K, dt, ac.AUTO) == want, (dt, M, N, K)


def test_workspace_for_repacking_misaligned_problems(abi):
    """AUTO asks for room to repack a large problem the tiled kernels cannot address; small ones
    and explicit variants get nothing."""
    f = abi.mi355_gemm_workspace_bytes
    r256 = lambda x: -(-x // 256) * 256
    # N % 4 != 0: B gets 3 zero rows, C a padded copy with rows of a multiple of 64 elements; A stays where it is
    assert f(1000, 50257, 768, ac.BF16, ac.AUTO) == r256(50260 * 768 * 2) + r256(1000 * 50304 * 2) + \
        f(1000, 50260, 768, ac.BF16, ac.AUTO)
    # K*2 % 16 != 0: A and B repacked to K = 1008 in rows of 1024 elements (a multiple of 128 bytes),
    # N = 1003 -> 1004 in rows of 1024
    assert f(1001, 1003, 1001, ac.BF16, ac.AUTO) == r256(1001 * 1024 * 2) + r256(1004 * 1024 * 2) + r256(1001 * 1024 * 2) + \
        f(1001, 1004, 1008, ac.BF16, ac.AUTO)
    assert f(100, 30, 77, ac.BF16, ac.AUTO) == 0                   # too small to bother
    assert f(1001, 1003, 1001, ac.BF16, ac.SIMPLE) == 0


def test_select_variant(abi):
    assert abi.mi355_gemm_select_variant(8192, 8192, 8192, ac.BF16) in (ac.BASIC, ac.PINGPONG)
    assert abi.mi355_gemm_select_variant(16, 14336, 4096, ac.BF16) == ac.SKINNY
    assert abi.mi355_gemm_select_variant(64, 4096, 14336, ac.F16) == ac.SKINNY
    assert abi.mi355_gemm_select_variant(256, 4096, 14336, ac.F16) == ac.BASIC   # 128x128 tiles + K splits
    assert abi.mi355_gemm_select_variant(16, 14336, 4096, ac.E4M3) == ac.SKINNY
    assert abi.mi355_gemm_select_variant(256, 14336, 4096, ac.E4M3) == ac.BASIC
    assert abi.mi355_gemm_select_variant(100, 30, 77, ac.BF16) == ac.SIMPLE
    assert abi.mi355_gemm_select_variant(8192, 8192, 8192, 9) == ac.ERR_DTYPE


def test_alternate_variant_in_the_plan(abi):
    """Two workgroups per CU on 256x128 tiles: AUTO takes it for 16-bit inputs with at most four
    k-steps and at least 1024 tiles (tiles that are nearly all epilogue); explicitly it takes any
    problem the tiled kernels take, except fp8; it never wants a workspace."""
    sel = abi.mi355_gemm_select_variant
    assert sel(8192, 8192, 256, ac.BF16) == ac.ALTERNATE
    assert sel(16384, 16384, 128, ac.F16) == ac.ALTERNATE
    assert sel(4096, 8192, 200, ac.BF16) == ac.ALTERNATE          # 16 x 64 tiles, four k-steps (the last ragged)
    assert sel(8192, 8192, 320, ac.BF16) == ac.BASIC              # five k-steps
    assert sel(4096, 4096, 256, ac.BF16) == ac.BASIC              # 512 tiles: one per workgroup
    assert sel(8192, 8192, 256, ac.E4M3) == ac.BASIC              # fp8: two k-steps, but no such kernel
    assert sel(64, 4096 * 128, 256, ac.BF16) == ac.SKINNY         # few rows: the streaming kernel comes first
    assert ac.plan(abi, 8192, 8192, 256, ac.BF16) == (ac.ALTERNATE, 256, 128, 1, 0, 1)
    assert ac.plan(abi, 1000, 1004, 4096, ac.F16, ac.ALTERNATE) == (ac.ALTERNATE, 256, 128, 1, 0, 1)
    assert ac.plan(abi, 8192, 8192, 8192, ac.E4M3, ac.ALTERNATE)[0] == ac.ERR_VARIANT
    assert abi.mi355_gemm_check(512, 512, 64, 64, 64, 512, ac.E4M3, ac.BF16, ac.ALTERNATE) == ac.ERR_VARIANT
    assert abi.mi355_gemm_check(512, 512, 68, 68, 68, 512, ac.BF16, ac.BF16, ac.ALTERNATE) == ac.ERR_SHAPE   # K bytes % 16
    assert abi.mi355_gemm_check(512, 512, 72, 72, 72, 512, ac.BF16, ac.F16, ac.ALTERNATE) == ac.OK
    assert abi.mi355_gemm_check(512, 512, 72, 72, 72, 512, ac.BF16, ac.F16, 6) == ac.ERR_VARIANT
    for M, N, K in [(8192, 8192, 256), (8192, 8192, 8192), (300, 200, 64)]:
        assert abi.mi355_gemm_workspace_bytes(M, N, K, ac.BF16, ac.ALTERNATE) == 0
    assert abi.mi355_gemm_workspace_bytes(8192, 8192, 256, ac.BF16, ac.AUTO) == 0


@pytest.mark.parametrize("tm,tn", [(32, 32), (16, 16), (1, 1), (1, 56), (3, 5), (7, 9), (33, 31), (2, 24), (17, 1),
                                   (17, 17), (17, 16), (64, 64)])
def test_tile_map_is_a_bijection(abi, tm, tn):
    seen = set()
    a, b = ctypes.c_int64(), ctypes.c_int64()
    for blk in range(tm * tn):
        assert abi.mi355_gemm_tile_coord(blk, tm, tn, ctypes.byref(a), ctypes.byref(b)) == 0
        assert 0 <= a.value < tm and 0 <= b.value < tn
        seen.add((a.value, b.value))
    assert len(seen) == tm * tn
    assert abi.mi355_gemm_tile_coord(tm * tn, tm, tn, ctypes.byref(a), ctypes.byref(b)) == ac.ERR_SHAPE


def test_tile_map_keeps_an_xcd_compact(abi):
    """Blocks b, b+8, b+16, ... run on one XCD.  The 32 that are co-resident at the start must
    touch few distinct A and B panels so they share them through that XCD's L2."""
    tm = tn = 32
    a, b = ctypes.c_int64(), ctypes.c_int64()
    for xcd in range(8):
        rows, cols = set(), set()
        for i in range(32):
            abi.mi355_gemm_tile_coord(xcd + 8 * i, tm, tn, ctypes.byref(a), ctypes.byref(b))
            rows.add(a.value)
            cols.add(b.value)
        assert len(rows) + len(cols) <= 12, (xcd, rows, cols)


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """The public header compiles as C99 and as C++, and a C program linked against the library
    can call the entry points that need no GPU."""
    import os
    src = tmp_path / "use_abi.c"
    src.write_text(r'''
#include <stdio.h>
#include "mi355_gemm.h"
int main(void) {
  int rows, cols, splits, tail_tiles, tail_splits;
  int v = mi355_gemm_plan(4096, 6144, 4096, MI355_BF16, MI355_VARIANT_AUTO, &rows, &cols, &splits, &tail_tiles, &tail_splits);
  if (mi355_gemm_version() < 1) return 1;
  if (mi355_gemm_check(256, 256, 64, 64, 64, 256, MI355_BF16, MI355_BF16, MI355_VARIANT_AUTO) != MI355_OK) return 2;
  if (mi355_gemm_tn(NULL, NULL, NULL, 256, 256, 64, 64, 64, 256, MI355_BF16, MI355_BF16, 1.0f, MI355_VARIANT_AUTO, NULL, 0, NULL) != MI355_ERR_NULL) return 3;
  printf("%d %d %d %d %d %d %s\n", v, rows, cols, splits, tail_tiles, tail_splits, mi355_gemm_strerror(MI355_ERR_SHAPE));
  return 0;
}
''')
    inc = os.path.dirname(ac.HEADER)
    libdir = os.path.dirname(ac.LIB)
    exe = tmp_path / "use_abi"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", inc, str(src), "-o", str(exe),
                    "-L", libdir, "-l:libmi355gemm.so", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split(None, 6)
    assert [int(x) for x in out[:6]] == [ac.BASIC, 256, 256, 1, 128, 2] and "constraint" in out[6]
    subprocess.run(["g++", "-std=c++11", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", "-I", inc, ac.HEADER], check=True)


def test_plan_invariants_over_random_shapes(abi):
    """3000 seeded random problems per input type: whatever the planner picks must be launchable as
    the kernels assume (splits divide the k-steps and leave at least 16, split items fit the CUs,
    a tail split only on 256x256 tiles and only for the tiles of the last round) and the workspace
    query must match it."""
    import random
    rng = random.Random(7)
    seen = set()
    seen_pieces = set()
    seen_alternate = False
    for dt, es in ((ac.BF16, 2), (ac.F16, 2), (ac.E4M3, 1)):
        for _ in range(3000):
            M = rng.choice([rng.randint(1, 300), rng.randint(1, 5000), rng.randint(1, 20000)])
            N = 4 * rng.choice([rng.randint(1, 100), rng.randint(1, 2000), rng.randint(1, 8000)])
            K = (16 // es) * rng.choice([rng.randint(1, 64), rng.randint(1, 1024), rng.randint(1, 4096)])
            v, rows, cols, splits, tail_tiles, tail_splits = ac.plan(abi, M, N, K, dt)
            steps = -(-K * es // 128)
            # two workgroups per CU: 16-bit inputs, at most four k-steps, at least 1024 tiles of 256x128
            alternates = es == 2 and steps <= 4 and -(-M // 256) * -(-N // 128) >= 1024
            if v == ac.ALTERNATE:
                assert alternates and (rows, cols, splits, tail_tiles) == (256, 128, 1, 0), (M, N, K)
                assert abi.mi355_gemm_workspace_bytes(M, N, K, dt, ac.AUTO) == 0
                seen_alternate = True
                continue
            assert v in (ac.BASIC, ac.SKINNY) and (not alternates or v == ac.SKINNY), (M, N, K, v)
            one_row = -(-N // 128)      # 65...128 rows: one row of 128x128 tiles on the nine-slot ring
            parts = max([1] + [p for p in range(2, 17) if one_row * p <= 256 and steps // p >= 16])
            deep = M <= 128 and one_row <= 256 and one_row * parts >= 96 and (one_row >= 32 or (one_row >= 16 and steps >= 128))
            assert (v == ac.SKINNY) == (M <= 64 or (not deep and M <= 128 and -(-N // 64) <= 256 and M * K * es <= 2200000))
            if deep and M > 64:
                assert (v, rows, cols) == (ac.BASIC, 128, 128), (M, N, K)
            # Two launches: the plan describes the first piece, a whole number of rounds of 256 x 256 tiles cut off
            # along one axis; the workspace is what the hungrier piece wants on the tile kernel.
            first_rows, first_cols = ctypes.c_int64(), ctypes.c_int64()
            pieces = abi.mi355_gemm_pieces(M, N, K, dt, ac.AUTO, ctypes.byref(first_rows), ctypes.byref(first_cols))
            Mp, Np = first_rows.value, first_cols.value
            assert pieces in (1, 2) and (pieces == 2) == ((Mp, Np) != (M, N))
            if pieces == 2:
                seen_pieces.add(Mp != M)
                assert v == ac.BASIC and steps >= 16 and (Mp == M) != (Np == N) and 0 < Mp <= M and 0 < Np <= N
                assert (Mp if Mp != M else Np) % 256 == 0 and (-(-Mp // 256) * -(-Np // 256)) % 256 == 0
                assert (-(-M // 256) * -(-N // 256)) % 256 != 0
                rest = (M - Mp, N) if Mp != M else (M, N - Np)
                assert abi.mi355_gemm_pieces(Mp, Np, K, dt, ac.BASIC, None, None) == 1      # explicit variants never cut
            M_all, N_all, M, N = M, N, Mp, Np
            tiles = -(-M // rows) * -(-N // cols)
            assert splits >= 1 and tail_splits >= 1 and tail_tiles >= 0
            if splits > 1:
                assert tail_tiles == 0, (M, N, K, splits)      # the k-steps need not divide: cuts differ by one k-step
                assert steps // splits >= (16 if v == ac.BASIC else 8), (M, N, K, splits)
            want = splits * M * N * 4 if splits > 1 else 0
            if v == ac.BASIC:
                assert (rows, cols) in ((256, 256), (256, 128), (128, 128))
                if splits > 1:
                    assert tiles * splits <= 256
                if tail_tiles:
                    assert (rows, cols) == (256, 256) and splits == 1 and tail_splits > 1
                    assert 256 <= tiles <= 3 * 256 and tail_tiles == tiles % 256
                    assert tail_tiles * tail_splits <= 256 and steps // tail_splits >= 16      # uneven cuts allowed
                    want = tail_tiles * tail_splits * 256 * 256 * 4
                seen.add((rows, cols, splits > 1, tail_tiles > 0))
            if pieces == 2:
                assert abi.mi355_gemm_workspace_bytes(M, N, K, dt, ac.BASIC) == want, (M, N, K)
                want = max(want, abi.mi355_gemm_workspace_bytes(rest[0], rest[1], K, dt, ac.BASIC))
            assert abi.mi355_gemm_workspace_bytes(M_all, N_all, K, dt, ac.AUTO) == want, (M_all, N_all, K)
    assert len(seen) >= 7 and seen_alternate and seen_pieces == {False, True}, (seen, seen_pieces)


def test_noalloc_entry_point_decides_before_any_hip_call(abi):
    """mi355_gemm_tn_noalloc runs its argument checks and the does-it-fit decision before it touches
    the device, so both can be provoked here: the pointers only need to look aligned."""
    p = 1 << 20
    f = abi.mi355_gemm_tn_noalloc
    assert f(None, p, p, 256, 256, 64, 64, 64, 256, ac.BF16, ac.BF16, 1.0, ac.AUTO, None) == ac.ERR_NULL
    assert f(p, p, p, 256, 256, 64, 32, 64, 256, ac.BF16, ac.BF16, 1.0, ac.AUTO, None) == ac.ERR_SHAPE
    assert f(p, p, p, 256, 256, 64, 64, 64, 256, ac.BF16, ac.BF16, 1.0, 9, None) == ac.ERR_VARIANT
    assert f(p, p, p, 0, 256, 64, 64, 64, 256, ac.BF16, ac.BF16, 1.0, ac.AUTO, None) == ac.OK      # nothing to do
    # a misaligned problem whose repacked operands (400 MB) are beyond the 64 MiB buffer
    assert abi.mi355_gemm_workspace_bytes(8191, 8193, 8190, ac.BF16, ac.AUTO) > ac.NOALLOC_SCRATCH_BYTES
    assert f(p, p, p, 8191, 8193, 8190, 8190, 8190, 8193, ac.BF16, ac.BF16, 1.0, ac.AUTO, None) == ac.ERR_SCRATCH
    assert b"MI355_NOALLOC_SCRATCH_BYTES" in abi.mi355_gemm_strerror(ac.ERR_SCRATCH)
    # split partials never exceed the buffer: at most 256 split items of at most 256 x 256 floats
    import random
    rng = random.Random(11)
    for _ in range(2000):
        M, N, K = rng.randint(1, 20000), 4 * rng.randint(1, 8000), 16 * rng.randint(1, 2048)   # aligned: no repacking
        for dt in (ac.BF16, ac.E4M3):
            assert abi.mi355_gemm_workspace_bytes(M, N, K, dt, ac.AUTO) <= ac.NOALLOC_SCRATCH_BYTES, (M, N, K, dt)
