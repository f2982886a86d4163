"""ctypes view of include/mi355_gemm.h for the tests (and a model of the stub a non-Python host
would write).  Loads the in-tree library; raises if it has not been built."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "cute-examples_amd", "gemm_kernels", "libmi355gemm.so")
LIB_SYNC_SCALES = os.path.join(ROOT, "cute-examples_amd", "gemm_kernels", "libmi355gemm_syncscales.so")
HEADER = os.path.join(ROOT, "include", "mi355_gemm.h")

BF16, F16, E4M3, F32 = 0, 1, 2, 3
AUTO, BASIC, PINGPONG, SKINNY, SIMPLE, ALTERNATE = 0, 1, 2, 3, 4, 5
OK, ERR_NULL, ERR_DTYPE, ERR_SHAPE, ERR_VARIANT, ERR_WORKSPACE, ERR_LAUNCH, ERR_ALIGN, ERR_SCRATCH = 0, -1, -2, -3, -4, -5, -6, -7, -8
NOALLOC_SCRATCH_BYTES = 64 << 20


def declared_symbols():
    """Function names declared in the public header."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def load(path=LIB):
    if not os.path.exists(path):
        raise RuntimeError(os.path.basename(path) + " is not built; run python cute-examples_amd/build.py")
    L = ctypes.CDLL(path)
    i64, vp, ci, f32, sz = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
    L.mi355_gemm_tn.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, f32, ci, vp, sz, vp]
    L.mi355_gemm_tn.restype = ci
    L.mi355_gemm_tn_scaled.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, f32, vp, vp, ci, vp, sz, vp]
    L.mi355_gemm_tn_scaled.restype = ci
    L.mi355_gemm_tn_noalloc.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, f32, ci, vp]
    L.mi355_gemm_tn_noalloc.restype = ci
    L.mi355_quantize_e4m3.argtypes = [vp, ci, i64, vp, vp, vp]
    L.mi355_quantize_e4m3.restype = ci
    u8p = vp
    L.mi355_gemm_tn_mxfp8.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, u8p, i64, u8p, i64, ci, ci, vp, sz, vp]
    L.mi355_gemm_tn_mxfp8.restype = ci
    L.mi355_gemm_mx_workspace_bytes.argtypes = [i64, i64, i64, ci]
    L.mi355_gemm_mx_workspace_bytes.restype = sz
    L.mi355_gemm_mx_check.argtypes = [i64, i64, i64, i64, i64, i64, ci]
    L.mi355_gemm_mx_check.restype = ci
    L.mi355_mx_shuffle_scales.argtypes = [u8p, i64, i64, i64, u8p, vp]
    L.mi355_mx_shuffle_scales.restype = ci
    L.mi355_mx_shuffled_bytes.argtypes = [i64, i64]
    L.mi355_mx_shuffled_bytes.restype = sz
    L.mi355_quantize_mxfp8.argtypes = [vp, ci, i64, i64, i64, vp, u8p, ci, vp]
    L.mi355_quantize_mxfp8.restype = ci
    L.mi355_gemm_workspace_bytes.argtypes = [i64, i64, i64, ci, ci]
    L.mi355_gemm_workspace_bytes.restype = sz
    ip = ctypes.POINTER(ctypes.c_int)
    L.mi355_gemm_plan.argtypes = [i64, i64, i64, ci, ci, ip, ip, ip, ip, ip]
    L.mi355_gemm_plan.restype = ci
    L.mi355_gemm_pieces.argtypes = [i64, i64, i64, ci, ci, ctypes.POINTER(i64), ctypes.POINTER(i64)]
    L.mi355_gemm_pieces.restype = ci
    L.mi355_gemm_select_variant.argtypes = [i64, i64, i64, ci]
    L.mi355_gemm_select_variant.restype = ci
    L.mi355_gemm_check.argtypes = [i64, i64, i64, i64, i64, i64, ci, ci, ci]
    L.mi355_gemm_check.restype = ci
    L.mi355_gemm_tile_coord.argtypes = [i64, i64, i64, ctypes.POINTER(i64), ctypes.POINTER(i64)]
    L.mi355_gemm_tile_coord.restype = ci
    L.mi355_calibrate_sink_bytes.argtypes = []
    L.mi355_calibrate_sink_bytes.restype = sz
    L.mi355_calibrate_mfma.argtypes = [ci, vp, sz, vp, sz, ci, vp, ctypes.POINTER(ctypes.c_double), vp]
    L.mi355_calibrate_mfma.restype = ci
    L.mi355_calibrate_mfma_shape.argtypes = [ci, ci, vp, sz, vp, sz, ci, vp, ctypes.POINTER(ctypes.c_double), vp]
    L.mi355_calibrate_mfma_shape.restype = ci
    L.mi355_calibrate_read.argtypes = [vp, sz, vp, vp]
    L.mi355_calibrate_read.restype = ci
    L.mi355_clock_probe_bytes.argtypes = [ci, ci]
    L.mi355_clock_probe_bytes.restype = sz
    L.mi355_clock_probe.argtypes = [ci, ci, ci, vp, vp]
    L.mi355_clock_probe.restype = ci
    L.mi355_gemm_strerror.argtypes = [ci]
    L.mi355_gemm_strerror.restype = ctypes.c_char_p
    L.mi355_gemm_version.argtypes = []
    L.mi355_gemm_version.restype = ci
    return L


def torch_code(dtype):
    import torch
    return {torch.bfloat16: BF16, torch.float16: F16, torch.float8_e4m3fn: E4M3}[dtype]


def gemm_tn(L, A, B, C, scale=1.0, variant=AUTO, stream=None):
    """Call mi355_gemm_tn on torch device tensors through the C ABI (no torch types cross it)."""
    import torch
    M, K = A.shape
    N = B.shape[0]
    in_dt, out_dt = torch_code(A.dtype), torch_code(C.dtype)
    ws_bytes = L.mi355_gemm_workspace_bytes(M, N, K, in_dt, variant)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=A.device) if ws_bytes else None
    s = stream if stream is not None else torch.cuda.current_stream().cuda_stream
    rc = L.mi355_gemm_tn(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0), B.stride(0),
                         C.stride(0), in_dt, out_dt, scale, variant,
                         ws.data_ptr() if ws is not None else None, ws_bytes, s)
    return rc


def gemm_tn_noalloc(L, A, B, C, scale=1.0, variant=AUTO, stream=None):
    """Call mi355_gemm_tn_noalloc on torch device tensors: no workspace crosses the boundary."""
    import torch
    M, K = A.shape
    N = B.shape[0]
    s = stream if stream is not None else torch.cuda.current_stream().cuda_stream
    return L.mi355_gemm_tn_noalloc(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0), B.stride(0),
                                   C.stride(0), torch_code(A.dtype), torch_code(C.dtype), scale, variant, s)


def gemm_tn_mxfp8(L, A_q, B_q, sa, sb, C, shuffled=False, stream=None):
    """Call mi355_gemm_tn_mxfp8 on torch device tensors.  With shuffled=True the scales are first
    re-laid with mi355_mx_shuffle_scales (as a caller would do once for weights)."""
    import torch
    M, K = A_q.shape
    N = B_q.shape[0]
    s = stream if stream is not None else torch.cuda.current_stream().cuda_stream
    out_dt = torch_code(C.dtype)
    if shuffled:
        pa = torch.empty(max(L.mi355_mx_shuffled_bytes(M, K), 8), dtype=torch.uint8, device=A_q.device)
        pb = torch.empty(max(L.mi355_mx_shuffled_bytes(N, K), 8), dtype=torch.uint8, device=A_q.device)
        rc = L.mi355_mx_shuffle_scales(sa.data_ptr(), M, K, sa.stride(0), pa.data_ptr(), s)
        rc = rc or L.mi355_mx_shuffle_scales(sb.data_ptr(), N, K, sb.stride(0), pb.data_ptr(), s)
        if rc:
            return rc
        ws_bytes = L.mi355_gemm_mx_workspace_bytes(M, N, K, 1)     # partial results of a K split, if any
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=A_q.device)
        return L.mi355_gemm_tn_mxfp8(A_q.data_ptr(), B_q.data_ptr(), C.data_ptr(), M, N, K, A_q.stride(0),
                                     B_q.stride(0), C.stride(0), pa.data_ptr(), 0, pb.data_ptr(), 0, 1, out_dt,
                                     ws.data_ptr(), ws_bytes, s)
    ws_bytes = L.mi355_gemm_mx_workspace_bytes(M, N, K, 0)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=A_q.device)
    return L.mi355_gemm_tn_mxfp8(A_q.data_ptr(), B_q.data_ptr(), C.data_ptr(), M, N, K, A_q.stride(0),
                                 B_q.stride(0), C.stride(0), sa.data_ptr(), sa.stride(0), sb.data_ptr(),
                                 sb.stride(0), 0, out_dt, ws.data_ptr(), ws_bytes, s)


def plan(L, M, N, K, in_dt, variant=AUTO):
    """(variant, tile_rows, tile_cols, k_splits, tail_tiles, tail_splits) from mi355_gemm_plan."""
    v = [ctypes.c_int() for _ in range(5)]
    rc = L.mi355_gemm_plan(M, N, K, in_dt, variant, *[ctypes.byref(x) for x in v])
    return (rc,) + tuple(x.value for x in v)
