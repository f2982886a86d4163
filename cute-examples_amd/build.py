"""Build the gfx950 kernel library and the gemm_kernels._C extension in-tree.

    python cute-examples_amd/build.py            # both
    python cute-examples_amd/build.py --lib-only  # libmi355gemm.so only (no torch headers needed)

Outputs land in cute-examples_amd/gemm_kernels/: libmi355gemm.so (the C ABI of
include/mi355_gemm.h), _C.<abi>.so (the torch binding, linked against it via $ORIGIN) and
libmi355gemm_syncscales.so, the same library with the block-scaled kernel in its fallback form
(MI355_MX_SYNC_SCALES), which the GPU tests run beside the default one.
Counterpart in the reference: kernels/setup.py:8-28 + build.sh:1-7.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "gemm_kernels")
LIB = os.path.join(OUT, "libmi355gemm.so")
LIB_SYNC_SCALES = os.path.join(OUT, "libmi355gemm_syncscales.so")

HIP_SOURCES = ["gemm_api.hip", "gemm_tn_simple.hip", "gemm_tn_ring_bf16.hip", "gemm_tn_ring_f16.hip", "gemm_tn_ring_e4m3.hip", "gemm_tn_ring_mx.hip", "ring_plan.hip", "gemm_tn_pingpong.hip", "gemm_tn_alternate.hip", "gemm_tn_stream.hip", "quantize_e4m3.hip", "mx_scales.hip", "calibrate.hip"]

# Sources whose device assembly is verified after compilation (check_async_loads.py): the copies'
# LDS base in all of them, the asynchronous scale loads in the block-scaled one.
CHECKED_SOURCES = ["gemm_tn_ring_bf16.hip", "gemm_tn_ring_f16.hip", "gemm_tn_ring_e4m3.hip", "gemm_tn_ring_mx.hip"]
CHECKED_SOURCE = "gemm_tn_ring_mx.hip"
# Sources whose kernels must keep the hardware's distances the compiler does not enforce (wide
# stores and their data registers, inline-assembly MFMAs and their results): every GEMM kernel.
HAZARD_SOURCES = CHECKED_SOURCES + ["gemm_tn_pingpong.hip", "gemm_tn_alternate.hip", "gemm_tn_stream.hip", "calibrate.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 target feature and says so once per file.
    for line in proc.stdout.splitlines():
        if "packed-fp32-ops" not in line:
            print(line)
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (proc.returncode, " ".join(cmd)))


def build_lib():
    """Compile every source to an object (in parallel), check the generated assembly of the
    block-scaled kernel (check_async_loads.py), link."""
    import glob
    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    sys.path.insert(0, HERE)
    import check_async_loads

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    with tempfile.TemporaryDirectory() as tmp:
        def compile_one(src, defines=(), subdir=""):
            os.makedirs(os.path.join(tmp, subdir), exist_ok=True)
            obj = os.path.join(tmp, subdir, src.replace(".hip", ".o"))
            extra = ["-save-temps=obj"] if src in HAZARD_SOURCES else []
            _run([hipcc] + HIPCC_FLAGS + ["-c"] + extra + list(defines) + ["-o", obj, os.path.join(CSRC, src)])
            return obj

        # The block-scaled kernel's asynchronous scale loads are sound only if the compiler never copies
        # their destination registers (check_async_loads.check).  If a toolchain does, or when
        # MI355_MX_SYNC_SCALES=1 asks for it, that one source is built with loads that wait for
        # themselves instead: slower, no assumption.
        sync_scales = ["-DMI355_MX_SYNC_SCALES"] if os.environ.get("MI355_MX_SYNC_SCALES") == "1" else []

        with ThreadPoolExecutor(max_workers=min(len(HIP_SOURCES) + 1, os.cpu_count() or 1)) as pool:
            # the fallback form of the block-scaled kernel, for the second library, beside everything else
            fallback = pool.submit(compile_one, CHECKED_SOURCE, ["-DMI355_MX_SYNC_SCALES"], "sync_scales")
            objs = list(pool.map(lambda src: compile_one(src, sync_scales if src == CHECKED_SOURCE else ()), HIP_SOURCES))
            fallback_obj = fallback.result()
        copies = 0
        for src in CHECKED_SOURCES:
            asm = glob.glob(os.path.join(tmp, src.replace(".hip", "") + "-hip-amdgcn-*gfx950.s"))
            if len(asm) != 1:
                raise RuntimeError("expected one device assembly file for %s, found %r" % (src, asm))
            if src == CHECKED_SOURCE and not sync_scales:
                try:
                    print("check_async_loads: %d scale operands ok" % check_async_loads.check(asm[0]), flush=True)
                except RuntimeError as e:
                    print("check_async_loads: %s\n  -> rebuilding %s with scale loads that wait for themselves "
                          "(MI355_MX_SYNC_SCALES)" % (e, src), flush=True)
                    sync_scales = ["-DMI355_MX_SYNC_SCALES"]
                    compile_one(src, sync_scales)    # same object and assembly file names: both are replaced
            elif src == CHECKED_SOURCE:
                print("check_async_loads: scale loads wait for themselves (MI355_MX_SYNC_SCALES); register check skipped", flush=True)
            copies += check_async_loads.check_lds_base(asm[0])
        print("check_async_loads: %d direct-to-LDS copies ok" % copies, flush=True)
        stores = mfmas = 0
        for src in HAZARD_SOURCES:
            asm = glob.glob(os.path.join(tmp, src.replace(".hip", "") + "-hip-amdgcn-*gfx950.s"))
            if len(asm) != 1:
                raise RuntimeError("expected one device assembly file for %s, found %r" % (src, asm))
            n_st, n_mf = check_async_loads.check_hazard_distances(asm[0])
            stores, mfmas = stores + n_st, mfmas + n_mf
            check_async_loads.check_no_scratch(asm[0])
        print("check_async_loads: %d stores keep their data registers for %d wait states, %d inline MFMAs keep their "
              "results untouched for %d" % (stores, check_async_loads.STORE_DATA_WINDOW, mfmas,
                                             check_async_loads.MFMA_RESULT_WINDOW), flush=True)
        _run([hipcc] + HIPCC_FLAGS + ["-o", LIB] + objs)
        # The same library around the fallback form of the block-scaled kernel, held to the same distances.
        asm = glob.glob(os.path.join(tmp, "sync_scales", CHECKED_SOURCE.replace(".hip", "") + "-hip-amdgcn-*gfx950.s"))
        if len(asm) != 1:
            raise RuntimeError("expected one device assembly file for the fallback build, found %r" % (asm,))
        check_async_loads.check_lds_base(asm[0])
        check_async_loads.check_hazard_distances(asm[0])
        check_async_loads.check_no_scratch(asm[0])
        main_obj = os.path.join(tmp, CHECKED_SOURCE.replace(".hip", ".o"))
        _run([hipcc] + HIPCC_FLAGS + ["-o", LIB_SYNC_SCALES] + [fallback_obj if o == main_obj else o for o in objs])
    return LIB


def ext_path():
    return os.path.join(OUT, "_C" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_ext():
    import pybind11
    import torch
    from torch.utils import cpp_extension as ce

    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
           "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-Wno-deprecated-declarations"]
    for inc in ce.include_paths("cuda") + [sysconfig.get_paths()["include"], pybind11.get_include()]:
        cmd += ["-isystem", inc]
    cmd += ["-o", ext_path(), os.path.join(CSRC, "torch_binding.cpp"),
            "-L" + OUT, "-l:libmi355gemm.so", "-L" + tlib, "-L/opt/rocm/lib",
            "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python", "-lc10", "-lc10_hip", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib, "-Wl,-rpath,/opt/rocm/lib"]
    _run(cmd)
    return ext_path()


def main(argv):
    build_lib()
    if "--lib-only" not in argv:
        build_ext()


if __name__ == "__main__":
    main(sys.argv[1:])
