"""Builds the two native artefacts of the package, in-tree, for gfx950 only.

1. ``sarathi_amd/lib/libsarathi_ops_hip.so`` -- the HIP kernels behind the C ABI
   declared in ``include/sarathi_ops.h`` (hipcc, ``--offload-arch=gfx950``; no
   torch dependency).
2. ``sarathi_amd/_C.so`` -- the pybind11 / PyTorch-ROCm front end
   (``csrc/torch_binding.cpp``), which links against (1).

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is
installed.  Run as ``python build.py`` or call :func:`build`.
"""
import concurrent.futures
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
PKG = os.path.join(HERE, "sarathi_amd")
LIB_DIR = os.path.join(PKG, "lib")
OBJ_DIR = os.path.join(HERE, "build", "obj")

HIP_SOURCES = ["rms_norm.hip", "gated_act.hip", "rope.hip", "moe_topk.hip", "moe_align.hip",
               "moe_gemm.hip", "moe_gemm_wide.hip", "moe_sum.hip", "kv_cache.hip",
               "moe_fused_routing.hip", "stream_copy.hip", "moe_balance.hip", "moe_gemm_f32.hip",
               "moe_gemm_rider.hip"]
CXX_SOURCES = ["abi_misc.cpp"]

ABI_LIB = os.path.join(LIB_DIR, "libsarathi_ops_hip.so")
EXT_LIB = os.path.join(PKG, "_C.so")

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# -ffp-contract=off: the kernels round exactly where they say they do; the one
#   fused multiply-add that is wanted (sum of squares) is written as fmaf.
# packed-fp32-ops off: keeps hipcc from forming v_pk_*_f32 instructions.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall", "-Wno-unused-command-line-argument",
]
# extra hipcc flags for tuning builds, e.g. -DSARATHI_KV_STORE_POLICY=18
HIP_FLAGS += os.environ.get("SARATHI_HIPCC_EXTRA_FLAGS", "").split()


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build step failed:\n  %s\n%s" % (" ".join(cmd), out))
    if verbose and out.strip():
        print(out, flush=True)


def build_abi_library(verbose=False, jobs=8):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    cmds, objs = [], []
    for src in HIP_SOURCES + CXX_SOURCES:
        obj = os.path.join(OBJ_DIR, src + ".o")
        objs.append(obj)
        cmds.append([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", ABI_LIB] + objs, verbose)
    return ABI_LIB


def build_torch_extension(verbose=False):
    import torch  # noqa: F401  (headers and libraries come from the installed wheel)
    from torch.utils import cpp_extension

    inc = ["-I" + p for p in cpp_extension.include_paths()]
    inc += ["-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(ROCM, "include")]
    torch_lib = cpp_extension.library_paths()[0]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
        "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H",
        "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi, "-DUSE_ROCM=1", "-D__HIP_PLATFORM_AMD__=1",
        "-Wno-deprecated-declarations",
    ] + inc + [
        os.path.join(CSRC, "torch_binding.cpp"), "-o", EXT_LIB,
        "-L" + LIB_DIR, "-lsarathi_ops_hip", "-Wl,-rpath,$ORIGIN/lib",
        "-L" + torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-ltorch_python",
    ]
    _run(cmd, verbose)
    return EXT_LIB


def build(verbose=False):
    """Compile everything, unconditionally.  Returns the two library paths."""
    return build_abi_library(verbose), build_torch_extension(verbose)


if __name__ == "__main__":
    paths = build(verbose="-q" not in sys.argv)
    print("built:", *paths, sep="\n  ")
