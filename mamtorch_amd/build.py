"""In-tree build of the native code: libmam_hip.so (HIP kernels + C ABI, gfx950) and
mam_torch_ops.so (torch.ops registration that calls the C ABI).

Run ``python -m mamtorch_amd.build``.  hipcc cross-compiles for gfx950 without a GPU.  The
libraries are written to ``mamtorch_amd/lib/``.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")
HIP_LIB = os.path.join(LIB_DIR, "libmam_hip.so")
OPS_LIB = os.path.join(LIB_DIR, "mam_torch_ops.so")

HIP_SOURCES = ["mam_common.hip", "mam_forward.hip", "mam_backward.hip", "mam_selcount.hip", "mam_csr.hip",
               "mam_spmm.hip", "mam_prune.hip", "mam_select.hip", "mam_module.hip"]

# -ffp-contract=off: a product that feeds an add must stay an fp32 multiply followed by an fp32
# add (bit-exact forward).  Packed-FP32 instructions are disabled for the device pass.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall",
             "-Wno-unused-command-line-argument"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        # MAM_HIPFLAGS: extra compiler flags, e.g. -D switches of tuning constants
        out = _run([hipcc] + HIP_FLAGS + os.environ.get("MAM_HIPFLAGS", "").split()
                   + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(compile_one, HIP_SOURCES))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB] + objs)
    return HIP_LIB


def build_torch_ops(verbose=False):
    import torch
    from torch.utils import cpp_extension

    os.makedirs(LIB_DIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for p in cpp_extension.include_paths("cuda"):
        inc += ["-isystem", p]
    cmd = (["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unknown-pragmas",
            "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
            "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
           + inc + [os.path.join(CSRC, "torch_binding.cpp"), "-o", OPS_LIB,
                    "-L" + LIB_DIR, "-lmam_hip", "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-lc10",
                    "-ltorch_hip", "-lc10_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib,
                    "-Wl,--no-as-needed"])
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return OPS_LIB


def build_all(verbose=False):
    return build_hip(verbose), build_torch_ops(verbose)


if __name__ == "__main__":
    for path in build_all(verbose=True):
        print("built", path)
    sys.exit(0)
