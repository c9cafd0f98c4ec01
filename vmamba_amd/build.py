"""Builds the native pieces in-tree with hipcc / g++ (no GPU needed: gfx950 is cross-compiled).

  libss2d_hip.so                  HIP kernels + C ABI (include/ss2d_hip.h)
  selective_scan_cuda_oflex*.so   thin PyTorch C++ extension over the C ABI, importable under the
                                  name the reference probes for (classification/models/csms6s.py:9-14)

Usage:  python -m vmamba_amd.build [--no-torch-ext]
"""
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libss2d_hip.so")
HIP_SOURCES = ["cross_scan.hip", "cross_merge.hip", "selective_scan.hip", "scan_chan.hip", "scan_small.hip", "layer_norm.hip", "dwconv.hip",
               "ss2d_core.hip", "ss2d_core_small.hip", "ss2d_core_tiled.hip", "core_pads.hip", "dt_proj.hip", "cross_flex.hip",
               "selective_scan_bwd.hip", "mlp_fused.hip", "linear_cl.hip", "stem_conv.hip", "mean_pool.hip"]
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_hip(verbose=True, jobs=None):
    """Every .hip source to an object (in parallel), then one shared library."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    flags = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
             # keep the compiler from forming packed-fp32 VALU ops
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wall", "-Wno-unused-function"]
    objdir = os.path.join(CSRC, "_build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.splitext(src)[0] + ".o") for src in HIP_SOURCES]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc] + flags + ["-c", os.path.join(CSRC, src), "-o", obj])

    jobs = jobs or min(len(HIP_SOURCES), max(1, min(os.cpu_count() or 1, 16)))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(HIP_SOURCES, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB])
    return LIB


def torch_ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(PKG, "selective_scan_cuda_oflex" + suffix)


def build_torch_ext():
    import torch
    from torch.utils import cpp_extension

    out = torch_ext_path()
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = cpp_extension.include_paths() + [os.path.join(ROCM, "include"), sysconfig.get_paths()["include"]]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=selective_scan_cuda_oflex", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations"]
    cmd += [f"-I{p}" for p in inc]
    cmd += [os.path.join(CSRC, "torch_ext.cpp"), "-o", out,
            f"-L{tlib}", "-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10_hip", "-ltorch_hip",
            f"-L{PKG}", "-lss2d_hip", f"-L{os.path.join(ROCM, 'lib')}", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}", f"-Wl,-rpath,{os.path.join(ROCM, 'lib')}"]
    _run(cmd)
    return out


def build_all(torch_ext=True):
    build_hip()
    if torch_ext and os.path.exists(os.path.join(CSRC, "torch_ext.cpp")):
        build_torch_ext()


if __name__ == "__main__":
    build_all(torch_ext="--no-torch-ext" not in sys.argv)
