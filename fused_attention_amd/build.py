"""Builds the gfx950 kernel library, the torch-free smoke binary and the torch binding in-tree.

Counterpart of the reference's two build files: setup.py (reference setup.py:7-20, a
CUDAExtension named `fused_attn`) and CMakeLists.txt (reference CMakeLists.txt:49-58, the
standalone `test` executable).  Here the device code is compiled once by hipcc for gfx950 into
a plain shared library with a C ABI, and the torch binding is host-only C++ compiled by g++
that links against it, so no source ever passes through a CUDA-to-HIP translation step.
"""
import os
import subprocess
import sys
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libfused_attn_gfx950.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)
SMOKE_PATH = os.path.join(PKG_DIR, "fa_test")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-Wno-unused-value",
    # the direct-to-LDS loads name M0 as clobbered, which clang reports as a reserved register
    "-Wno-inline-asm",
    # keep the compiler from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX")
    return os.path.join(REPO_DIR, "fused_attn" + suffix)


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "is not a recognized feature for this target" not in line
    )
    if out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError("build step failed (exit %d): %s" % (proc.returncode, " ".join(cmd)))


def build_kernel_library():
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    _run([hipcc] + HIPCC_FLAGS + ["-fPIC", "-shared",
                                  os.path.join(CSRC, "fused_attn_capi.hip"), "-o", LIB_PATH])
    return LIB_PATH


def build_smoke_binary():
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    _run([hipcc] + HIPCC_FLAGS + [os.path.join(CSRC, "test.hip"), "-o", SMOKE_PATH,
                                  "-L" + PKG_DIR, "-lfused_attn_gfx950", "-Wl,-rpath,$ORIGIN"])
    return SMOKE_PATH


def build_torch_binding():
    import torch
    from torch.utils import cpp_extension as ce

    torch_lib = ce.library_paths()[0]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=fused_attn",
           "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in ce.include_paths() + [os.path.join(ROCM, "include"), sysconfig.get_paths()["include"],
                                     os.path.join(REPO_DIR, "include")]:
        cmd += ["-I" + inc]
    cmd += [os.path.join(CSRC, "fused_attn_extention.cpp"), "-o", ext_path(),
            "-L" + PKG_DIR, "-lfused_attn_gfx950",
            "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-ltorch_python",
            "-Wl,-rpath,$ORIGIN/fused_attention_amd", "-Wl,-rpath," + torch_lib,
            "-Wl,--no-as-needed"]
    _run(cmd)
    return ext_path()


def build_all():
    build_kernel_library()
    build_smoke_binary()
    build_torch_binding()


if __name__ == "__main__":
    what = sys.argv[1:] or ["all"]
    for w in what:
        {"all": build_all, "lib": build_kernel_library, "smoke": build_smoke_binary,
         "ext": build_torch_binding}[w]()
