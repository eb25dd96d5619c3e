"""Builds libpypto_amd.so (HIP kernels + C ABI) for gfx950, in-tree, with hipcc.

    python -m pypto_amd.build            # compile the library, then the pybind11 layer on top of it (_host.so)
    python -m pypto_amd.build --host     # the pybind11 layer only
    python -m pypto_amd.build --verbose  # also print register / LDS usage per kernel
    python -m pypto_amd.build --sanitize # host code with AddressSanitizer and UndefinedBehaviorSanitizer, into
                                         # libpypto_amd_san.so: for the boundary's validation paths on a machine
                                         # without a GPU (tests/test_abi_host_sanitized.py runs tests/test_abi_host.py on it)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_PATH = os.path.join(HERE, "libpypto_amd.so")
SOURCES = ["api.cpp", "timing.cpp", "sfa_kernels.hip", "indexer_kernels.hip", "select_experts_kernels.hip", "gqa_kernels.hip", "prolog_kernels.hip", "mla_prolog_kernels.hip", "attention_pre_kernels.hip", "gather_kernels.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-x", "hip",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators in architectural VGPRs: the attention kernel rescales its accumulators with VALU
    # multiplies, and with AGPR accumulators the compiler keeps a VGPR copy of all of them alive
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-I", INCLUDE, "-I", CSRC]
    if verbose:
        cmd += ["-Rpass-analysis=kernel-resource-usage"]
    cmd += [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB_PATH]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err)
    return LIB_PATH


HOST_PATH = os.path.join(HERE, "_host.so")


def build_host():
    """The pybind11 layer (csrc/host_binding.cpp -> pypto_amd/_host.so): host C++ only, compiled with g++ against the
    torch headers and linked to torch's HIP stream / allocator libraries; the C entry points of libpypto_amd.so are handed
    to it by address at load time (pypto_amd/_runtime.py), so it does not link against the library."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce
    torch_lib = ce.library_paths()[0]
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wno-deprecated-declarations",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_host", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for inc in ce.include_paths() + [sysconfig.get_paths()["include"], "/opt/rocm/include", INCLUDE]:
        cmd += ["-isystem" if "torch" in inc or "rocm" in inc else "-I", inc]
    cmd += [os.path.join(CSRC, "host_binding.cpp"), "-o", HOST_PATH,
            "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
            "-ltorch_python", f"-Wl,-rpath,{torch_lib}"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("host binding build failed:\n" + res.stderr)
    return HOST_PATH


SAN_LIB_PATH = os.path.join(HERE, "libpypto_amd_san.so")


def build_sanitized():
    """The library with its host side under ASan + UBSan (the device code is compiled as usual, without optimisation:
    the host objects refer to it, but nothing this build is used for launches a kernel).  The sanitizer runtime is
    linked shared, so a process that loads the library preloads sanitizer_runtime()."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "--offload-arch=gfx950", "-O1", "-g0", "-std=c++17", "-fPIC", "-shared", "-x", "hip",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
           "-fno-sanitize-recover=undefined", "-shared-libsan", "-Wno-unused-command-line-argument",
           "-Wno-unknown-attributes", "-I", INCLUDE, "-I", CSRC]
    cmd += [os.path.join(CSRC, s) for s in SOURCES] + ["-o", SAN_LIB_PATH]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stderr)
    return SAN_LIB_PATH


def sanitizer_runtime():
    clang = os.path.join(os.path.dirname(os.path.realpath(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"))), "..", "llvm", "bin", "clang")
    if not os.path.exists(clang):
        clang = "/opt/rocm/llvm/bin/clang"
    return subprocess.run([clang, "-print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True, text=True, check=True).stdout.strip()


if __name__ == "__main__":
    if "--sanitize" in sys.argv:
        print(build_sanitized())
    elif "--host" in sys.argv:
        print(build_host())
    else:
        print(build(verbose="--verbose" in sys.argv))
        print(build_host())
