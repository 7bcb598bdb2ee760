"""Builds, in-tree, librecis_hip.so (the C-ABI HIP library for gfx950) and recis.so (the
``TORCH_LIBRARY(recis)`` registration on top of it).

Usage: ``python -m recis_amd.build``. Every ``csrc/*.hip`` file is compiled with hipcc for
gfx950 and linked into ``recis_amd/lib/librecis_hip.so``; every ``csrc/torch/*.cc`` file (host
code only) is compiled with g++ against the installed torch headers and linked into
``recis_amd/lib/recis.so``, which finds librecis_hip.so beside itself. No GPU is needed to build.
"""
import concurrent.futures
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(CSRC, "_obj")
LIB_PATH = os.path.join(LIB_DIR, "librecis_hip.so")
TORCH_CSRC = os.path.join(CSRC, "torch")
TORCH_LIB_PATH = os.path.join(LIB_DIR, "recis.so")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# packed-fp32 instructions are disabled on purpose: some of their forms have
# produced silently wrong results on this hardware generation's toolchain.
COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(HERE, "..", "include"),
]


def sources():
    return sorted(
        os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip")
    )


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + COMMON_FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(
        l for l in (r.stdout + r.stderr).splitlines()
        if "packed-fp32-ops" not in l and "is not a recognized feature" not in l
    )
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
    return obj, out


def build(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    jobs = min(8, max(1, len(srcs)))
    objs = []
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        for obj, out in ex.map(_compile, srcs):
            objs.append(obj)
            if verbose and out.strip():
                print(out)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", LIB_PATH)
    build_torch_library(verbose)
    return LIB_PATH


def _compile_host(args):
    src, flags = args
    obj = os.path.join(OBJ_DIR, "torch_" + os.path.basename(src)[:-3] + ".o")
    r = subprocess.run(["g++"] + flags + ["-c", src, "-o", obj], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("g++ failed on %s:\n%s" % (src, r.stdout + r.stderr))
    return obj


def build_torch_library(verbose=True):
    """recis.so: the torch-facing side (operators and custom classes under the ``recis``
    namespace). Host code only: tensors in, plain pointers out to librecis_hip.so."""
    import torch
    from torch.utils import cpp_extension

    os.makedirs(OBJ_DIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    flags = ["-std=c++17", "-O2", "-fPIC", "-w", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
             "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
             "-I", os.path.join(HERE, "..", "include"), "-I", TORCH_CSRC]
    for inc in cpp_extension.include_paths("cuda"):
        flags += ["-isystem", inc]
    srcs = sorted(os.path.join(TORCH_CSRC, f) for f in os.listdir(TORCH_CSRC) if f.endswith(".cc"))
    with concurrent.futures.ThreadPoolExecutor(min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile_host, [(s, flags) for s in srcs]))
    cmd = ["g++", "-shared", "-fPIC", "-o", TORCH_LIB_PATH] + objs + [
        "-L", LIB_DIR, "-lrecis_hip", "-Wl,-rpath,$ORIGIN", "-L", torch_lib, "-Wl,-rpath," + torch_lib,
        "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
        # the event helpers of ATen's headers are inline and call the HIP runtime directly
        "-L", os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib"), "-lamdhip64",
        "-Wl,--no-undefined", "-Wl,--allow-shlib-undefined"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link of recis.so failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", TORCH_LIB_PATH)
    return TORCH_LIB_PATH


if __name__ == "__main__":
    build()
