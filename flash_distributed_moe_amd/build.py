"""Builds libflashMoe.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m flash_distributed_moe_amd.build
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libflashMoe.so")

# -packed-fp32-ops: keep the compiler from forming packed float32 instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-DNDEBUG",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-return-type-c-linkage",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    for src in sources():
        obj = os.path.join(LIB_DIR, os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = [hipcc] + HIPCC_FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stderr=subprocess.PIPE, text=True)))
    for cmd, p in procs:
        _, err = p.communicate()
        err = "\n".join(l for l in err.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            sys.stderr.write(err + "\n")
            raise RuntimeError("hipcc failed: " + " ".join(cmd))
        if verbose and err.strip():
            sys.stderr.write(err + "\n")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs + [
        "-Wl,--version-script=" + os.path.join(CSRC, "lib.version"), "-Wl,-soname,libflashMoe.so"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    return LIB_PATH


PY_SRC = os.path.join(CSRC, "py", "flashMoeLauncherModule.cpp")
ROOT = os.path.dirname(HERE)


def py_extension_path():
    import sysconfig

    return os.path.join(ROOT, "flashMoeLauncher" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_py_extension(verbose=True):
    """The `flashMoeLauncher` Python extension (pybind11 over the C++ interface), next to the
    package so that `import flashMoeLauncher` finds it with the repository root on sys.path.
    Host code only: compiled with g++ against torch's headers."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    out = py_extension_path()
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + sysconfig.get_paths()["include"]]
    cmd += ["-I" + p for p in cpp_extension.include_paths()] + ["-I/opt/rocm/include"]
    cmd += [PY_SRC, "-o", out, "-L" + tlib, "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip",
            "-lc10_hip", "-ltorch_python", "-L" + LIB_DIR, "-lflashMoe", "-L/opt/rocm/lib",
            "-lamdhip64", "-Wl,-rpath,$ORIGIN/flash_distributed_moe_amd/lib", "-Wl,-rpath," + tlib]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    print(build())
    print(build_py_extension())
