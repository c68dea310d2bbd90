"""Builds ``libpccnn_hip.so`` (every HIP source under csrc/) for gfx950 with hipcc.

    python -m pccnn_lib_amd.build

hipcc cross-compiles without a GPU, so the library is built in-tree ahead of any GPU run.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libpccnn_hip.so")

HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17",
    # packed-fp32 VALU forms are switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-ignored-optimization-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _up_to_date(obj, src):
    """True if the object file is newer than its source and every header beside it."""
    if not os.path.exists(obj):
        return False
    deps = [src] + glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    return os.path.getmtime(obj) > max(os.path.getmtime(d) for d in deps)


def build(verbose=True, jobs=8, incremental=False):
    """Compiles every source (``incremental``: only those changed since their object file was written) and links."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.basename(src) + ".o") for src in sources()]
    srcs = [src for src, obj in zip(sources(), objs) if not (incremental and _up_to_date(obj, src))]
    for i in range(0, len(srcs), jobs):
        batch = []
        for src in srcs[i:i + jobs]:
            obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
            cmd = [hipcc] + HIPCC_FLAGS + ["-c", src, "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            batch.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        for src, p in batch:
            out, _ = p.communicate()
            out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
            if p.returncode != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
            if verbose and out.strip():
                print(out)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


EXT_SOURCE = os.path.join(CSRC, "ops_module.cpp")


def extension_path():
    """Where the compiled ``pccnn_lib_ops`` module goes: the repository root, beside the package, so that
    ``import pccnn_lib_ops`` finds it (an extension module takes precedence over the .py of the same name there)."""
    import sysconfig
    return os.path.join(os.path.dirname(HERE), "pccnn_lib_ops" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_extension(verbose=True):
    """Compiles csrc/ops_module.cpp - the ``pccnn_lib_ops`` PyTorch extension (pybind11, host code only) - against
    this interpreter's torch and links it to libpccnn_hip.so (found at run time relative to the module)."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    cxx = os.environ.get("CXX", "g++")
    out = extension_path()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wno-attributes",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=pccnn_lib_ops",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in cpp_extension.include_paths("cuda") + [sysconfig.get_paths()["include"],
                                                       os.path.join(os.path.dirname(HERE), "include")]:
        cmd += ["-isystem" if "torch" in inc or "rocm" in inc else "-I", inc]
    cmd += [EXT_SOURCE, "-o", out, "-L" + torch_lib, "-L" + HERE, "-l:libpccnn_hip.so", "-ltorch", "-ltorch_cpu",
            "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip", "-Wl,-rpath,$ORIGIN/pccnn_lib_amd",
            "-Wl,-rpath," + torch_lib]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("compiling the pccnn_lib_ops extension failed:\n%s" % res.stdout)
    if verbose and res.stdout.strip():
        print(res.stdout)
    return out


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv)
    if "--no-extension" not in sys.argv:
        print("built", build_extension())
    print("built", LIB_PATH)
    sys.exit(0)
