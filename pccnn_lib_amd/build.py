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


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv)
    print("built", LIB_PATH)
    sys.exit(0)
