"""Builds libmrl_hip.so (gfx950) from csrc/*.hip with hipcc, in-tree.

    python -m mindspeed_rl_amd._build

The library lands in ``mindspeed_rl_amd/lib/libmrl_hip.so`` next to this file so that it
travels with the source tree; nothing is installed into site-packages.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
PROJECT_DIR = os.path.dirname(PKG_DIR)
REPO_ROOT = os.path.dirname(PROJECT_DIR)
CSRC_DIR = os.path.join(PROJECT_DIR, "csrc")
INCLUDE_DIR = os.path.join(REPO_ROOT, "include")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmrl_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU ops are switched off for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument"]


def sources():
    return sorted(os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".hip"))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature and says so; that line is noise
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), out))
    if verbose and out.strip():
        print(out, flush=True)


def build(verbose=False, jobs=None):
    """Compiles every csrc/*.hip for gfx950 and links libmrl_hip.so.  Always recompiles."""
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + ".o") for s in srcs]
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16)

    def compile_one(pair):
        src, obj = pair
        _run([HIPCC, *DEVICE_FLAGS, "-I", INCLUDE_DIR, "-I", CSRC_DIR, "-c", src, "-o", obj], verbose)

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    tmp = LIB_PATH + ".tmp"
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
