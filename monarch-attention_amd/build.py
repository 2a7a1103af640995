"""Build libma_hip.so (HIP kernels + C ABI) for gfx950 with hipcc.

    python monarch-attention_amd/build.py          # in-tree: lib/libma_hip.so

hipcc cross-compiles without a GPU.  The library is kept in-tree so that it
travels with the source tree; nothing is installed.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.environ.get("MA_LIB_OUT") or os.path.join(LIB_DIR, "libma_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

# -packed-fp32-ops is switched off for the device code on purpose: the packed
# fp32 VALU forms are not used by these kernels.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # MFMA results straight into VGPRs: the kernels consume every accumulator on the VALU right
         # away (softmax, rounding), so AGPR accumulators only add a v_accvgpr_read per value
         "-mllvm", "-amdgpu-mfma-vgpr-form",
         "-I", os.path.join(ROOT, "include"), "-I", CSRC] + os.environ.get("MA_EXTRA_FLAGS", "").split()


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def depends_on(src: str) -> set:
    """`src` and the headers of this tree it includes, directly or not."""
    seen, todo = set(), [src]
    while todo:
        f = todo.pop()
        if f in seen or not os.path.exists(f):
            continue
        seen.add(f)
        with open(f) as fh:
            for line in fh:
                if line.startswith('#include "'):
                    name = line.split('"')[1]
                    todo += [os.path.join(CSRC, name), os.path.join(ROOT, "include", name)]
    return seen


def build(verbose: bool = False, jobs: int = 8, incremental: bool = False) -> str:
    """Compile every source and link the library.  incremental: keep the objects that are newer than
    their source and every header it includes (a developer's shortcut; the default compiles everything)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(f) for f in depends_on(src)):
            return obj
        cmd = [hipcc, *FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        # the host pass does not know the device-only target feature: drop that warning
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, sources()))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))
