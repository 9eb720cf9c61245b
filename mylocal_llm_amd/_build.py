"""Build libqmoe_hip.so from the HIP sources in csrc/ (gfx950 only, in-tree)."""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libqmoe_hip.so")
SOURCES = ("qmoe_linear.hip", "qmoe_stream.hip", "qmoe_span.hip", "qmoe_router.hip", "qmoe_moe.hip", "qmoe_decode.hip", "qmoe_decode2.hip", "qmoe_gemm.hip", "qmoe_front.hip", "qmoe_few.hip", "qmoe_host.hip", "qmoe_probe.hip", "qmoe_status.hip")
# Packed fp32 VALU forms are switched off for all device code.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


TIMELINE_LIB_PATH = os.path.join(_HERE, "libqmoe_hip_timeline.so")


def build_library(verbose=False, timeline=False):
    """Compile every source for gfx950 and link the shared library; always recompiles.
    ``timeline`` builds the measurement variant beside it (libqmoe_hip_timeline.so): the MoE decode
    kernels then write per-wave time stamps of their phases, read back through qmoe_timeline_read."""
    objdir = os.path.join(_HERE, "build_timeline" if timeline else "build")
    os.makedirs(objdir, exist_ok=True)
    hipcc = _hipcc()
    extra = ["-DQMOE_TIMELINE"] if timeline else []
    lib_path = TIMELINE_LIB_PATH if timeline else LIB_PATH

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stderr[-4000:]}")
        if verbose:
            print("compiled", src)
        return obj

    with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        objects = list(pool.map(compile_one, SOURCES))
    tmp = lib_path + ".tmp"
    proc = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objects],
                          capture_output=True, text=True)
    if proc.returncode:
        raise RuntimeError(f"link failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp, lib_path)
    return lib_path


if __name__ == "__main__":
    import sys
    print(build_library(verbose=True, timeline="--timeline" in sys.argv[1:]))
