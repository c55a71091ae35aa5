"""Builds libspark_shim_hip.so (HIP kernels + C ABI, gfx950 only) next to this file with hipcc."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
SO = PKG / "libspark_shim_hip.so"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden",
         # packed FP32 arithmetic is kept off: the compiler must not form v_pk_*_f32 from ordinary float code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


# extra compiler flags for diagnostic builds, e.g. SPARK_HIPCC_EXTRA="-DSPK_EXL3_TRACE -DSPK_MX_TRACE" (per-block time stamps
# of the single-launch kernels, read through spark_debug_exl3_trace / spark_debug_mx_trace)
EXTRA = os.environ.get("SPARK_HIPCC_EXTRA", "").split()


def sources():
    return sorted(CSRC.glob("*.hip")) + sorted(CSRC.glob("*.cpp"))


def build(verbose=False):
    """Compiles every source (always: this is the build check) and links the shared library."""
    objdir = PKG / "build"
    objdir.mkdir(exist_ok=True)

    def cc(src):
        obj = objdir / (src.stem + ".o")
        cmd = [HIPCC, *FLAGS, *EXTRA, "-c", str(src), "-o", str(obj)]
        if src.suffix == ".cpp":
            cmd = [HIPCC, "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-x", "c++", "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"{' '.join(cmd)}\n{r.stderr}")
        if verbose and r.stderr.strip():
            print(r.stderr, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        objs = list(ex.map(cc, sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(SO)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{r.stderr}")
    return SO


if __name__ == "__main__":
    print(build(verbose=True))
