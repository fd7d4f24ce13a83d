"""Build the gfx950 shared library ``libtk3d.so`` from ``csrc/*.hip`` with hipcc.

Run as ``python -m torkit3d_amd.build``. hipcc cross-compiles for gfx950 without a
GPU, so the library can be built on a CPU-only host and shipped.
"""
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libtk3d.so")

# -ffp-contract=off: the only fused multiply-adds are the ones the sources spell.
# -packed-fp32-ops is switched off for the device pass (the host pass does not
# know the feature and says so; that warning is harmless).
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the Hilbert curve table of the chamfer sort is worked out at compile time
    "-fconstexpr-steps=200000000",
    "-Wall",
    "-Wno-unused-function",
]


# Matrix instructions that write ordinary vector registers (no copies out of the
# accumulation registers before the vector ALU can use a result). An LLVM option: other
# ROCm releases may not know it, so it is used only where a trial compilation accepts it;
# the kernels are correct either way.
MFMA_VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]


def optional_flags():
    """Those of the optional compiler flags that this hipcc accepts."""
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "probe.hip")
        with open(src, "w") as f:
            f.write("__global__ void probe() {}\n")
        res = subprocess.run([hipcc_path(), "--offload-arch=gfx950", "-c", src, "-o",
                              os.path.join(tmp, "probe.o")] + MFMA_VGPR_FORM,
                             stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return list(MFMA_VGPR_FORM) if res.returncode == 0 else []


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose=False, jobs=None):
    """Compile every kernel source for gfx950 (one hipcc process per source file, run side
    by side) and link ``libtk3d.so`` in-tree."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"] + optional_flags()
    include = ["-I", os.path.join(REPO, "include"), "-I", CSRC]

    def run(cmd):
        if verbose:
            print(" ".join(cmd))
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + out)
        if verbose and out.strip():
            print(out)

    def compile_one(src):
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        run([hipcc_path()] + compile_flags + include + ["-c", src, "-o", obj])
        return obj

    srcs = sources()
    with ThreadPoolExecutor(max_workers=jobs or min(len(srcs), os.cpu_count() or 1, 16)) as pool:
        objects = list(pool.map(compile_one, srcs))
    run([hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH + ".tmp"]
        + objects)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    shutil.rmtree(objdir, ignore_errors=True)  # (objects are rebuilt by every call anyway)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
