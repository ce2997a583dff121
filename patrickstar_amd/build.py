"""Builds libps_adam.so (the C-ABI HIP library) for gfx950 with hipcc, in-tree."""
import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, "libps_adam.so")
SOURCES = [os.path.join(PKG_DIR, "csrc", "ps_adam.hip")]
INCLUDE = os.path.join(ROOT, "include")

# -ffp-contract=off: fused multiply-adds are written out explicitly; the compiler must not add or remove any.
# -fhip-fp32-correctly-rounded-divide-sqrt: IEEE-rounded '/' and sqrtf (hipcc's default, stated on purpose).
# Denormals are kept: -fgpu-flush-denormals-to-zero is not given.
# packed-fp32 ops are switched off: the compiler otherwise pairs independent float ops into v_pk_* forms.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-fast-math",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wall",
    "-Wextra",
    "-Wno-unused-function",
]


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the HIP library cannot be built")


def compile_shared(sources, target, verbose=False, extra_flags=()):
    """hipcc the given sources into one shared library with this package's flags."""
    # compile beside the target and rename: a process that has the old library mapped keeps its own copy
    tmp = target + f".{os.getpid()}.tmp"
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-I", INCLUDE, *sources, "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    try:
        subprocess.check_call(cmd)
        os.replace(tmp, target)
    finally:
        if os.path.exists(tmp):
            os.remove(tmp)
    return target


def build(verbose=False, extra_flags=()):
    """Compile the package's HIP sources into patrickstar_amd/libps_adam.so (returned)."""
    return compile_shared(SOURCES, LIB_PATH, verbose, extra_flags)


if __name__ == "__main__":
    print(build(verbose=True))
