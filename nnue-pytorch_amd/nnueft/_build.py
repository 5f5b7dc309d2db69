"""Compiles csrc/*.hip into libnnueft.so next to this file (hipcc, gfx950 only)."""
import glob
import os
import shutil
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
CSRC = os.path.join(_ROOT, "csrc")
INCLUDE = os.path.join(os.path.dirname(_ROOT), "include")
LIB_PATH = os.path.join(_PKG, "libnnueft.so")

# -ffp-contract=off: the fp32 paths promise a rounding after every multiply and add.
# packed-fp32 ops are switched off: some of their forms have produced wrong values on this hardware.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fPIC",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: libnnueft.so cannot be built")


def build(verbose: bool = False, extra_flags=(), lib_path: str = LIB_PATH) -> str:
    """Compile every kernel source and link the C-ABI library.  Always recompiles.

    extra_flags / lib_path build a variant (e.g. -DNNUEFT_SEG_U=16) next to the default library."""
    hipcc = hipcc_path()
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError(f"no kernel sources under {CSRC}")
    objs = []
    procs = []
    objdir = os.path.join(CSRC, "build", os.path.basename(lib_path).replace(".so", ""))
    os.makedirs(objdir, exist_ok=True)
    for src in srcs:
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-I", INCLUDE, "-I", CSRC, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out, flush=True)
    tmp = lib_path + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}")
    os.replace(tmp, lib_path)
    return lib_path


if __name__ == "__main__":
    print(build(verbose=True))
