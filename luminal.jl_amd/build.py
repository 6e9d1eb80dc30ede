"""Build libluminal_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

Usage: python luminal.jl_amd/build.py            # rebuild everything
The library lands in luminal.jl_amd/lib/ and is what the ctypes binding loads.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libluminal_hip.so"
SOURCES = ["api.hip", "prefill_valu.hip", "prefill_mfma.hip", "prefill_f32.hip", "decode.hip", "decode_mfma.hip", "cache_ops.hip", "calib.hip"]

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar fp32 code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# extra -D switches for one-off kernel experiments (never set by the tests, the bench or the driver)
HIPCC_FLAGS += os.environ.get("LMH_EXTRA_FLAGS", "").split()


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the HIP extension cannot be built")


def library_path():
    return os.path.join(LIBDIR, LIBNAME)


def build_library(verbose=True):
    """Compile every .hip source for gfx950 and link the shared library. Always recompiles."""
    hipcc = hipcc_path()
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print("[build]", " ".join(cmd), flush=True)
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs = []
    for src, obj, proc in procs:
        out, _ = proc.communicate()
        # the host pass does not know the gfx-only target feature; that note is expected
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    tmp = library_path() + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    os.replace(tmp, library_path())
    return library_path()


if __name__ == "__main__":
    print(build_library(verbose="-q" not in sys.argv))
