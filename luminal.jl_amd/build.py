"""Build libluminal_hip.so (hand-written HIP for gfx950) and libluminal_hip_calib.so (measurement kernels the
benchmark uses) in-tree with hipcc.

Usage: python luminal.jl_amd/build.py            # rebuild everything
The libraries land in luminal.jl_amd/lib/ and are what the ctypes binding loads.

LMH_EXTRA_FLAGS (extra -D switches for kernel experiments) is refused unless LMH_MEASUREMENT_BUILD=1 is set too;
the library is then compiled with -DLMH_MEASUREMENT_BUILD, answers 1 to lmh_measurement_build(), and the binding
refuses to load it unless the same variable is set in the loading process.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libluminal_hip.so"
CALIB_LIBNAME = "libluminal_hip_calib.so"
LIBRARIES = {
    LIBNAME: ["api.hip", "prefill_valu.hip", "prefill_mfma.hip", "prefill_f32.hip", "decode.hip", "decode_mfma.hip", "cache_ops.hip"],
    CALIB_LIBNAME: ["calib.hip"],
}

# Sources that only a measurement build contains: switch in LMH_EXTRA_FLAGS -> (source, flags for that file alone).
# -amdgpu-mfma-vgpr-form: with one wave per SIMD the compiler otherwise keeps every MFMA result in the accumulation
# registers and moves the scores out of them one by one.
MEASUREMENT_SOURCES = {
    "-DLMH_W64_KERNEL": ("prefill_mfma_w64.hip", ["-mllvm", "-amdgpu-mfma-vgpr-form"]),
}

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar fp32 code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def experiment_flags():
    """Extra -D switches for one-off kernel experiments (never set by the tests, the bench or the driver)."""
    extra = os.environ.get("LMH_EXTRA_FLAGS", "").split()
    if not extra:
        return []
    if os.environ.get("LMH_MEASUREMENT_BUILD") != "1":
        raise RuntimeError("LMH_EXTRA_FLAGS=%r is set: experiment switches change what the kernels compute. Unset it, or set "
                           "LMH_MEASUREMENT_BUILD=1 to build a library that is marked as a measurement build." % " ".join(extra))
    print("[build] MEASUREMENT BUILD with %s: not a product library" % " ".join(extra), flush=True)
    return extra + ["-DLMH_MEASUREMENT_BUILD"]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the HIP extension cannot be built")


def library_path(name=LIBNAME):
    return os.path.join(LIBDIR, name)


def build_library(verbose=True):
    """Compile every .hip source for gfx950 and link the shared libraries. Always recompiles."""
    hipcc = hipcc_path()
    flags = HIPCC_FLAGS + experiment_flags()
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    file_flags = {}
    libraries = {name: list(sources) for name, sources in LIBRARIES.items()}
    for switch, (src, src_flags) in MEASUREMENT_SOURCES.items():
        if switch in flags:
            libraries[LIBNAME].append(src)
            file_flags[src] = src_flags
    for libname, sources in libraries.items():
        for src in sources:
            obj = os.path.join(objdir, src.replace(".hip", ".o"))
            cmd = [hipcc] + flags + file_flags.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]
            if verbose:
                print("[build]", " ".join(cmd), flush=True)
            procs.append((libname, src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs = {name: [] for name in libraries}
    for libname, src, obj, proc in procs:
        out, _ = proc.communicate()
        # the host pass does not know the gfx-only target feature; that note is expected
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
        objs[libname].append(obj)
    for libname in libraries:
        tmp = library_path(libname) + ".tmp"
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs[libname]
        if verbose:
            print("[build]", " ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("link of %s failed:\n%s" % (libname, res.stdout))
        os.replace(tmp, library_path(libname))
    return library_path()


if __name__ == "__main__":
    print(build_library(verbose="-q" not in sys.argv))
