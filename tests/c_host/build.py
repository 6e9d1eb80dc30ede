"""Builds tests/c_host/abi_client: the plain-C consumer of libluminal_hip.so (gcc, C99, the public header only)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
BINARY = os.path.join(HERE, "abi_client")


def command(out=BINARY):
    libdir = os.path.join(ROOT, "luminal.jl_amd", "lib")
    # the library is found next to the repository at run time ($ORIGIN), its own HIP dependency through the system's
    # loader configuration; -rpath-link only tells the link step where that dependency lives
    return ["gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
            os.path.join(HERE, "abi_client.c"), "-o", out, "-L", libdir, "-lluminal_hip", "-lm",
            "-Wl,-rpath,$ORIGIN/../../luminal.jl_amd/lib", "-Wl,-rpath-link,/opt/rocm/lib"]


def build(out=BINARY, verbose=False):
    cmd = command(out)
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("gcc failed on abi_client.c:\n" + res.stdout)
    return out


if __name__ == "__main__":
    print(build(verbose=True))
