"""luminal.jl_amd — MI355X (gfx950) backend for the attention hot path of Luminal.jl.

csrc/      hand-written HIP kernels + the C ABI (include/luminal_hip.h) -> lib/libluminal_hip.so
binding.py ctypes binding of that ABI
host.py    mirror of the reference's Graph / flash_attention / execute / compile / device API
build.py   hipcc build of the shared library
synth.py   the seeded input generator of the benchmark configurations

The directory name contains a dot, so it is imported through importlib (see
__graft_entry__.load_package) under the module name `luminal_jl_amd`.
"""
from . import binding, host, synth  # noqa: F401
from .host import *  # noqa: F401,F403
