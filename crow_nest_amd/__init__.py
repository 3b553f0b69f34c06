"""MI355X-native NVFP4 weight x activation path behind the reference engine's kernel-call API.

The product is ``libcrow_hip.so`` (gfx950 HIP kernels + a C ABI, ``include/crow_hip.h``); this
package is its host-side mirror of the reference's Rust interface for the path
(``Kernels::f`` / ``launch_v``, ``load_fp4``, ``dense_proj`` ...).  PyTorch only provides device
memory.  There is no CPU fallback: without the built library, or without a gfx950 device, every
entry point raises.
"""
from .lib import CrowHipError, build, library_path  # noqa: F401
