"""randumb_amd: MI355X (gfx950) implementation of RANDUMB's pseudorandom-matrix hot path.

Python surface mirroring the reference package ``rten_cpp`` (Clyde013/randumb) over hand-written HIP kernels
reached through the C ABI of ``librandumb_hip.so``.
"""
from . import _lib, hip  # noqa: F401

__all__ = ["hip"]
