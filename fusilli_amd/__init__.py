"""MI355X (gfx950) execution backend behind Fusilli's graph API.

``fusilli_amd.capi`` binds the C ABI of ``include/fusilli_hip.h`` (hand-written
HIP kernels in ``fusilli_amd/csrc``); the C++ graph front end lives in
``include/fusilli.h``.  There is no CPU execution path in this package.
"""
from . import capi, synth  # noqa: F401

__all__ = ["capi", "synth"]
