"""vibevoice.c_amd — MI355X (gfx950) backend for vibevoice.c's accelerator seam.

The product is ``lib/libvibevoice_hip.so``: a C-ABI shared library, written in
HIP, that exports the transformer-layer ops and the runtime calls of the
reference's ``include/vibevoice/device.h`` (declared in
``include/vibevoice_hip.h``). This Python package is only a thin ctypes view
of that ABI (``device``) for tests and benchmarks; there is no CPU fallback
anywhere in it, and importing ``device`` fails loudly when the library has not
been built.

The directory name contains a dot, so it cannot be imported by name; load it
with ``load_package()`` from ``__graft_entry__`` (or see that function for the
three-line importlib recipe).
"""
__all__ = ["device", "build"]
