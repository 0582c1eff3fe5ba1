"""CPU oracle for the ADAMAH quantized-decode op surface.

TEST INFRASTRUCTURE ONLY.  This package restates, in NumPy, the arithmetic of the
reference backend (adamah-MAIN/adamah/adamah.c + shaders/src/**/*.comp) and of the
reference's own NumPy forward pass (tests/diagnostics/diag_inference.py).  It exists so
that the HIP library can be checked against it; nothing in the shipped package
(`adam_amd/`) imports it.  Only tests, the smoke entry and the CPU-baseline leg of the
benchmark may load it, and only as the checker or the timed baseline.
"""
from .adamah_np import NumpyAdamah, init  # noqa: F401
from . import blocks  # noqa: F401
