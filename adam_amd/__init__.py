"""adam_amd: MI355X (gfx950) backend for ADAM's quantized decode path.

`adam_amd.adamah` is the drop-in for the reference `adamah` Python package (same op surface,
backed by libadamah_hip.so); `adam_amd.engine` is the decode harness that issues the reference
model engine's op sequence through it.
"""
from .adamah import *  # noqa: F401,F403
from .adamah import Adamah, init, DecodePlanOp, __version__  # noqa: F401
