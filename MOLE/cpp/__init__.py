"""Where the reference keeps its native extension.  The C ABI of the MI355X implementation is declared in
mole_hip.h in this directory (it forwards to include/mole_hip.h), implemented by the HIP sources beside it and built
into libmole_hip.so in this directory by `python -m mole_amd.build`; LIB_PATH names the built library."""
import os

from mole_amd._lib import LIB_PATH  # noqa: F401

HEADER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mole_hip.h")
