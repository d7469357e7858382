"""The tutel.impls.fast_dispatch interface the layer calls (MOLE/moe/layer.py:4, 445-458)."""
from mole_amd.moe.fast_dispatch import extract_critical, fast_decode, fast_encode  # noqa: F401
