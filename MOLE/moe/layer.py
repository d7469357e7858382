"""`MOLE.moe.layer` (MOLE/moe/layer.py): MOLEModule and the autograd nodes its forward names."""
from mole_amd.moe.layer import BatchFusedFWD, MOLEModule, pfetchbwd  # noqa: F401
