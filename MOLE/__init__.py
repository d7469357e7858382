"""Import path of the reference package: `MOLE.moe.layer`, `MOLE.utils.*`, `MOLE.core` resolve to the
MI355X implementation in mole_amd (the reference tree imports the same modules as `UniMoE.*`,
MOLE/moe/layer.py:3-13; see the UniMoE package beside this one)."""
from mole_amd import core  # noqa: F401
