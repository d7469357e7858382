"""`MOLE.utils.Ugate` (MOLE/utils/Ugate.py)."""
from mole_amd.utils.Ugate import *  # noqa: F401,F403
