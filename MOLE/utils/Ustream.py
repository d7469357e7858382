"""`MOLE.utils.Ustream` (MOLE/utils/Ustream.py)."""
from mole_amd.utils.Ustream import *  # noqa: F401,F403
