"""`MOLE.utils.Uparam` (MOLE/utils/Uparam.py)."""
from mole_amd.utils.Uparam import *  # noqa: F401,F403
