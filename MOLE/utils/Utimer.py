"""`MOLE.utils.Utimer` (MOLE/utils/Utimer.py)."""
from mole_amd.utils.Utimer import *  # noqa: F401,F403
from mole_amd.utils.Utimer import UATimer  # noqa: F401
