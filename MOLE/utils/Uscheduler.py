"""`MOLE.utils.Uscheduler` (MOLE/utils/Uscheduler.py)."""
from mole_amd.utils.Uscheduler import *  # noqa: F401,F403
