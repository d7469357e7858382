"""The package name the reference's own modules import (MOLE/moe/layer.py:3-13: `UniMoE.core`,
`UniMoE.utils.Uparam`, `UniMoE.utils.Ugate`, ...): an alias of the MOLE package, so those import lines work
unchanged."""
import sys

import MOLE
import MOLE.core
import MOLE.moe
import MOLE.moe.fast_dispatch
import MOLE.moe.layer
import MOLE.utils
import MOLE.utils.Ugate
import MOLE.utils.Uparam
import MOLE.utils.Uscheduler
import MOLE.utils.Ustream
import MOLE.utils.Utimer

for _name, _mod in list(sys.modules.items()):
    if _name == "MOLE" or _name.startswith("MOLE."):
        sys.modules["UniMoE" + _name[4:]] = _mod
