"""`MOLE.core` - the module the reference builds with pybind (MOLE/cpp/core.cpp:1347-1469)."""
from mole_amd.core import *  # noqa: F401,F403
from mole_amd.core import (BatchFusedFWD, MOLECore, UniMem, clear_virtual_mem, create_UniMem, default_wait_comm,  # noqa: F401
                           default_wait_comp, default_wait_tran, destroy_UniMem, disable_multi_stream, fast_assign_prefetch,
                           fetch_top_prefetched_batch, get_stream_cdata, get_UniMem, pool_prefetch, synchronize_tran,
                           view_pool_size)
