"""Stream roles of the expert pipeline.

Mirror of MOLE/utils/Ustream.py:6-73 and MOLE/cpp/stream.cpp:84-144.  The reference owns 16 streams
and makes stream 2 ("comp") torch's current stream; here compute stays on torch's current stream and
the slot pool owns the two copy streams, both created at default priority by mole_unimem_create:
"tran" (host -> pool prefetches and state loads) and "tranback" (gradient / parameter / moment
write-backs).  "comm" has no work on one GPU and is the compute stream.  With multi-stream switched
off (core.disable_multi_stream, stream.cpp:84-95) every role hands out the compute stream.
"""
import torch

from .. import core


class ExpertStreamCtx(object):
    _instance = None

    def __new__(cls, *args, **kw):
        if cls._instance is None:
            cls._instance = object.__new__(cls)
            cls._instance.disable = kw.get("disable", False)
            cls._instance.device = kw.get("device", "cuda:0")
            cls._instance.default = torch.cuda.current_stream(device=cls._instance.device)
            if cls._instance.disable:
                core.disable_multi_stream()
        return cls._instance

    def __init__(self, *args, **kw):
        pass

    @staticmethod
    def _pool_stream(handle_of):
        um = core.get_UniMem()
        inst = ExpertStreamCtx._instance
        if um is None or inst.disable or not core.multi_stream_enabled():
            return ExpertStreamCtx.comp_stream()
        return torch.cuda.ExternalStream(handle_of(um), device=inst.device)

    @staticmethod
    def tran_stream():
        return ExpertStreamCtx._pool_stream(lambda um: um.tran_stream_handle())

    @staticmethod
    def tran_back_stream():
        return ExpertStreamCtx._pool_stream(lambda um: um.tranback_stream_handle())

    @staticmethod
    def comp_stream():
        return torch.cuda.current_stream(device=ExpertStreamCtx._instance.device)

    comm_stream = comp_stream

    @staticmethod
    def default_stream():
        return ExpertStreamCtx._instance.default
