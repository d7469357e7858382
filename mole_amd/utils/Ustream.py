"""Stream roles of the expert pipeline.

Mirror of MOLE/utils/Ustream.py:6-73 and MOLE/cpp/stream.cpp:84-144.  The reference owns 16 streams
and makes stream 2 ("comp") torch's current stream; here compute simply stays on torch's current
stream and the only extra stream is the slot pool's copy stream ("tran"), created at default
priority by mole_unimem_create.  comm / tranback have no work on one GPU and alias the compute
stream.
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
        return cls._instance

    def __init__(self, *args, **kw):
        pass

    @staticmethod
    def tran_stream():
        um = core.get_UniMem()
        if um is None or ExpertStreamCtx._instance.disable:
            return ExpertStreamCtx.comp_stream()
        return torch.cuda.ExternalStream(um.tran_stream_handle(), device=ExpertStreamCtx._instance.device)

    @staticmethod
    def comp_stream():
        return torch.cuda.current_stream(device=ExpertStreamCtx._instance.device)

    comm_stream = comp_stream
    tran_back_stream = comp_stream

    @staticmethod
    def default_stream():
        return ExpertStreamCtx._instance.default
