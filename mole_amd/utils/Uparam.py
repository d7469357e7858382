"""Owners of the expert parameters: GPU-resident ("static") and pinned-host ("dynamic", offloaded).

Mirror of MOLE/utils/Uparam.py:145-196 (CPUHostBatchedParameter) and 337-405
(GPUHostBatchedParameter): batched [count, *size] storage, the same initialisation
(kaiming_uniform with a=sqrt(5) for weights, fan_out when `transposed`; U(-1/sqrt(fan_in), ..) for
biases), gradient buffers alongside.  Offloaded parameters live in pinned host memory allocated as
such (torch pin_memory=True), never registered after the fact.  Optimizer state (momentum,
variance) of the reference is allocated lazily because it is not on the forward/backward path.
"""
import math

import torch


def _init_(t: torch.Tensor, count, bias, fan_in, transposed):
    for i in range(count):
        if bias:
            bound = 1 / math.sqrt(fan_in)
            torch.nn.init.uniform_(t[i], -bound, bound)
        else:
            torch.nn.init.kaiming_uniform_(t[i], a=math.sqrt(5), mode="fan_out" if transposed else "fan_in")


class GPUHostBatchedParameter(object):
    def __init__(self, size, count, dtype, device, moe, p_id, bias=False, fan_in=0, transposed=False):
        self.count, self.size, self.dtype, self.device = count, size, dtype, device
        self.bias, self.p_id, self.moe = bias, p_id, moe
        if count > 0:
            init = torch.empty((count, *list(size)), device=device, dtype=torch.float32)
            _init_(init, count, bias, fan_in, transposed)
            self.all_tensors = init.to(dtype).contiguous()
            self.grad_tensors = torch.zeros((count, *list(size)), device=device, dtype=dtype)
            self.all_tensors.grad = self.grad_tensors
            moe.set_GPUParamCore(p_id, self.all_tensors, self.grad_tensors, self.bias)
        else:
            self.all_tensors = 0
        self.lazy_zero_grad = True

    def fetch_single(self, id):
        return self.all_tensors[id]

    def fetch_single_grad(self, id):
        return self.grad_tensors[id]

    def fetch_all_with_grad(self):
        ret = self.all_tensors
        ret.grad = self.grad_tensors
        return ret


class CPUHostBatchedParameter(object):
    def __init__(self, size, count, dtype, moe, p_id, bias=False, fan_in=0, transposed=False, device_s_experts=-1):
        self.count, self.size, self.dtype, self.device = count, size, dtype, "cpu"
        self.p_id, self.bias, self.moe = p_id, bias, moe
        self.adam_state = True
        if count > 0:
            pin = torch.cuda.is_available()
            init = torch.empty((count, *list(size)), dtype=torch.float32)
            _init_(init, count, bias, fan_in, transposed)
            self.all_tensors = torch.empty((count, *list(size)), dtype=dtype, pin_memory=pin)
            self.all_tensors.copy_(init)
            del init
            self.all_tensors.adam_state = self.adam_state
            self.all_tensors.grad_ = torch.zeros((count, *list(size)), dtype=dtype, pin_memory=pin)
            self.all_tensors.grad_.lazy_zero = True
            # Adam moments (Uparam.py:178-181), fp32 whatever the parameter dtype.  Pinned memory is
            # scarce, so they exist only when the core runs the in-pipeline Adam that reads them.
            if getattr(moe, "adv_adam", False):
                self.all_tensors.momentum = torch.zeros((count, *list(size)), dtype=torch.float32, pin_memory=pin)
                self.all_tensors.variance = torch.zeros((count, *list(size)), dtype=torch.float32, pin_memory=pin)
            else:
                self.all_tensors.momentum = None
                self.all_tensors.variance = None
            moe.set_CPUParamCore(p_id, self.all_tensors, self.all_tensors.grad_, self.all_tensors.momentum,
                                 self.all_tensors.variance, self.bias, self.p_id)
        else:
            self.all_tensors = None

    def fetch_single(self, id):
        return self.all_tensors[id]

    def fetch_single_grad(self, id):
        return self.all_tensors.grad_[id]

    def unset_lazy_zero(self):
        if self.count > 0:
            self.all_tensors.grad_.lazy_zero = False
