"""Owners of the expert parameters: GPU-resident ("static") and pinned-host ("dynamic", offloaded).

Mirror of MOLE/utils/Uparam.py:8-107 (UnifiedCPUTensor), 145-196 (CPUHostBatchedParameter) and 337-405
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


class UnifiedCPUTensor(object):
    """One pinned host pool per process for the offloaded experts of all layers (Uparam.py:8-107): four flat
    pinned arrays - parameters, gradients, momentum, variance - of `device_s_experts` experts each, cut by
    parameter kind into [device_s_experts, *size] regions from which every layer takes its `count` experts in
    construction order.  One allocation per array instead of one per layer and kind: pinning is slow and
    the pinned total is what the host limits.  Momentum and variance are fp32 and are allocated only when asked
    for (with_adam_state), since pinned memory is scarce; the reference keeps all four in the parameter dtype."""
    _instance = None
    _optimizer = None

    def __new__(cls, *args, **kw):
        if cls._instance is None:
            inst = object.__new__(cls)
            inst.tensors, inst.grad, inst.momentum, inst.variance = {}, {}, {}, {}
            inst.counter, inst.counter_grad, inst.counter_momentum, inst.counter_variance = {}, {}, {}, {}
            inst.inited = False
            inst.numel = 0
            cls._instance = inst
        return cls._instance

    def __init__(self, *args, **kw):
        pass

    @staticmethod
    def reset():
        UnifiedCPUTensor._instance = None

    @staticmethod
    def init(sizes, device_s_experts, dtype, with_adam_state=False):
        """sizes: the per-expert shapes of the parameter kinds, [[F, M], [F], [F, M], [M]]."""
        inst = UnifiedCPUTensor()
        if inst.inited:
            return
        inst.inited = True
        if device_s_experts <= 0:
            return
        per_expert = sum(math.prod(sz) for sz in sizes)
        inst.numel = device_s_experts * per_expert
        pin = torch.cuda.is_available()
        inst.pool_t = torch.zeros(inst.numel, dtype=dtype, pin_memory=pin)
        inst.pool_g = torch.zeros(inst.numel, dtype=dtype, pin_memory=pin)
        inst.pool_m = torch.zeros(inst.numel, dtype=torch.float32, pin_memory=pin) if with_adam_state else None
        inst.pool_v = torch.zeros(inst.numel, dtype=torch.float32, pin_memory=pin) if with_adam_state else None
        inst.pool_t.grad_, inst.pool_t.momentum, inst.pool_t.variance = inst.pool_g, inst.pool_m, inst.pool_v
        inst.pool_t_d = inst.pool_g_d = inst.pool_m_d = inst.pool_v_d = 0

    @staticmethod
    def _region(pool, start, shape):
        return None if pool is None else pool[start:start + math.prod(shape)].view(shape)

    @staticmethod
    def get_tensor(size, device_s_experts, count, dtype, p_id):
        inst = UnifiedCPUTensor._instance
        if inst is None or not inst.inited or inst.numel == 0:
            raise RuntimeError("UnifiedCPUTensor.init(sizes, device_s_experts, dtype) must run before the layers are built")
        if p_id not in inst.tensors:
            shape = (device_s_experts, *list(size))
            x = math.prod(shape)
            if inst.pool_t_d + x > inst.numel:
                raise RuntimeError("UnifiedCPUTensor: the pool is too small for this parameter kind")
            inst.tensors[p_id] = UnifiedCPUTensor._region(inst.pool_t, inst.pool_t_d, shape)
            inst.grad[p_id] = UnifiedCPUTensor._region(inst.pool_g, inst.pool_g_d, shape)
            inst.momentum[p_id] = UnifiedCPUTensor._region(inst.pool_m, inst.pool_m_d, shape)
            inst.variance[p_id] = UnifiedCPUTensor._region(inst.pool_v, inst.pool_v_d, shape)
            inst.pool_t_d += x
            inst.pool_g_d += x
            inst.pool_m_d += x
            inst.pool_v_d += x
            inst.counter[p_id] = inst.counter_grad[p_id] = inst.counter_momentum[p_id] = inst.counter_variance[p_id] = 0
        c = inst.counter[p_id]
        if c + count > inst.tensors[p_id].shape[0]:
            raise RuntimeError(f"UnifiedCPUTensor: {c + count} experts of kind {p_id} asked for, the pool holds "
                               f"{inst.tensors[p_id].shape[0]}")
        inst.counter[p_id] += count
        return inst.tensors[p_id][c:c + count]

    @staticmethod
    def _take(store, counters, count, p_id):
        inst = UnifiedCPUTensor._instance
        c = counters[p_id]
        counters[p_id] += count
        return None if store[p_id] is None else store[p_id][c:c + count]

    @staticmethod
    def get_grad(size, device_s_experts, count, dtype, p_id):
        inst = UnifiedCPUTensor._instance
        return UnifiedCPUTensor._take(inst.grad, inst.counter_grad, count, p_id)

    @staticmethod
    def get_momentum(size, device_s_experts, count, dtype, p_id):
        inst = UnifiedCPUTensor._instance
        return UnifiedCPUTensor._take(inst.momentum, inst.counter_momentum, count, p_id)

    @staticmethod
    def get_variance(size, device_s_experts, count, dtype, p_id):
        inst = UnifiedCPUTensor._instance
        return UnifiedCPUTensor._take(inst.variance, inst.counter_variance, count, p_id)

    @staticmethod
    def get_cpu_experts():
        inst = UnifiedCPUTensor._instance
        return [inst.pool_t] if inst is not None and inst.numel > 0 else []


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
    """device_s_experts == -1: pinned arrays of this layer's own (Uparam.py:153-181); otherwise views into the
    process-wide UnifiedCPUTensor pool, which holds device_s_experts experts over all layers."""

    def __init__(self, size, count, dtype, moe, p_id, bias=False, fan_in=0, transposed=False, device_s_experts=-1):
        self.count, self.size, self.dtype, self.device = count, size, dtype, "cpu"
        self.p_id, self.bias, self.moe = p_id, bias, moe
        self.adam_state = True
        if count > 0:
            pin = torch.cuda.is_available()
            shape = (count, *list(size))
            want_state = getattr(moe, "adv_adam", False)
            if device_s_experts == -1:
                self.all_tensors = torch.empty(shape, dtype=dtype, pin_memory=pin)
                grad = torch.zeros(shape, dtype=dtype, pin_memory=pin)
                # Adam moments (Uparam.py:178-181), fp32 whatever the parameter dtype.  Pinned memory is
                # scarce, so they exist only when the core runs the in-pipeline Adam that reads them.
                mom = torch.zeros(shape, dtype=torch.float32, pin_memory=pin) if want_state else None
                var = torch.zeros(shape, dtype=torch.float32, pin_memory=pin) if want_state else None
            else:
                args = (size, device_s_experts, count, dtype, p_id)
                self.all_tensors = UnifiedCPUTensor.get_tensor(*args)
                grad = UnifiedCPUTensor.get_grad(*args)
                mom = UnifiedCPUTensor.get_momentum(*args)
                var = UnifiedCPUTensor.get_variance(*args)
                if want_state and (mom is None or var is None):
                    raise RuntimeError("UnifiedCPUTensor.init(..., with_adam_state=True) is needed for the in-pipeline Adam")
            init = torch.empty(shape, dtype=torch.float32)
            _init_(init, count, bias, fan_in, transposed)
            self.all_tensors.copy_(init)
            del init
            self.all_tensors.adam_state = self.adam_state
            self.all_tensors.grad_ = grad
            self.all_tensors.grad_.lazy_zero = True
            self.all_tensors.momentum, self.all_tensors.variance = mom, var
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
