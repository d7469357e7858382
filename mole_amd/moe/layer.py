"""The MoE layer module - drop-in for MOLE/moe/layer.py (class MOLEModule, lines 18-501).

Constructor and forward keep the reference's names, argument order and defaults
(layer.py:29, layer.py:429).  forward is gate -> route -> dispatch -> expert FFN -> combine
(layer.py:440-462), followed by the prefetch trigger for the next layer (layer.py:464-472).

Two execution shapes, same results:
  * fused (default): one autograd node over the ragged, expert-contiguous layout.  Nothing is
    padded, nothing is read back to the host, every step is a kernel of libmole_hip.so.
  * reference_layout=True: the reference's literal call sequence - extract_critical, fast_encode
    into a zero-padded [E, C, M], BatchFusedFWD.apply over all E*C rows, fast_decode.

New, optional keyword arguments (all defaulting to the reference's behaviour): dtype,
normalize_gate, gelu_bwd ("tanh" = the derivative the reference compiles, MOLE/cpp/define.hpp:6;
"exact" = erf derivative), gate_logit_bias, reference_layout, activated_only (offloaded experts that
received no token are neither copied to the pool nor launched; False restores the reference's
every-expert-in-index-order behaviour), resident (experts that a forward pass brought into the pool are
not fetched again for its backward pass while they are still there; with a pool large enough for all
offloaded experts of all layers every expert keeps a slot of its own).
"""
import time

import torch

from .. import _lib as L
from .. import core
from .. import hip_ops as H
from ..core import BatchFusedFWD, MOLECore
from ..utils import Ugate
from ..utils.Utimer import UATimer
from ..utils.Uparam import CPUHostBatchedParameter, GPUHostBatchedParameter, UnifiedCPUTensor
from . import fast_dispatch as tutel_fast_dispatcher


class pfetchbwd(torch.autograd.Function):
    """Identity on the layer input whose backward - which runs once this layer's own backward is
    done - starts the previous layer's backward prefetch (the counterpart of layer.py:464-472; the
    reference calls it at layer.py:436 without defining it)."""

    @staticmethod
    def forward(ctx, input_, module):
        ctx.module = module
        return input_.view_as(input_)

    @staticmethod
    def backward(ctx, grad):
        m = ctx.module
        if m.moe_id > 0:
            prev = MOLEModule._instance[m.moe_id - 1]
            if prev.global_prefetch:
                prev.global_prefetch_bwd()
            prev.local_prefetch_bwd()
        return grad, None


class _FusedMoE(torch.autograd.Function):
    """x [S,M] -> y [S,M] on the ragged layout; the whole of layer.py:442-458 in one node."""

    @staticmethod
    def forward(ctx, x, wg, dummy_param, module, capacity_factor, time_it=False):
        m = module
        ctx.time_it = time_it
        # an output the loss does not use (l_aux, mostly) arrives as None in backward instead of as a tensor of zeros
        # that autograd would have to fill first: one small kernel and its place in the queue less per step
        ctx.set_materialize_grads(False)
        S, M = x.shape
        k = min(m.topk, m.total_experts)
        scores, r = Ugate.gate_scores_route(x, wg, m.gate[0].logit_bias, k, capacity_factor, m.normalize_gate)
        rows = S * k
        if capacity_factor > 0:
            E = m.total_experts
            rows = min(rows, E * k * int(capacity_factor * ((S + E - 1) // E)))
        xd = H.dispatch_fwd(x, r.row, max(rows, 1))
        out, saved = m.MOLECore.forward(xd, True, r.offsets, r.kept_rows, return_saved=True)
        y = H.combine_fwd(out, r.row, r.gates)
        m.last_route = r
        ctx.m, ctx.r, ctx.saved = m, r, saved
        ctx.save_for_backward(x, wg, scores, out)
        return y, r.l_aux.view(())

    @staticmethod
    def backward(ctx, dy, d_l_aux):
        m, r = ctx.m, ctx.r
        x, wg, scores, out = ctx.saved_tensors
        if dy is None:            # only l_aux was used
            dy = torch.zeros_like(x)
        if ctx.time_it:
            UATimer.track_bwd_start(m.moe_id)
        # l_aux reaches the gate only when the caller added it to the loss (an unused output arrives as zeros,
        # which costs nothing: the term rides along in the same kernel)
        aux = {} if d_l_aux is None else dict(counts0=r.counts[0], d_l_aux=d_l_aux)
        d_o, dlogits = H.combine_bwd_gate(dy.contiguous(), out, r.row, r.gates, scores, r.idx, m.normalize_gate,
                                          through_softmax=True, **aux)
        gxd = m.MOLECore.backward(d_o, saved=ctx.saved)
        ctx.saved = None
        wg32 = wg.detach().float().contiguous()
        dx = H.dispatch_bwd(gxd, r.row, dlogits, wg32)
        dwg = H.gate_wgrad(dlogits, x).to(wg.dtype)
        if ctx.time_it:
            UATimer.track_bwd_end(m.moe_id)
        return dx, dwg, torch.zeros_like(m.dummy_param), None, None, None


class MOLEModule(torch.nn.Module):
    _instance = []
    _fwdgaps = []
    _bwdgaps = []
    _forwarding_count = None
    _backwarding_count = None
    _cpu_optimizer = None
    use_prefetch = True
    _moe_scale = 1.0
    step = 0

    def __init__(self, total_d_experts, total_s_experts, embed_dim, ffn_dim, pool_size, topk, ebatch_size, dist, act,
                 acc_step, adv_adam, use_pool, pool_for_extra=[False, False, False], overlap=True,
                 gate_control_by_umoe=True, hybrid_adam=False, device_s_experts=-1, dtype=torch.float32,
                 normalize_gate=True, gelu_bwd="tanh", gate_logit_bias=None, reference_layout=False,
                 activated_only=True, resident=True):
        super().__init__()
        if not torch.cuda.is_available():
            raise RuntimeError("MOLEModule needs an MI355X: the expert path exists only as HIP kernels")
        self.acc_step = acc_step
        self.topk = topk
        self.local_rank = dist["local_rank"]
        self.world_size = dist["world_size"]
        self.rank = dist["rank"]
        self.device = torch.device(f"cuda:{self.local_rank}")
        self.param_dtype = dtype
        self.normalize_gate = normalize_gate
        self.reference_layout = reference_layout

        core.create_UniMem(self.local_rank, pool_size, dtype, [[ffn_dim, embed_dim], [ffn_dim], [ffn_dim, embed_dim],
                                                              [embed_dim]])
        assert total_d_experts % self.world_size == 0
        assert total_s_experts % self.world_size == 0
        use_pool = use_pool if pool_size != -1 else False

        self.MOLECore = MOLECore(use_pool, pool_for_extra[0], pool_for_extra[1], pool_for_extra[2],
                                 total_s_experts // self.world_size, total_d_experts // self.world_size, ebatch_size,
                                 dist["world_size"], act, adv_adam, acc_step, 0, dist["local_rank"],
                                 len(MOLEModule._instance), total_d_experts + total_s_experts, gelu_bwd=gelu_bwd,
                                 activated_only=activated_only, resident=resident)

        # only EP = DP; on one GPU every expert is local
        self.d_experts = total_d_experts // self.world_size
        self.s_experts = total_s_experts // self.world_size
        self.total_experts = total_d_experts + total_s_experts
        self.pool_size = pool_size
        self.use_pool = use_pool
        self.ebatch_size = ebatch_size
        self.embed_dim = embed_dim
        self.ffn_dim = ffn_dim

        # the gate is a plain list unless torch is to own it (layer.py:75-78)
        self.gate = [Ugate.MOLETopk(embed_dim, self.total_experts)]
        if not gate_control_by_umoe:
            self.gate = torch.nn.ModuleList(self.gate)
        self.gate[0].linear = self.gate[0].linear.to(device=self.device)
        if gate_logit_bias is not None:
            self.gate[0].logit_bias = gate_logit_bias.to(device=self.device, dtype=torch.float32).contiguous()

        # exists so that autograd records the expert node (layer.py:80-81)
        self.dummy_param = torch.empty(0, device=self.device, requires_grad=True)
        self.capacity_on = True
        self.act_str = act
        assert isinstance(act, str)

        gp = dict(dtype=dtype, device=self.device, moe=self.MOLECore)
        self.FC1_W_GPU = GPUHostBatchedParameter(size=[ffn_dim, embed_dim], count=self.s_experts, p_id=0, **gp)
        self.FC1_B_GPU = GPUHostBatchedParameter(size=[ffn_dim], count=self.s_experts, bias=True, p_id=1,
                                                 fan_in=embed_dim, **gp)
        self.FC2_W_GPU = GPUHostBatchedParameter(size=[ffn_dim, embed_dim], count=self.s_experts, p_id=2,
                                                 transposed=True, **gp)
        self.FC2_B_GPU = GPUHostBatchedParameter(size=[embed_dim], count=self.s_experts, bias=True, p_id=3,
                                                 fan_in=ffn_dim, **gp)
        # device_s_experts > 0: the offloaded experts of all layers share one pinned host pool (layer.py:98-100)
        UnifiedCPUTensor()
        UnifiedCPUTensor.init([[ffn_dim, embed_dim], [ffn_dim], [ffn_dim, embed_dim], [embed_dim]], device_s_experts,
                              dtype, with_adam_state=bool(adv_adam))
        cp = dict(dtype=dtype, moe=self.MOLECore, device_s_experts=device_s_experts)
        self.FC1_W_CPU = CPUHostBatchedParameter(size=[ffn_dim, embed_dim], count=self.d_experts, p_id=0, **cp)
        self.FC1_B_CPU = CPUHostBatchedParameter(size=[ffn_dim], count=self.d_experts, p_id=1, bias=True,
                                                 fan_in=embed_dim, **cp)
        self.FC2_W_CPU = CPUHostBatchedParameter(size=[ffn_dim, embed_dim], count=self.d_experts, p_id=2,
                                                 transposed=True, **cp)
        self.FC2_B_CPU = CPUHostBatchedParameter(size=[embed_dim], count=self.d_experts, p_id=3, bias=True,
                                                 fan_in=ffn_dim, **cp)

        self.overlap = overlap
        self.adv_adam = adv_adam
        self.hybrid_adam = hybrid_adam
        self.use_prefetch = False
        self.local_prefetch_fwd_count = 0
        self.local_prefetch_bwd_count = 0
        self.global_prefetch_fwd_count = 0
        self.global_prefetch_bwd_count = 0
        self.global_prefetch = False
        self.grad_use_pool, self.mome_use_pool, self.vari_use_pool = pool_for_extra
        self.l_aux = None
        self.moe_id = len(MOLEModule._instance)
        MOLEModule._instance.append(self)

    # ---- prefetch API (layer.py:138-180) -----------------------------------------------------
    def dummy_fetch(self, batch_size):
        torch.cuda.synchronize()
        time0 = time.time()
        if self.pool_size >= 1 and self.d_experts > 0:
            self.MOLECore.dummy_fetch(min(self.d_experts, batch_size))
        core.synchronize_tran()
        torch.cuda.synchronize()
        return time.time() - time0

    def global_prefetch_fwd(self):
        for batch in self.global_prefetch_fwd_count or []:
            MOLEModule._instance[batch[0]].MOLECore.prefetch_fwd(batch[1])

    def global_prefetch_bwd(self):
        for batch in self.global_prefetch_bwd_count or []:
            MOLEModule._instance[batch[0]].MOLECore.prefetch_bwd(batch[1])

    def local_prefetch_fwd(self):
        self.MOLECore.prefetch_fwd(self.local_prefetch_fwd_count)

    def local_prefetch_bwd(self):
        self.MOLECore.prefetch_bwd(self.local_prefetch_bwd_count)

    def prefetch_fwd(self, batch_size):
        self.MOLECore.prefetch_fwd(batch_size)

    def prefetch_bwd(self, batch_size):
        self.MOLECore.prefetch_bwd(batch_size)

    def set_prefetch(self, fwd_prefetch_num, bwd_prefetch_num):
        self.fwd_prefetch_num = fwd_prefetch_num
        self.bwd_prefetch_num = bwd_prefetch_num
        self.actual_prefetch_num = max(fwd_prefetch_num, bwd_prefetch_num)
        self.local_prefetch_fwd_count = fwd_prefetch_num
        self.local_prefetch_bwd_count = bwd_prefetch_num
        self.use_prefetch = True
        self.prefetched_fwd = 0
        self.prefetched_bwd = 0

    # ---- forward (layer.py:429-476) -----------------------------------------------------------
    def forward(self, input_, adam_param={"beta1": 0.9, "beta2": 0.999, "lr": 0.001, "t": 100, "lam": 1, "eps": 1e-8},
                capacity_factor=1.0, time_it=False, prefetch=False):
        original_shape = input_.shape
        original_dtype = input_.dtype
        if time_it:      # the profiling window of the scheduler: this layer's forward and backward spans are recorded
            UATimer.track_fwd_start(self.moe_id)
        if prefetch:
            input_ = pfetchbwd.apply(input_, self)
        resized_input = input_.reshape(-1, self.embed_dim)
        if resized_input.dtype != self.param_dtype:
            resized_input = resized_input.to(self.param_dtype)
        resized_input = resized_input.contiguous()

        if self.reference_layout:
            scores = self.gate[0](resized_input)
            crit, l_aux = tutel_fast_dispatcher.extract_critical(
                scores, top_k=self.topk, capacity_factor=capacity_factor, normalize_gate=self.normalize_gate)
            self.l_aux = l_aux
            dispatched_input = tutel_fast_dispatcher.fast_encode(data=resized_input, critial_data=crit)
            experts_output = BatchFusedFWD.apply(dispatched_input, self, self.dummy_param, time_it, prefetch)
            expert_output = tutel_fast_dispatcher.fast_decode(data=experts_output, critial_data=crit)
        else:
            expert_output, self.l_aux = _FusedMoE.apply(resized_input, self.gate[0].linear.weight, self.dummy_param,
                                                        self, float(capacity_factor), bool(time_it))

        expert_output = expert_output.reshape(original_shape)
        out = expert_output.to(original_dtype)
        if time_it:
            UATimer.track_fwd_end(self.moe_id)

        if prefetch:
            if self.moe_id < len(MOLEModule._instance) - 1:
                nxt = MOLEModule._instance[self.moe_id + 1]
                if self.global_prefetch:
                    nxt.global_prefetch_fwd()
                nxt.local_prefetch_fwd()
            elif self.moe_id == len(MOLEModule._instance) - 1:
                if self.global_prefetch:
                    MOLEModule._instance[-1].global_prefetch_bwd()
                MOLEModule._instance[-1].local_prefetch_bwd()
        return out

    # ---- optimizer hooks (layer.py:135-136, 343-348) --------------------------------------------
    def set_hybrid_adam_count(self, hybrid_adam_count):
        self.MOLECore.set_hybrid_adam_count(hybrid_adam_count)

    def unset_lazy_zero(self):
        for p in (self.FC1_W_CPU, self.FC1_B_CPU, self.FC2_W_CPU, self.FC2_B_CPU):
            p.unset_lazy_zero()

    def set_lazy_zero(self):
        self.MOLECore.set_lazy_zero()

    # ---- layer state for checkpoints (layer.py:350-427) ------------------------------------------
    def _expert_stores(self):
        """(parameter store of kind p for the GPU-resident experts, for the offloaded ones), p = 0..3"""
        return ((self.FC1_W_GPU, self.FC1_W_CPU), (self.FC1_B_GPU, self.FC1_B_CPU),
                (self.FC2_W_GPU, self.FC2_W_CPU), (self.FC2_B_GPU, self.FC2_B_CPU))

    @torch.no_grad()
    def get_layer_state(self, grad):
        """{"gate": [weight, bias or None], "experts": one [fc1_w, fc1_b, fc2_w, fc2_b] per expert (GPU-resident
        first, then offloaded), "grad": the same per expert, then the gate's gradients; empty unless grad}: all
        CPU tensors, the layout MOLEModule.get_layer_state returns in the reference."""
        core.synchronize_tran()           # host arrays may still be the target of a write-back
        lin = self.gate[0].linear
        state = {"gate": [lin.weight.detach().cpu(), lin.bias.detach().cpu() if lin.bias is not None else None]}
        experts, grads = [], []
        for which, count in ((0, self.s_experts), (1, self.d_experts)):
            for i in range(count):
                experts.append([st[which].fetch_single(i).detach().cpu().clone() for st in self._expert_stores()])
        if grad:
            for which, count in ((0, self.s_experts), (1, self.d_experts)):
                for i in range(count):
                    grads.append([st[which].fetch_single_grad(i).detach().cpu().clone() for st in self._expert_stores()])
            grads.append(lin.weight.grad.cpu() if lin.weight.grad is not None else None)
            grads.append(lin.bias.grad.cpu() if lin.bias is not None and lin.bias.grad is not None else None)
        state["experts"], state["grad"] = experts, grads
        return state

    @torch.no_grad()
    def set_layer_state(self, states, grad):
        """Inverse of get_layer_state (layer.py:350-395)."""
        core.synchronize_tran()           # no prefetch may be reading the host arrays while they change
        torch.cuda.synchronize()
        lin = self.gate[0].linear
        lin.weight.copy_(states["gate"][0])
        if lin.bias is not None:
            lin.bias.copy_(states["gate"][1])
        j = 0
        for which, count in ((0, self.s_experts), (1, self.d_experts)):
            for i in range(count):
                for st, t in zip(self._expert_stores(), states["experts"][j]):
                    st[which].fetch_single(i).copy_(t)
                j += 1
        if grad:
            gs = states["grad"]
            j = 0
            for which, count in ((0, self.s_experts), (1, self.d_experts)):
                for i in range(count):
                    for st, t in zip(self._expert_stores(), gs[j]):
                        st[which].fetch_single_grad(i).copy_(t)
                    j += 1
            self.MOLECore.host_gradients_changed()
            lin.weight.grad = None if gs[j] is None else gs[j].to(lin.weight.device)
            if lin.bias is not None and gs[j + 1] is not None:
                lin.bias.grad = gs[j + 1].to(lin.bias.device)

    # ---- parameter access (layer.py:478-500) ---------------------------------------------------
    def d_experts_param(self):
        if self.d_experts > 0:
            return [self.FC1_W_CPU.all_tensors, self.FC1_B_CPU.all_tensors, self.FC2_W_CPU.all_tensors,
                    self.FC2_B_CPU.all_tensors]
        return []

    def s_experts_param(self):
        if self.s_experts > 0:
            return [self.FC1_W_GPU.fetch_all_with_grad(), self.FC1_B_GPU.fetch_all_with_grad(),
                    self.FC2_W_GPU.fetch_all_with_grad(), self.FC2_B_GPU.fetch_all_with_grad()]
        return []

    def gate_param(self):
        lin = self.gate[0].linear
        return [lin.weight, lin.bias] if lin.bias is not None else [lin.weight]

    @classmethod
    def reset_instances(cls):
        """Forget all layers and free the process-global slot pool (tests, benchmarks)."""
        cls._instance = []
        core.destroy_UniMem()
        UnifiedCPUTensor.reset()
