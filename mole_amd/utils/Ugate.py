"""Gate of the MoE layer: Linear without bias, softmax over experts.

Mirror of MOLE/utils/Ugate.py:5-14 (same class name, same `linear` attribute).  For bf16 tokens the scores
come from one fused kernel of the C ABI (mole_gate_fwd); otherwise the logits come from the MFMA NT GEMM
(mole_gemm_nt) and the softmax from mole_softmax_fwd.  The backward is the softmax/linear backward in the
same library: mole_softmax_bwd, then dlogits . Wg and dlogits^T . x on the grouped-GEMM tiles / the gate
weight-gradient kernel.  `logit_bias` ([E], optional, not trained) is
added to the logits before the softmax - the reference gate has none.
"""
import torch

from .. import hip_ops as H


class _GateFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, logit_bias):
        scores = gate_scores(x, weight, logit_bias)
        ctx.save_for_backward(x, weight, scores)
        return scores

    @staticmethod
    def backward(ctx, dscores):
        x, weight, scores = ctx.saved_tensors
        dlogits = H.softmax_bwd(dscores.float().contiguous(), scores)
        xc = x.detach().contiguous()
        dx = H.gate_input_grad(dlogits, weight.detach().float(), x.dtype) if ctx.needs_input_grad[0] else None
        dw = H.gate_wgrad(dlogits, xc).to(weight.dtype) if ctx.needs_input_grad[1] else None
        return dx, dw, None


def gate_scores(x: torch.Tensor, weight: torch.Tensor, logit_bias=None) -> torch.Tensor:
    """softmax(x @ weight.T + logit_bias) in fp32; x [S,M] fp32 or bf16, weight [E,M] fp32."""
    return H.gate_fwd(x.detach().contiguous(), weight.detach().contiguous(), logit_bias)


def gate_scores_route(x: torch.Tensor, weight: torch.Tensor, logit_bias, top_k: int, capacity_factor: float,
                      normalize_gate: bool):
    """(gate_scores(x, weight, logit_bias), the routing of those scores on the ragged layout): what MOLETopk.forward and
    tutel's extract_critical do between them (MOLE/moe/layer.py:442-446), in one library call where it offers one."""
    return H.gate_route(x.detach().contiguous(), weight.detach().contiguous(), logit_bias, top_k, capacity_factor,
                        normalize_gate)


class MOLETopk(torch.nn.Module):
    def __init__(self, model_dim, total_experts) -> None:
        super().__init__()
        self.total_experts = total_experts
        self.linear = torch.nn.Linear(model_dim, total_experts, bias=False)
        self.logit_bias = None

    def forward(self, input):
        return _GateFn.apply(input, self.linear.weight, self.logit_bias)
