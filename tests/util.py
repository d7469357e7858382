"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """max |got - want| / max |want|: the relative error the 1e-5 (fp32) and 2e-2 (bf16)
    tolerances of the parity tests are stated in."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    denom = float(want.abs().max())
    if denom == 0.0:
        return float(got.abs().max())
    return float((got - want).abs().max()) / denom


def rel_err_dev(got: torch.Tensor, want: torch.Tensor) -> float:
    """rel_err evaluated where the tensors live (fp32 arithmetic on the GPU): for comparisons of hundreds of
    megabytes, where the trip through fp64 on the host would dominate the test."""
    got, want = got.detach().float(), want.detach().float().to(got.device)
    denom = float(want.abs().max()) if want.numel() else 0.0
    diff = float((got - want).abs().max()) if want.numel() else 0.0
    return diff if denom == 0.0 else diff / denom


def row_rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """max over rows of max_j |got[i,j] - want[i,j]| / max_j |want[i,j]|: every row is held to the tolerance
    relative to its own magnitude, so that a row of small values cannot hide behind a large one elsewhere.
    Rows whose reference is all zero count with their absolute error."""
    got = got.detach().double().cpu().reshape(-1, got.shape[-1])
    want = want.detach().double().cpu().reshape(-1, want.shape[-1])
    if want.numel() == 0:
        return 0.0
    diff = (got - want).abs().amax(dim=1)
    mag = want.abs().amax(dim=1)
    return float(torch.where(mag > 0, diff / mag.clamp_min(1e-300), diff).max())


def expert_rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """max over experts e of max |got[e] - want[e]| / max |want[e]| for [E, ...] parameter gradients: every expert
    is held to the tolerance relative to its own largest gradient, so that an expert with few rows and small
    gradients cannot hide behind a loaded one.  An expert whose reference gradient is all zero (no rows) counts
    with its absolute error."""
    E = want.shape[0]
    got = got.detach().double().cpu().reshape(E, -1)
    want = want.detach().double().cpu().reshape(E, -1)
    if want.numel() == 0:
        return 0.0
    diff = (got - want).abs().amax(dim=1)
    mag = want.abs().amax(dim=1)
    return float(torch.where(mag > 0, diff / mag.clamp_min(1e-300), diff).max())


FP32_TOL = 1e-5
BF16_TOL = 2e-2


def tol(dtype) -> float:
    return FP32_TOL if dtype == torch.float32 else BF16_TOL


def zipf_scores(S, E, seed, ties=False):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(S, E, generator=g)
    logits += torch.log(torch.arange(1, E + 1, dtype=torch.float32) ** -1.2)[torch.randperm(E, generator=g)]
    s = torch.softmax(logits, dim=-1)
    if ties and E >= 4:
        s[:, E - 1] = s[:, 0]          # whole duplicated columns: exact ties in every row
        s[::3, 1] = s[::3, 2]
    return s.contiguous()


def crit_to_numpy(r):
    """mole_amd.hip_ops.Route -> dict of numpy arrays (one host copy for the whole comparison)."""
    return dict(idx=r.idx.cpu().numpy(), loc=r.loc.cpu().numpy(), gates=r.gates.cpu().numpy(),
                row=r.row.cpu().numpy(), counts=r.counts.cpu().numpy(), kept=r.kept_rows.cpu().numpy(),
                offsets=r.offsets.cpu().numpy(), capacity=int(r.capacity.cpu()), l_aux=float(r.l_aux.cpu()))
