"""Actor-side per-token helpers that sit next to the loss: proximal log-prob approximations and M2PO masking.

Host-side mirror of ``compute_prox_logp_approximations`` (areal/trainer/ppo/actor.py:604-684) and
``_apply_m2po_masking`` (areal/trainer/ppo/actor.py:769-850).
"""
from __future__ import annotations

import torch

from . import _native as N
from .functional import _f32, _mask_u8, _ptr, _require_gpu, _stream

PROX_APPROX_METHOD_LOGLINEAR = "loglinear"
PROX_APPROX_METHOD_LINEAR = "linear"
PROX_APPROX_METHOD_ROLLOUT = "rollout"
PROX_APPROX_METHODS_ALL = [PROX_APPROX_METHOD_LOGLINEAR, PROX_APPROX_METHOD_LINEAR, PROX_APPROX_METHOD_ROLLOUT]
_METHOD_IDS = {PROX_APPROX_METHOD_LOGLINEAR: 0, PROX_APPROX_METHOD_LINEAR: 1, PROX_APPROX_METHOD_ROLLOUT: 2}


@torch.no_grad()
def compute_prox_logp_approximations(old_logp: torch.Tensor, logprobs: torch.Tensor, versions: torch.Tensor,
                                     current_version: int, method: str | None = None) -> dict[str, torch.Tensor]:
    """Version-aware interpolation between behaviour and current log-probs; actor.py:604-684.

    Returns ``{method: tensor}`` for the one method asked for, or for all three when ``method`` is None.  Unknown
    method names give an empty dict, as in the reference.
    """
    _require_gpu(old_logp, "old_logp")
    shape = old_logp.shape
    lo = _f32(old_logp.detach()).reshape(-1)
    ln = _f32(logprobs.detach()).reshape(-1)
    ver = versions.to(device=lo.device, dtype=torch.int32).contiguous().reshape(-1)
    if not (lo.numel() == ln.numel() == ver.numel()):
        raise ValueError("old_logp, logprobs and versions must have the same number of elements")
    lib = N.load()
    out = {}
    for m in ([method] if method else PROX_APPROX_METHODS_ALL):
        if m not in _METHOD_IDS:
            continue
        res = torch.empty_like(lo)
        with torch.cuda.device(lo.device):
            N.check(lib.aa_prox_logp_approx(_ptr(lo), _ptr(ln), _ptr(ver), lo.numel(), int(current_version),
                                            _METHOD_IDS[m], _ptr(res), _stream(lo.device)), "aa_prox_logp_approx")
        out[m] = res.view(shape)
    return out


@torch.no_grad()
def apply_m2po_masking(old_logp: torch.Tensor, prox_logp: torch.Tensor, loss_mask: torch.Tensor,
                       m2_threshold: float) -> torch.Tensor:
    """Loss mask with the highest second-momentum tokens removed; actor.py:769-850.

    Tokens are dropped from the largest ``(old_logp - prox_logp) ** 2`` down until the mean over the remaining valid
    tokens is below ``m2_threshold``; at least one valid token is always kept.  Returns a bool mask of the shape of
    ``loss_mask``.
    """
    _require_gpu(old_logp, "old_logp")
    shape = loss_mask.shape
    lo = _f32(old_logp.detach()).reshape(-1)
    lp = _f32(prox_logp.detach()).reshape(-1)
    m8 = _mask_u8(loss_mask).reshape(-1)
    n = m8.numel()
    if not (lo.numel() == lp.numel() == n):
        raise ValueError("old_logp, prox_logp and loss_mask must have the same number of elements")
    if n == 0:
        return loss_mask.bool()
    lib = N.load()
    dev = lo.device
    ws = torch.empty(lib.aa_m2po_workspace_bytes(n), dtype=torch.uint8, device=dev)
    out = torch.empty(n, dtype=torch.bool, device=dev)
    info = torch.empty(2, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        N.check(lib.aa_m2po_mask(_ptr(lo), _ptr(lp), _ptr(m8), n, float(m2_threshold), _ptr(out), _ptr(info), _ptr(ws),
                                 ws.numel(), _stream(dev)), "aa_m2po_mask")
    return out.view(shape)


class _KdTerms(torch.autograd.Function):
    """sum(term) / max(sum(mask), 1) of ``aa_kd_terms`` and the per-token terms; differentiable in ``logp``."""

    @staticmethod
    def forward(ctx, logp, old, teacher, mask_u8, pure):
        from .functional import _count_nonzero

        lib = N.load()
        dev = logp.device
        n = logp.numel()
        term = torch.empty(n, dtype=torch.float32, device=dev)
        dterm = torch.empty(n, dtype=torch.float32, device=dev)
        mean = torch.empty((), dtype=torch.float32, device=dev)
        n_valid = _count_nonzero(mask_u8)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(lib.aa_kd_terms(_ptr(logp), _ptr(old), _ptr(teacher), _ptr(mask_u8), n, 1 if pure else 0, _ptr(term),
                                    _ptr(dterm), st), "aa_kd_terms")
            N.check(lib.aa_masked_sum(_ptr(term), None, n, _ptr(n_valid), None, _ptr(mean), st), "aa_masked_sum")
        ctx.save_for_backward(dterm, n_valid)
        ctx.mark_non_differentiable(term)
        return mean, term

    @staticmethod
    def backward(ctx, g_mean, _g_term):
        dterm, n_valid = ctx.saved_tensors
        return dterm * (g_mean / n_valid.clamp(min=1).float()), None, None, None, None


def distillation_terms(logprobs: torch.Tensor, old_logp: torch.Tensor | None, teacher_logp: torch.Tensor,
                       loss_mask: torch.Tensor, pure: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """The reverse-KL terms of the joint-distillation branch of the actor loss; actor.py:482-511.

    ``pure`` (``rl_loss_weight == 0``): per token ``exp(logp - old) * (teacher - logp.detach()) * mask``
    (actor.py:494-498); otherwise ``(logp - teacher) * mask`` (actor.py:505).  Returns
    ``(sum(term) / max(sum(mask), 1), term)``: the first is differentiable in ``logprobs``, the second is detached.
    """
    _require_gpu(logprobs, "logprobs")
    shape = logprobs.shape
    if teacher_logp.shape != shape or loss_mask.shape != shape or (pure and old_logp.shape != shape):
        raise ValueError("logprobs, old_logp, teacher_logp and loss_mask must have the same shape")
    lp = logprobs.reshape(-1)
    if lp.dtype != torch.float32 or not lp.is_contiguous():
        lp = lp.float().contiguous()
    old = _f32(old_logp.detach()).reshape(-1) if pure else None
    mean, term = _KdTerms.apply(lp, old, _f32(teacher_logp.detach()).reshape(-1), _mask_u8(loss_mask).reshape(-1),
                                bool(pure))
    return mean, term.view(shape)
