"""Actor-side per-token helpers that sit next to the loss: proximal log-prob approximations and M2PO masking.

Host-side mirror of ``compute_prox_logp_approximations`` (areal/trainer/ppo/actor.py:604-684) and
``_apply_m2po_masking`` (areal/trainer/ppo/actor.py:769-850).
"""
from __future__ import annotations

from typing import Any

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


_LOGSTAT_METHOD_KEYS = ("approx_logp", "behave_imp_weight", "importance_weight", "abs_error", "rel_error",
                        "squared_error", "behave_imp_weight_abs_error", "behave_imp_weight_rel_error",
                        "importance_weight_abs_error", "importance_weight_rel_error")


def _moment_rows(table: torch.Tensor) -> list[dict[str, torch.Tensor]]:
    """``[rows, 4]`` of {sum, min, max, count} -> one dict of 0-d tensors per row, with one division for all rows."""
    cols = torch.cat([table, (table[:, 0] / table[:, 3])[:, None]], dim=1)
    rows = []
    for row in cols.unbind(0):
        s, lo, hi, c, avg = row.unbind(0)
        rows.append(dict(sum=s, avg=avg, min=lo, max=hi, count=c))
    return rows


@torch.no_grad()
def proximal_logging_stats(old_logp: torch.Tensor, logprobs: torch.Tensor, prox_logp_gt: torch.Tensor | None,
                           versions: torch.Tensor | None, current_version: int | None, mask: torch.Tensor,
                           prox_logp_method: str = "recompute") -> dict[str, dict]:
    """What ``grpo_loss_fn`` logs under its ``compute_logp`` and ``version_stats`` scopes (actor.py:573-594,
    982-1110), already reduced over ``mask``: one pass over the tokens instead of one tensor and one reduction per
    logged quantity.

    Returns ``{"compute_logp": {name: moments}, "version_stats": {...}}`` with ``moments`` = ``{"sum", "avg", "min",
    "max", "count"}`` of 0-d device tensors.  The names and the conditions under which each appears are the
    reference's: ``prox_logp_gt`` whenever it is given; nothing more without ``versions`` / ``current_version``;
    ``loglinear/{approx_logp, behave_imp_weight, importance_weight}`` for the ``"loglinear"`` method; all three
    methods with their error metrics for ``"metrics"`` with ground truth; ``kl_div_direct / taylor / dual``.
    ``version_stats`` holds ``sample_staleness_proximal``, ``sample_staleness_theta`` (moments over the selected
    tokens with ``version >= 0``; ``count`` is ``n_valid_generated_tokens``), ``v_theta`` and ``v_proximal``; it
    is empty without versions.  Nothing is read back: whether any generated token is selected is the ``count``.
    """
    _require_gpu(old_logp, "old_logp")
    lo = _f32(old_logp.detach()).reshape(-1)
    ln = _f32(logprobs.detach()).reshape(-1)
    m8 = _mask_u8(mask.to(lo.device)).reshape(-1)
    n = lo.numel()
    if ln.numel() != n or m8.numel() != n:
        raise ValueError("old_logp, logprobs and mask must have the same number of elements")
    gt = _f32(prox_logp_gt.detach()).reshape(-1) if prox_logp_gt is not None else None
    have_versions = versions is not None and current_version is not None
    ver = versions.to(device=lo.device, dtype=torch.int32).contiguous().reshape(-1) if have_versions else None
    methods, with_errors = 0, False
    if have_versions and prox_logp_method == "loglinear":
        methods = 1
    elif have_versions and prox_logp_method == "metrics" and gt is not None:
        methods, with_errors = 7, True
    lib = N.load()
    dev = lo.device
    out = torch.empty(36, 4, dtype=torch.float32, device=dev)
    scratch = torch.empty(lib.aa_logging_stats_scratch_bytes(n), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        N.check(lib.aa_logging_stats(_ptr(lo), _ptr(ln), _ptr(gt), _ptr(ver), _ptr(m8), n,
                                     int(current_version) if have_versions else 0, methods, 1 if with_errors else 0,
                                     _ptr(out), _ptr(scratch), scratch.numel(), _stream(dev)), "aa_logging_stats")
    rows = _moment_rows(out)
    compute_logp: dict[str, dict] = {}
    if gt is not None:
        compute_logp["prox_logp_gt"] = rows[0]
    version_stats: dict[str, Any] = {}
    if have_versions:
        for m, name in enumerate(PROX_APPROX_METHODS_ALL):
            if not (methods >> m) & 1:
                continue
            for j, key in enumerate(_LOGSTAT_METHOD_KEYS[: 10 if with_errors else 3]):
                compute_logp[f"{name}/{key}"] = rows[4 + 10 * m + j]
        for j, key in enumerate(("kl_div_direct", "kl_div_taylor", "kl_div_dual")):
            compute_logp[key] = rows[1 + j]
        version_stats = dict(sample_staleness_proximal=rows[34],
                             sample_staleness_theta=rows[35],
                             v_theta=int(current_version), v_proximal=int(current_version) - 1)
    return dict(compute_logp=compute_logp, version_stats=version_stats)
