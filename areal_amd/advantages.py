"""Advantage pipeline of the PPO actor on the GPU: GAE, reward / advantage normalisation, masked moments.

Host-side mirror of ``Normalization`` (areal/utils/data.py:1378-1596), of the GAE loop of
``PPOActor._compute_advantages`` (areal/trainer/ppo/actor.py:209-236) and of the masked reductions the statistics
tracker performs per tensor (areal/utils/stats_tracker.py:227-285).  Everything runs in the HIP library; CPU tensors
are refused.
"""
from __future__ import annotations

import ctypes as C
from typing import Any, Mapping

import torch

from . import _native as N
from .functional import _f32, _mask_u8, _ptr, _require_gpu, _stream

_LEVELS = {None: 0, "none": 0, "batch": 1, "group": 2}


class Normalization:
    """``Normalization(config)(x, loss_mask)`` with the reference's semantics (data.py:1378-1504).

    ``config`` is any object with the attributes of ``NormConfig``.  Sums are accumulated in float64 whatever
    ``high_precision`` says.  One process only: with ``torch.distributed`` initialised on more than one rank the
    batch-level statistics would need an all-reduce, which this build does not have.
    """

    def __init__(self, config: Any):
        self.mean_level = config.mean_level
        self.mean_leave1out = config.mean_leave1out
        self.std_level = config.std_level
        self.std_unbiased = config.std_unbiased
        self.group_size = config.group_size
        self.eps = config.eps
        for name, level in (("mean_level", self.mean_level), ("std_level", self.std_level)):
            if level not in _LEVELS:
                raise ValueError(f"{name} must be 'batch', 'group' or None, got {level}")
        if (self.mean_level == "group" or self.std_level == "group") and self.group_size < 1:
            raise ValueError(
                f"group_size must be a positive integer when using group normalization, got {self.group_size}"
            )

    @torch.no_grad()
    def __call__(self, x: torch.Tensor, loss_mask: torch.Tensor | None = None, high_precision: bool = True,
                 reduce_group=None) -> torch.Tensor:
        _require_gpu(x, "x")
        if torch.distributed.is_available() and torch.distributed.is_initialized():
            if torch.distributed.get_world_size(reduce_group) > 1:
                raise NotImplementedError("Normalization across ranks is not part of this build (one GPU)")
        if loss_mask is not None and loss_mask.shape != x.shape:
            raise ValueError(f"loss_mask shape {tuple(loss_mask.shape)} != x shape {tuple(x.shape)}")
        if x.ndim == 0:
            raise ValueError("x must have a batch dimension")
        bs = x.shape[0]
        if x.numel() == 0:
            return x.float()
        xf = _f32(x)
        mf = None if loss_mask is None else _f32(loss_mask)
        inner = xf.numel() // bs
        params = N.NormParams(_LEVELS[self.mean_level], int(bool(self.mean_leave1out)), _LEVELS[self.std_level],
                              int(bool(self.std_unbiased)), float(self.eps), int(self.group_size))
        lib = N.load()
        dev = xf.device
        grouped = params.mean_level == 2 or params.std_level == 2
        n_bytes = lib.aa_normalize_scratch_bytes(bs, inner, int(self.group_size) if grouped else max(bs, 1))
        scratch = torch.empty(max(n_bytes, 32) // 8, dtype=torch.float64, device=dev)
        out = torch.empty_like(xf)
        with torch.cuda.device(dev):
            N.check(
                lib.aa_normalize(_ptr(xf), _ptr(mf), bs, inner, C.byref(params), _ptr(out), _ptr(scratch),
                                 scratch.numel() * 8, _stream(dev)),
                "aa_normalize",
            )
        return out


@torch.no_grad()
def gae_advantages(rewards: torch.Tensor, values: torch.Tensor | None, loss_mask: torch.Tensor,
                   seq_no_eos_mask: torch.Tensor | None, discount: float, gae_lambda: float
                   ) -> tuple[torch.Tensor, torch.Tensor]:
    """``(advantages, returns)`` of the GAE loop in ``PPOActor._compute_advantages`` (actor.py:209-232).

    ``rewards``, ``values``, ``loss_mask`` are the padded ``[bs, max_seqlen]`` tensors of that function (the mask
    already rolled by -1), ``seq_no_eos_mask`` is ``[bs]``; ``values=None`` stands for zeros (actor.py:210-211).
    """
    _require_gpu(rewards, "rewards")
    if rewards.ndim != 2:
        raise ValueError(f"expected rewards [bs, max_seqlen], got {tuple(rewards.shape)}")
    if loss_mask.shape != rewards.shape or (values is not None and values.shape != rewards.shape):
        raise ValueError("rewards, values and loss_mask must have the same shape")
    bs, L = rewards.shape
    if seq_no_eos_mask is not None and tuple(seq_no_eos_mask.shape) != (bs,):
        raise ValueError(f"seq_no_eos_mask shape {tuple(seq_no_eos_mask.shape)} != ({bs},)")
    assert L > 0, "max_seqlen must be positive"
    dev = rewards.device
    r, m = _f32(rewards), _f32(loss_mask)
    v = None if values is None else _f32(values)
    ne = None if seq_no_eos_mask is None else _mask_u8(seq_no_eos_mask.to(dev) != 0)
    adv = torch.empty_like(r)
    ret = torch.empty_like(r)
    lib = N.load()
    with torch.cuda.device(dev):
        N.check(
            lib.aa_gae(_ptr(r), _ptr(v), _ptr(m), _ptr(ne), bs, L, float(discount), float(gae_lambda), _ptr(adv),
                       _ptr(ret), _stream(dev)),
            "aa_gae",
        )
    return adv, ret


@torch.no_grad()
def masked_moments(values: Mapping[str, torch.Tensor], mask: torch.Tensor) -> dict[str, dict[str, torch.Tensor]]:
    """Sum, mean, min, max and count of every tensor in ``values`` over ``mask``, in one launch.

    These are the quantities ``stats_tracker.stat(..., denominator=mask)`` reduces one tensor at a time
    (stats_tracker.py:227-285).  Returns ``{name: {"sum", "avg", "min", "max", "count"}}`` of 0-d device tensors;
    ``avg`` is NaN and ``min`` / ``max`` are +/-inf when the mask selects nothing.
    """
    names = list(values)
    if not names:
        return {}
    if len(names) > 16:
        raise ValueError("at most 16 tensors per call")
    _require_gpu(mask, "mask")
    m8 = _mask_u8(mask.reshape(-1))
    n = m8.numel()
    tensors = []
    for k in names:
        t = values[k]
        _require_gpu(t, k)
        if t.numel() != n:
            raise ValueError(f"{k} has {t.numel()} elements, the mask has {n}")
        tensors.append(_f32(t.detach()).reshape(-1))
    dev = m8.device
    out = torch.empty(len(names), 4, dtype=torch.float32, device=dev)
    ptrs = (C.c_void_p * len(names))(*[t.data_ptr() for t in tensors])
    lib = N.load()
    with torch.cuda.device(dev):
        N.check(lib.aa_masked_moments(ptrs, len(names), _ptr(m8), n, _ptr(out), _stream(dev)), "aa_masked_moments")
    res = {}
    for i, k in enumerate(names):
        s, lo, hi, c = out[i, 0], out[i, 1], out[i, 2], out[i, 3]
        res[k] = dict(sum=s, avg=s / c, min=lo, max=hi, count=c)
    return res


_KL_IDS = {"k1": 0, "k2": 1, "k3": 2}


@torch.no_grad()
def kl_regularized_rewards(old_logp: torch.Tensor, ref_logp: torch.Tensor | None, loss_mask: torch.Tensor,
                           seqlens: torch.Tensor, reward_score: torch.Tensor, kl_ctl: float,
                           kl_estimator: str = "k1", mask_no_eos_with_zero: bool = False
                           ) -> tuple[torch.Tensor, torch.Tensor]:
    """``(rewards, kl_rewards)`` of ``PPOActor._compute_advantages`` (actor.py:182-207) for padded ``[bs, L]`` inputs:
    the token-level KL penalty against the reference policy, the reward at each sequence's last position cleared
    and its scalar reward added one position earlier."""
    if kl_estimator not in _KL_IDS:
        raise ValueError(f"Invalid KL estimator: {kl_estimator}. Valid choices: k1, k2, k3")
    _require_gpu(old_logp, "old_logp")
    if old_logp.ndim != 2 or loss_mask.shape != old_logp.shape:
        raise ValueError("old_logp and loss_mask must be [bs, max_seqlen] tensors of the same shape")
    bs, L = old_logp.shape
    dev = old_logp.device
    lo, m = _f32(old_logp), _f32(loss_mask)
    lr = None if ref_logp is None else _f32(ref_logp)
    sl = seqlens.to(device=dev, dtype=torch.int64).contiguous()
    sc = _f32(reward_score.to(dev)).reshape(-1)
    if sl.numel() != bs or sc.numel() != bs:
        raise ValueError("seqlens and reward_score must have one entry per sequence")
    rewards, kl_rewards = torch.empty_like(lo), torch.empty_like(lo)
    with torch.cuda.device(dev):
        N.check(
            N.load().aa_kl_rewards(_ptr(lo), _ptr(lr), _ptr(m), _ptr(sl), _ptr(sc), bs, L, float(kl_ctl),
                                   _KL_IDS[kl_estimator], int(bool(mask_no_eos_with_zero)), _ptr(rewards),
                                   _ptr(kl_rewards), _stream(dev)),
            "aa_kl_rewards",
        )
    return rewards, kl_rewards


@torch.no_grad()
def reward_overlong_penalty(data: dict, overlong_tokens: int, overlong_penalty_factor: float,
                            max_response_length: int) -> dict:
    """Length penalty on the sequence rewards, in place on ``data["rewards"]`` like the reference
    (areal/utils/functional/functional.py:782-803): a response longer than ``max_response_length - overlong_tokens``
    loses ``overlong_penalty_factor`` per ``overlong_tokens`` tokens of excess.  ``data["loss_mask"]`` is ``[bs, L]``."""
    rewards, mask = data["rewards"], data["loss_mask"]
    _require_gpu(rewards, "rewards")
    if mask.ndim != 2 or rewards.numel() != mask.shape[0]:
        raise ValueError("rewards must have one entry per row of the [bs, max_seqlen] loss_mask")
    bs, L = mask.shape
    dev = rewards.device
    r = rewards if (rewards.dtype == torch.float32 and rewards.is_contiguous()) else _f32(rewards).contiguous()
    with torch.cuda.device(dev):
        N.check(
            N.load().aa_overlong_penalty(_ptr(r), _ptr(_f32(mask.to(dev)).contiguous()), bs, L, int(overlong_tokens),
                                         float(overlong_penalty_factor), int(max_response_length), _stream(dev)),
            "aa_overlong_penalty",
        )
    if r is not rewards:
        rewards.copy_(r.view_as(rewards))
    data["rewards"] = rewards
    return data


@torch.no_grad()
def masked_normalization(x: torch.Tensor, mask: torch.Tensor | None = None, dim=None, unbiased: bool = False,
                         eps: float = 1e-5, high_precision: bool = True, all_reduce: bool = True,
                         reduce_group=None) -> torch.Tensor:
    """Whitening by the masked mean and the ``E[x^2] - E[x]^2`` variance over ``dim`` (all axes when None);
    areal/utils/functional/functional.py:16-53.  Masked positions enter as zeros and are whitened like the rest, as
    in the reference.  Returns float32 of the shape of ``x``.

    Sums are accumulated in float64 whatever ``high_precision`` says.  The sums are local: with an initialised
    process group of more than one rank and ``all_reduce=True`` the call raises ``NotImplementedError``."""
    import torch.distributed as dist

    _require_gpu(x, "x")
    if all_reduce and dist.is_available() and dist.is_initialized() and dist.get_world_size(reduce_group) > 1:
        raise NotImplementedError("masked_normalization sums over one GPU only")
    nd = x.dim()
    dims = tuple(range(nd)) if dim is None else tuple(sorted(d % nd for d in ((dim,) if isinstance(dim, int) else dim)))
    keep = [d for d in range(nd) if d not in dims]
    perm = keep + list(dims)
    xv = _f32(x).permute(perm).contiguous()
    mv = None
    if mask is not None:
        mv = _f32(mask.to(x.device)).expand(x.shape).permute(perm).contiguous()
    rows = 1
    for d in keep:
        rows *= x.shape[d]
    cols = xv.numel() // rows if rows else 0
    out = torch.empty_like(xv)
    if xv.numel():
        lib = N.load()
        dev = x.device
        scratch = torch.empty(lib.aa_masked_normalization_scratch_bytes(rows, cols), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            N.check(lib.aa_masked_normalization(_ptr(xv), _ptr(mv), rows, cols, 1 if unbiased else 0, float(eps),
                                                _ptr(out), _ptr(scratch), scratch.numel(), _stream(dev)),
                    "aa_masked_normalization")
    inv = [0] * nd
    for i, d in enumerate(perm):
        inv[d] = i
    return out.permute(inv).contiguous()


class KLEstimator:
    """k1 / k2 / k3 estimator of the KL divergence per token, optionally clamped to [-10, 10];
    areal/utils/data.py:1598-1656.  Forward only (the reference uses it on detached log-probs)."""

    def __init__(self, kl_estimator: str = "k1", apply_clamp: bool = True):
        if kl_estimator not in _KL_IDS:
            raise ValueError(f"Invalid KL estimator: {kl_estimator}. Valid choices: k1, k2, k3")
        self.kl_estimator = kl_estimator
        self.apply_clamp = apply_clamp

    def __call__(self, log_probs: torch.Tensor, log_probs_base: torch.Tensor) -> torch.Tensor:
        return self._compute_approx_kl(log_probs, log_probs_base, self.kl_estimator, self.apply_clamp)

    @staticmethod
    @torch.no_grad()
    def _compute_approx_kl(log_probs: torch.Tensor, log_probs_base: torch.Tensor, kl_estimator: str = "k1",
                           apply_clamp: bool = True) -> torch.Tensor:
        if kl_estimator not in _KL_IDS:
            raise ValueError(f"Invalid KL estimator: {kl_estimator}. Valid choices: k1, k2, k3")
        _require_gpu(log_probs, "log_probs")
        if log_probs_base.shape != log_probs.shape:
            raise ValueError("log_probs and log_probs_base must have the same shape")
        a, b = _f32(log_probs), _f32(log_probs_base.to(log_probs.device))
        out = torch.empty_like(a)
        with torch.cuda.device(a.device):
            N.check(N.load().aa_kl_estimate(_ptr(a), _ptr(b), a.numel(), _KL_IDS[kl_estimator], 1 if apply_clamp else 0,
                                            _ptr(out), _stream(a.device)), "aa_kl_estimate")
        return out
