"""Drop-in functional API of the PPO/GRPO log-prob / entropy / actor-loss path.

Same names, argument meaning and error behaviour as the reference's
``areal.utils.functional`` (vocab_parallel.py:401-469, functional.py:185-559);
the arithmetic runs in hand-written gfx950 kernels reached through the C ABI of
``libareal_amd.so``.  PyTorch is used for device memory, streams and autograd
bookkeeping only.  Tensors must live on a ROCm device: there is no CPU path.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Any

import torch

from . import _native as N

__all__ = [
    "RejectionSamplingResult",
    "gather_logprobs",
    "gather_logprobs_entropy",
    "gather_logprobs_entropy_stats",
    "apply_rejection_sampling",
    "ppo_actor_loss_fn",
    "fused_logprobs_ppo_loss",
    "lm_head_logprobs_entropy",
    "lm_head_logprobs_entropy_stats",
]

_DTYPES = {torch.bfloat16: N.AA_BF16, torch.float16: N.AA_F16, torch.float32: N.AA_F32}


# ----------------------------------------------------------------------------
# helpers
# ----------------------------------------------------------------------------
def _ptr(t: torch.Tensor | None) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def _stream(device: torch.device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise N.NativeLibraryError(
            f"{name} is on {t.device}: areal_amd ops run on a ROCm GPU only (no CPU fallback)"
        )


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


def _mask_u8(mask: torch.Tensor) -> torch.Tensor:
    """One byte per token, non-zero = valid, without a copy for bool masks."""
    m = mask.contiguous()
    if m.dtype == torch.bool:
        return m.view(torch.uint8)
    return (m != 0).view(torch.uint8)


def _rows(logits: torch.Tensor) -> tuple[torch.Tensor, int, int, int]:
    """View logits as [T, V] rows with unit inner stride; returns (2-D tensor, T, V, row stride)."""
    V = logits.shape[-1]
    x = logits.reshape(-1, V)
    if x.dtype not in _DTYPES:
        x = x.float()
    if x.stride(-1) != 1 or (x.shape[0] > 1 and x.stride(0) < V):
        x = x.contiguous()
    T = x.shape[0]
    stride = x.stride(0) if T > 1 else V
    return x, T, V, stride


def _empty_rows_like(logits2d: torch.Tensor, stride: int) -> torch.Tensor:
    """An uninitialised [T, V] array for the gradient of ``logits2d``: the same row stride, and the same place inside
    a 16-byte piece of memory, so that the kernels walk both arrays alike (the fused kernel's fast path for rows that
    do not start on 16-byte boundaries asks for that)."""
    T, V = logits2d.shape
    lead = (logits2d.data_ptr() % 16) // logits2d.element_size()
    if stride == V and lead == 0:
        return torch.empty_like(logits2d, memory_format=torch.contiguous_format)
    flat = torch.empty(lead + (T - 1) * stride + V, dtype=logits2d.dtype, device=logits2d.device)
    return flat.as_strided((T, V), (stride, 1), lead)


def _check_tp(tp_group: Any) -> None:
    if tp_group is not None:
        import torch.distributed as dist

        if dist.get_world_size(tp_group) > 1:
            raise NotImplementedError(
                "vocab-parallel log-probs (tp_group with more than one rank) are not part of the "
                "single-GPU build; pass tp_group=None"
            )


_WORK: dict = {}


def _work_words(dev: torch.device) -> torch.Tensor:
    """Two zeroed int32 words per (device, stream) for the row hand-out of the fused kernel, which returns
    them to zero at the end of every launch."""
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    buf = _WORK.get(key)
    if buf is None:
        buf = _WORK[key] = torch.zeros(2, dtype=torch.int32, device=dev)
    return buf


def _ppo_params(eps_clip, eps_clip_higher, c_clip, has_w) -> N.PpoParams:
    if c_clip is not None:
        assert c_clip > 1.0, c_clip
    hi = eps_clip if eps_clip_higher is None else eps_clip_higher
    return N.PpoParams(
        clip_lo=1.0 - eps_clip,
        clip_hi=1.0 + hi,
        c_clip=0.0 if c_clip is None else float(c_clip),
        has_c_clip=0 if c_clip is None else 1,
        has_behave_weight=1 if has_w else 0,
    )


# ----------------------------------------------------------------------------
# log-probs / entropy
# ----------------------------------------------------------------------------
class _LogprobsEntropy(torch.autograd.Function):
    """logp, entropy, vocab max, vocab min of each row; differentiable in logits."""

    @staticmethod
    def forward(ctx, logits2d, labels1d, temperature, stride, want_entropy, want_minmax, inplace=False):
        lib = N.load()
        ctx.inplace = bool(inplace)
        T, V = logits2d.shape
        dev = logits2d.device
        kw = dict(dtype=torch.float32, device=dev)
        logp = torch.empty(T, **kw)
        entropy = torch.empty(T, **kw) if want_entropy else None
        need_bwd = ctx.needs_input_grad[0]
        row_lse = torch.empty(T, **kw) if need_bwd else None
        row_ez = torch.empty(T, **kw) if (need_bwd and want_entropy) else None
        vmax = torch.empty(T, **kw) if want_minmax else None
        vmin = torch.empty(T, **kw) if want_minmax else None
        with torch.cuda.device(dev):
            N.check(
                lib.aa_logits_fwd(
                    _ptr(logits2d), _DTYPES[logits2d.dtype], T, V, stride, _ptr(labels1d),
                    1.0 / float(temperature), _ptr(logp), _ptr(entropy), _ptr(row_lse), _ptr(row_ez),
                    _ptr(vmax), _ptr(vmin), _stream(dev),
                ),
                "aa_logits_fwd",
            )
        ctx.save_for_backward(logits2d, labels1d, row_lse, row_ez)
        ctx.temperature = float(temperature)
        ctx.stride = stride
        outs = (logp, entropy, vmax, vmin)
        ctx.mark_non_differentiable(*[o for o in (vmax, vmin) if o is not None])
        return outs

    @staticmethod
    def backward(ctx, g_logp, g_entropy, _g_vmax, _g_vmin):
        lib = N.load()
        logits2d, labels1d, row_lse, row_ez = ctx.saved_tensors
        T, V = logits2d.shape
        dev = logits2d.device
        if g_logp is None:
            g_logp = torch.zeros(T, dtype=torch.float32, device=dev)
        g_logp = _f32(g_logp)
        g_entropy = _f32(g_entropy) if (g_entropy is not None and row_ez is not None) else None
        if ctx.inplace:
            # the gradient takes the place of the logits (the kernel reads an element before it writes it); the version
            # bump below makes any other operation that kept the logits for its own backward fail loudly
            dlogits = logits2d.detach()
        else:  # the row stride of the input, so that both buffers are walked alike
            dlogits = _empty_rows_like(logits2d, ctx.stride)
        with torch.cuda.device(dev):
            N.check(
                lib.aa_logits_bwd(
                    _ptr(logits2d), _DTYPES[logits2d.dtype], T, V, ctx.stride, _ptr(labels1d),
                    1.0 / ctx.temperature, _ptr(row_lse), _ptr(row_ez), _ptr(g_logp), _ptr(g_entropy),
                    T, _ptr(dlogits), _stream(dev),
                ),
                "aa_logits_bwd",
            )
        if ctx.inplace:
            torch.autograd.graph.increment_version(logits2d)
        return dlogits, None, None, None, None, None, None


def _device_or_read_back_counts(T: int, T_active: int, mask_u8: torch.Tensor, on_device: bool) -> list[int]:
    """``kept_per_chunk`` of the lm_head step when the caller gave none: left to the device (the kernels stop at the
    rows in use, nothing is read back), or read back from the device (exact counts: one small copy that waits for the
    mask)."""
    chunk = int(N.load().aa_lmhead_chunk_tokens())
    n_chunks = (T + chunk - 1) // chunk
    if on_device:
        return [N.AA_LMHEAD_COUNT_ON_DEVICE] * n_chunks
    on = mask_u8.ne(0)
    if n_chunks * chunk != T_active:
        on = torch.nn.functional.pad(on, (0, n_chunks * chunk - T_active))
    return _HostCounts(on.view(n_chunks, chunk).sum(1)).tolist()


def _logprobs_impl(logits, labels, temperature, tp_group, want_entropy, want_minmax, inplace_backward=False):
    _check_tp(tp_group)
    _require_gpu(logits, "logits")
    assert logits.shape[0] > 0, "Input logits must have at least one element"
    if tuple(labels.shape) != tuple(logits.shape[:-1]):
        raise ValueError(f"labels shape {tuple(labels.shape)} != logits shape[:-1] {tuple(logits.shape[:-1])}")
    x, T, V, stride = _rows(logits)
    y = labels.reshape(-1).to(device=x.device, dtype=torch.int64).contiguous()
    logp, entropy, vmax, vmin = _LogprobsEntropy.apply(x, y, float(temperature), stride, want_entropy, want_minmax,
                                                       bool(inplace_backward))
    shp = labels.shape
    return (
        logp.view(shp),
        entropy.view(shp) if entropy is not None else None,
        vmax.view(shp) if vmax is not None else None,
        vmin.view(shp) if vmin is not None else None,
    )


def gather_logprobs(
    logits: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    tp_group: Any | None = None,
    chunk_size: int = 1024,
    inplace_backward: bool = False,
) -> torch.Tensor:
    """``log_softmax(logits.float() / temperature)[..., labels]`` as fp32, shaped like ``labels``.

    Same contract as vocab_parallel.py:401-431.  ``chunk_size`` is accepted and
    ignored: the kernel never materialises an fp32 copy of the logits, and the
    result does not depend on chunking.  ``inplace_backward=True`` (not in the
    reference): the backward pass writes the gradient over the logits instead
    of allocating a second ``[T, V]`` array; for callers that need the logits
    for nothing else after this op.
    """
    del chunk_size
    return _logprobs_impl(logits, labels, temperature, tp_group, False, False, inplace_backward)[0]


def gather_logprobs_entropy(
    logits: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    tp_group: Any | None = None,
    chunk_size: int = 1024,
    inplace_backward: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """(log-probs at ``labels``, entropy of each row); vocab_parallel.py:434-469.  ``inplace_backward`` as in
    ``gather_logprobs``."""
    del chunk_size
    logp, entropy, _, _ = _logprobs_impl(logits, labels, temperature, tp_group, True, False, inplace_backward)
    return logp, entropy


def gather_logprobs_entropy_stats(
    logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0, inplace_backward: bool = False
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(logp, entropy, vocab_min_logits, vocab_max_logits) from the same single pass.

    The last two are what FSDPEngine._get_vocab_min_max_logits
    (fsdp_engine.py:1893-1906) computes with two more passes over the logits.
    """
    logp, entropy, vmax, vmin = _logprobs_impl(logits, labels, temperature, None, True, True, inplace_backward)
    return logp, entropy, vmin, vmax


# ----------------------------------------------------------------------------
# rejection sampling
# ----------------------------------------------------------------------------
@dataclass
class RejectionSamplingResult:
    """functional.py:152-164"""

    loss_mask: torch.Tensor
    behave_imp_weight: torch.Tensor
    filtered_fraction: float


def _segments(shape, cu_seqlens, what: str):
    """(cu_seqlens int32 tensor or None, number of segments) for a 1-D packed or 2-D padded layout."""
    if len(shape) == 1:
        if cu_seqlens is None:
            raise ValueError(what)
        cu = cu_seqlens.to(dtype=torch.int32).contiguous()
        return cu, cu.shape[0] - 1
    return None, shape[0]


def _rejection_sampling_device(prox, old, mask_u8, shape, cu_seqlens, cfg):
    """Runs the kernel; returns (mask_out u8 [n], weight f32 [n], counts i32 [3]) without syncing."""
    lib = N.load()
    dev = prox.device
    n = prox.numel()
    cu, B = (None, 0)
    if cfg.level == "sequence":
        cu, B = _segments(
            shape, cu_seqlens, "cu_seqlens is required for 1D packed tensors in sequence-level filtering."
        )
        if cu is not None:
            cu = cu.to(dev)
    mask_out = torch.empty(n, dtype=torch.uint8, device=dev)
    w = torch.empty(n, dtype=torch.float32, device=dev)
    counts = torch.empty(3, dtype=torch.int32, device=dev)
    lower = cfg.lower
    with torch.cuda.device(dev):
        N.check(
            lib.aa_rejection_sampling(
                _ptr(prox), _ptr(old), _ptr(mask_u8), n, _ptr(cu), B,
                N.RS_LEVEL[cfg.level], N.RS_ACTION[cfg.action], N.RS_METRIC[cfg.metric], N.RS_AGG[cfg.agg],
                float(cfg.upper), 0.0 if lower is None else float(lower), 0 if lower is None else 1,
                _ptr(mask_out), _ptr(w), _ptr(counts), _stream(dev),
            ),
            "aa_rejection_sampling",
        )
    return mask_out, w, counts


class _HostCounts:
    """The counters of the rejection-sampling kernel on their way to the host.

    The copy into pinned memory is queued right behind the kernel and gets an event of its own, so reading the
    counters later (``filtered_fraction`` is a Python float, as in the reference) waits for that copy only and not
    for the long kernels queued after it: the host keeps running ahead of the GPU.  The wait polls the event: a
    blocking wait took 0.2 ms to wake up here, which a step of a few thousand tokens cannot hide.  After a bounded
    number of polls (some tens of milliseconds) it blocks after all."""

    _POLLS = 20000

    def __init__(self, counts: torch.Tensor):
        self._host = torch.empty(counts.shape, dtype=counts.dtype, pin_memory=True)
        with torch.cuda.device(counts.device):
            self._host.copy_(counts, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record()

    def tolist(self):
        event = self._event
        for _ in range(self._POLLS):
            if event.query():
                break
        else:
            event.synchronize()
        return self._host.tolist()


def _validate_rs(cfg) -> None:
    for field, table in (("level", N.RS_LEVEL), ("action", N.RS_ACTION), ("agg", N.RS_AGG)):
        if getattr(cfg, field) not in table:
            raise ValueError(f"Unknown {field}: {getattr(cfg, field)}")
    if cfg.metric not in N.RS_METRIC:
        raise ValueError(f"Unknown metric: {cfg.metric}")


def apply_rejection_sampling(
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    loss_mask: torch.Tensor,
    cu_seqlens: torch.Tensor | None,
    config: Any,
) -> RejectionSamplingResult:
    """Filter or clamp tokens / sequences by the divergence between the proximal
    and the behaviour policy; functional.py:185-426.

    ``config`` is any object with the attributes of ``RejectionSamplingConfig``.
    """
    if proximal_logprobs.shape != old_logprobs.shape:
        raise ValueError(
            f"proximal_logprobs shape {proximal_logprobs.shape} != old_logprobs shape {old_logprobs.shape}"
        )
    if proximal_logprobs.shape != loss_mask.shape:
        raise ValueError(
            f"proximal_logprobs shape {proximal_logprobs.shape} != loss_mask shape {loss_mask.shape}"
        )
    if proximal_logprobs.ndim not in (1, 2):
        raise ValueError(f"Expected 1D (packed) or 2D (padded) tensors, got ndim={proximal_logprobs.ndim}")
    _validate_rs(config)
    _require_gpu(proximal_logprobs, "proximal_logprobs")
    shape = proximal_logprobs.shape
    prox = _f32(proximal_logprobs.detach()).reshape(-1)
    old = _f32(old_logprobs.detach()).reshape(-1)
    m8 = _mask_u8(loss_mask).reshape(-1)
    mask_out, w, counts = _rejection_sampling_device(prox, old, m8, shape, cu_seqlens, config)
    total, hit, _ = counts.tolist()  # the reference returns a Python float here too
    if config.action == "mask":
        new_mask = mask_out.view(shape).to(loss_mask.dtype)
    else:
        new_mask = loss_mask
    return RejectionSamplingResult(
        loss_mask=new_mask,
        behave_imp_weight=w.view(shape),
        filtered_fraction=hit / max(total, 1),
    )


# ----------------------------------------------------------------------------
# PPO actor loss on log-probs
# ----------------------------------------------------------------------------
class _PpoLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logp, prox, adv, mask_eff, behave_w, cu, B, seq_level, params, n_valid):
        ctx.set_materialize_grads(False)  # no zero-filled gradients for the outputs that have none
        lib = N.load()
        dev = logp.device
        n = logp.numel()
        stat_loss = torch.empty(n, dtype=torch.float32, device=dev)
        ratio = torch.empty(n, dtype=torch.float32, device=dev)
        flags = torch.empty(n, dtype=torch.uint8, device=dev)
        g_logp = torch.empty(n, dtype=torch.float32, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(
                lib.aa_ppo_loss(
                    _ptr(logp), _ptr(prox), _ptr(adv), _ptr(mask_eff), _ptr(behave_w), n, _ptr(cu), B,
                    1 if seq_level else 0, C.byref(params), _ptr(n_valid), _ptr(stat_loss), _ptr(ratio),
                    _ptr(flags), _ptr(g_logp), st,
                ),
                "aa_ppo_loss",
            )
            N.check(
                lib.aa_masked_sum(_ptr(stat_loss), _ptr(mask_eff), n, _ptr(n_valid), None, _ptr(loss), st),
                "aa_masked_sum",
            )
        ctx.save_for_backward(g_logp)
        ctx.mark_non_differentiable(stat_loss, ratio, flags)
        return loss, stat_loss, ratio, flags

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        if g_loss is None:  # the loss was not used (gradients are not materialised, see forward)
            return (None,) * 10
        (g_logp,) = ctx.saved_tensors
        return (g_logp * g_loss,) + (None,) * 9


def _flag_bits(flags: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """(clip_mask, dual_clip_mask) as bool tensors from the kernels' flag bytes (bit 0, bit 1): one launch each, the
    0 / 1 bytes reinterpreted as bool."""
    return torch.bitwise_and(flags, 1).view(torch.bool), torch.bitwise_right_shift(flags, 1).view(torch.bool)


def _count_nonzero(mask_u8: torch.Tensor) -> torch.Tensor:
    lib = N.load()
    dev = mask_u8.device
    out = torch.empty(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        N.check(lib.aa_count_nonzero_u8(_ptr(mask_u8), mask_u8.numel(), _ptr(out), _stream(dev)), "aa_count_nonzero_u8")
    return out


def _stat_outputs(logp, prox, old, flags, w, mask_eff_u8):
    """The derived entries of the stat dict (functional.py:505-558) in one launch: ``approx_kl``, ``clip_mask``,
    ``dual_clip_mask`` and, with rejection sampling (``w`` given), ``behave_mask`` and ``behave_approx_kl``
    (None otherwise)."""
    lib = N.load()
    dev = logp.device
    n = logp.numel()
    logp = logp.detach()
    logp = logp if logp.is_contiguous() else logp.contiguous()
    approx_kl = torch.empty(n, dtype=torch.float32, device=dev)
    clip = torch.empty(n, dtype=torch.uint8, device=dev)
    dual = torch.empty(n, dtype=torch.uint8, device=dev)
    behave_mask = behave_kl = None
    if w is not None:
        behave_mask = torch.empty(n, dtype=torch.uint8, device=dev)
        behave_kl = torch.empty(n, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        N.check(
            lib.aa_ppo_stat_outputs(_ptr(logp), _ptr(prox), _ptr(old), _ptr(flags), _ptr(w), _ptr(mask_eff_u8), n,
                                    _ptr(approx_kl), _ptr(clip), _ptr(dual), _ptr(behave_mask), _ptr(behave_kl),
                                    _stream(dev)),
            "aa_ppo_stat_outputs",
        )
    as_bool = lambda t: None if t is None else t.view(torch.bool)
    return approx_kl, as_bool(clip), as_bool(dual), as_bool(behave_mask), behave_kl


def _rs_stats(stat, behave_mask, behave_kl, w, counts, shape):
    total, hit, _ = counts.tolist()
    stat.update(
        behave_approx_kl=behave_kl.view(shape),
        behave_imp_weight=w.view(shape),
        behave_mask=behave_mask.view(shape),
        filtered_fraction=hit / max(total, 1),
    )


def ppo_actor_loss_fn(
    logprobs: torch.Tensor,
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip: float,
    loss_mask: torch.Tensor,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling: Any | None = None,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
) -> tuple[torch.Tensor, dict]:
    """Decoupled-proximal clipped PPO actor loss; functional.py:429-559.

    Returns ``(loss, stat)`` with the reference's stat keys: ``loss``,
    ``importance_weight``, ``approx_kl``, ``clip_mask``, ``dual_clip_mask`` and,
    with rejection sampling, ``behave_approx_kl``, ``behave_imp_weight``,
    ``behave_mask``, ``filtered_fraction``.  The loss is differentiable in
    ``logprobs`` (closed-form gradient computed with the forward).
    """
    if importance_sampling_level not in ("token", "sequence"):
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. Must be 'token' or 'sequence'."
        )
    _require_gpu(logprobs, "logprobs")
    shape = logprobs.shape
    seq_level = importance_sampling_level == "sequence"
    cu, B = None, 0
    if seq_level:
        cu, B = _segments(
            shape,
            cu_seqlens,
            "cu_seqlens is required for 1D tensors (packed format). For a single sequence, use "
            "cu_seqlens=torch.tensor([0, seq_len], dtype=torch.int32).",
        )
        if cu is not None:
            cu = cu.to(logprobs.device)
    params = _ppo_params(eps_clip, eps_clip_higher, c_clip, rejection_sampling is not None)

    lp = _f32(logprobs).reshape(-1)
    prox = _f32(proximal_logprobs.detach()).reshape(-1)
    old = _f32(old_logprobs.detach()).reshape(-1)
    adv = _f32(advantages.detach()).reshape(-1)
    m8 = _mask_u8(loss_mask).reshape(-1)

    w = counts = None
    mask_eff = m8
    if rejection_sampling is not None:
        _validate_rs(rejection_sampling)
        mask_eff, w, counts = _rejection_sampling_device(prox, old, m8, shape, cu_seqlens, rejection_sampling)
        host_counts = _HostCounts(counts)
        if rejection_sampling.action != "mask":
            mask_eff = m8
        n_valid = counts  # counts[0] is the non-zero count of the original mask
    else:
        n_valid = _count_nonzero(m8)

    loss, stat_loss, ratio, flags = _PpoLoss.apply(lp, prox, adv, mask_eff, w, cu, B, seq_level, params, n_valid)
    approx_kl, clip, dual, behave_mask, behave_kl = _stat_outputs(lp, prox, old, flags, w, mask_eff)
    stat = dict(
        loss=stat_loss.view(shape),
        importance_weight=ratio.view(shape),
        approx_kl=approx_kl.view(shape),
        clip_mask=clip.view(shape),
        dual_clip_mask=dual.view(shape),
    )
    if rejection_sampling is not None:
        _rs_stats(stat, behave_mask, behave_kl, w, host_counts, shape)
    return loss, stat


# ----------------------------------------------------------------------------
# fused: logits -> logp/entropy -> token-level PPO loss -> d(logits), one pass
# ----------------------------------------------------------------------------
def _hand_out_once(ctx) -> None:
    """The fused steps keep their gradients in the buffers the forward pass wrote and scale them in place by the
    upstream factor, so those buffers can be handed out once: a second backward through a retained graph would scale
    them again."""
    if getattr(ctx, "handed_out", False):
        raise RuntimeError("the gradient of this fused step was already handed out; run the forward pass again "
                           "instead of a second backward through a retained graph")
    ctx.handed_out = True


def _finish_fused_loss(lib, params, stat_loss, logp, mask_eff, T_active, n_valid, grad_scale, loss, st) -> None:
    """The scalar the fused kernels' per-token losses add up to: the clipped surrogate over ``max(n, 1)``, or the
    negative log-likelihood over ``n + 1e-5`` (areal/trainer/sft/lm_engine.py:96)."""
    if params.loss_kind == 1:
        scratch = torch.empty(1, dtype=torch.float64, device=logp.device)
        cnt = torch.empty(1, dtype=torch.int32, device=logp.device)
        N.check(lib.aa_sft_loss(_ptr(logp), _ptr(mask_eff), T_active, None, 0, _ptr(n_valid), _ptr(grad_scale),
                                _ptr(loss), None, None, _ptr(scratch), _ptr(cnt), None, st), "aa_sft_loss")
    else:
        N.check(lib.aa_masked_sum(_ptr(stat_loss), _ptr(mask_eff), T_active, _ptr(n_valid), _ptr(grad_scale),
                                  _ptr(loss), st), "aa_masked_sum")


class _FusedLogitsPpo(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits2d, labels1d, stride, temperature, T_active, prox, adv, mask_eff, behave_w, params,
                n_valid, grad_scale, want_minmax, inplace=False):
        ctx.set_materialize_grads(False)  # no zero-filled gradients for the outputs that have none
        lib = N.load()
        T, V = logits2d.shape
        dev = logits2d.device
        f32 = dict(dtype=torch.float32, device=dev)
        logp = torch.empty(T, **f32)
        entropy = torch.empty(T, **f32)
        vmax = torch.empty(T, **f32) if want_minmax else None
        vmin = torch.empty(T, **f32) if want_minmax else None
        stat_loss = torch.empty(T_active, **f32)
        ratio = torch.empty(T_active, **f32)
        flags = torch.empty(T_active, dtype=torch.uint8, device=dev)
        loss = torch.empty((), **f32)
        if inplace:
            # the gradient takes the place of the logits: every kernel reads an element for the last time before it
            # writes it, so the two arrays of the C entry point may be one
            dlogits = logits2d.detach()
        else:
            dlogits = _empty_rows_like(logits2d, stride)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(
                lib.aa_logits_ppo_fused(
                    _ptr(logits2d), _DTYPES[logits2d.dtype], T, V, stride, _ptr(labels1d), 1.0 / float(temperature),
                    T_active, _ptr(prox), _ptr(adv), _ptr(mask_eff), _ptr(behave_w), C.byref(params),
                    _ptr(n_valid), _ptr(grad_scale), _ptr(logp), _ptr(entropy), _ptr(vmax), _ptr(vmin),
                    _ptr(stat_loss), _ptr(ratio), _ptr(flags), _ptr(dlogits), _ptr(_work_words(dev)), st,
                ),
                "aa_logits_ppo_fused",
            )
            _finish_fused_loss(lib, params, stat_loss, logp, mask_eff, T_active, n_valid, grad_scale, loss, st)
        if inplace:
            # written through a raw pointer: tell autograd, so that an operation that saved the logits for its own
            # backward fails loudly instead of reading gradients
            torch.autograd.graph.increment_version(logits2d)
        ctx.save_for_backward(dlogits)
        others = [logp, entropy, stat_loss, ratio, flags] + [t for t in (vmax, vmin) if t is not None]
        ctx.mark_non_differentiable(*others)
        return loss, logp, entropy, vmax, vmin, stat_loss, ratio, flags

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        if g_loss is None:
            return (None,) * 14
        _hand_out_once(ctx)
        lib = N.load()
        (dlogits,) = ctx.saved_tensors
        dev = dlogits.device
        g = _f32(g_loss).reshape(1)
        # d(logits) was written with the loss; an upstream factor other than 1 is
        # applied in place (the kernel returns at once when the factor is 1).
        T, V = dlogits.shape
        with torch.cuda.device(dev):
            N.check(
                lib.aa_scale_rows_inplace(_ptr(dlogits), _DTYPES[dlogits.dtype], T, V, dlogits.stride(0) if T > 1 else V,
                                          _ptr(g), _stream(dev)),
                "aa_scale_rows_inplace",
            )
        return (dlogits,) + (None,) * 13


def fused_logprobs_ppo_loss(
    logits: torch.Tensor,
    labels: torch.Tensor,
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip: float,
    loss_mask: torch.Tensor,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling: Any | None = None,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
    temperature: float = 1.0,
    loss_scale: torch.Tensor | float | None = None,
    inplace_backward: bool = False,
) -> tuple[torch.Tensor, dict]:
    """``gather_logprobs_entropy`` + ``ppo_actor_loss_fn`` (+ backward) in one pass over the logits.

    ``logits`` is ``[T_pad, V]`` and ``labels`` ``[T_pad]`` (the batch-padded
    micro-batch, fsdp_engine.py:1908-1936); the per-token tensors are the
    un-padded ``[T]`` ones with ``T <= T_pad``: rows past ``T`` are the padding
    the engine trims after the log-prob op (fsdp_engine.py:2027-2031) and get a
    zero gradient.  ``loss_scale`` is the factor the engine multiplies the loss
    with (fsdp_engine.py:2045); the returned loss already includes it, and
    ``loss.backward()`` hands back a gradient that was written during the
    forward pass.

    The stat dict has the keys of ``ppo_actor_loss_fn`` plus ``logprobs``,
    ``entropy``, ``vocab_min_logits`` and ``vocab_max_logits`` (all ``[T]``).
    With ``importance_sampling_level="sequence"`` the loss of a token depends on
    its whole sequence, so the call runs the unfused kernels instead.

    ``inplace_backward=True`` (no counterpart in the reference, whose autograd
    allocates the gradient) writes the gradient over the logits instead of into
    a second ``[T_pad, V]`` array: half the memory of the step (37 GB instead of
    74 GB at 122 k tokens of a 152 k vocabulary) and the same bits.  After the
    call ``logits`` holds its own gradient (for an upstream factor of 1), so it
    is for callers that need the logits for nothing else; an operation that
    saved them for its backward raises autograd's modified-in-place error.
    On the sequence-level path the gradient lands there during
    ``loss.backward()``.  Ignored where no gradient is produced.

    fp32 logits of more than 114 688 entries per row (``V % 8 == 0``) are kept
    on the chip in 24 bits per value between their one read and the write of
    the gradient: log-probs, entropy and the extrema come from the fp32 values,
    the entries of the gradient row are within ``|x| / temperature * 2**-16``
    (relative) of the fp32 ones.
    """
    if importance_sampling_level not in ("token", "sequence"):
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. Must be 'token' or 'sequence'."
        )
    _require_gpu(logits, "logits")
    if logits.ndim != 2 or labels.ndim != 1 or labels.shape[0] != logits.shape[0]:
        raise ValueError(f"expected logits [T, V] and labels [T], got {tuple(logits.shape)} and {tuple(labels.shape)}")
    assert logits.shape[0] > 0, "Input logits must have at least one element"
    T_active = loss_mask.shape[0]
    if loss_mask.ndim != 1 or T_active > logits.shape[0]:
        raise ValueError(f"loss_mask shape {tuple(loss_mask.shape)} does not fit logits {tuple(logits.shape)}")
    for name, t in (("proximal_logprobs", proximal_logprobs), ("old_logprobs", old_logprobs), ("advantages", advantages)):
        if t.shape != loss_mask.shape:
            raise ValueError(f"{name} shape {tuple(t.shape)} != loss_mask shape {tuple(loss_mask.shape)}")
    dev = logits.device
    scale_t = None
    if loss_scale is not None:
        scale_t = torch.as_tensor(loss_scale, dtype=torch.float32, device=dev).reshape(1)

    # Without a gradient to produce (evaluation, torch.no_grad) the step is the forward kernel (one read of the logits,
    # no [T, V] gradient buffer) followed by the loss on log-probs.
    forward_only = not (torch.is_grad_enabled() and logits.requires_grad)
    if importance_sampling_level == "sequence" or forward_only:
        logp, entropy, vmin, vmax = gather_logprobs_entropy_stats(logits, labels, temperature,
                                                                  inplace_backward and not forward_only)
        logp, entropy, vmin, vmax = (t[:T_active] for t in (logp, entropy, vmin, vmax))
        loss, stat = ppo_actor_loss_fn(
            logp, proximal_logprobs, old_logprobs, advantages, eps_clip, loss_mask, eps_clip_higher, c_clip,
            rejection_sampling, importance_sampling_level, cu_seqlens,
        )
        if scale_t is not None:
            loss = loss * scale_t.squeeze(0)
        stat.update(logprobs=logp.detach(), entropy=entropy.detach(), vocab_min_logits=vmin, vocab_max_logits=vmax)
        return loss, stat

    x, T, V, stride = _rows(logits)
    y = labels.to(device=dev, dtype=torch.int64).contiguous()
    prox = _f32(proximal_logprobs.detach())
    old = _f32(old_logprobs.detach())
    adv = _f32(advantages.detach())
    m8 = _mask_u8(loss_mask)
    params = _ppo_params(eps_clip, eps_clip_higher, c_clip, rejection_sampling is not None)
    w = counts = None
    mask_eff = m8
    if rejection_sampling is not None:
        _validate_rs(rejection_sampling)
        mask_eff, w, counts = _rejection_sampling_device(prox, old, m8, loss_mask.shape, cu_seqlens, rejection_sampling)
        host_counts = _HostCounts(counts)
        if rejection_sampling.action != "mask":
            mask_eff = m8
        n_valid = counts
    else:
        n_valid = _count_nonzero(m8)
    loss, logp, entropy, vmax, vmin, stat_loss, ratio, flags = _FusedLogitsPpo.apply(
        x, y, stride, float(temperature), T_active, prox, adv, mask_eff, w, params, n_valid, scale_t, True,
        bool(inplace_backward),
    )
    logp_a = logp[:T_active]
    approx_kl, clip, dual, behave_mask, behave_kl = _stat_outputs(logp_a, prox, old, flags, w, mask_eff)
    stat = dict(
        loss=stat_loss,
        importance_weight=ratio,
        approx_kl=approx_kl,
        clip_mask=clip,
        dual_clip_mask=dual,
        logprobs=logp_a,
        entropy=entropy[:T_active],
        vocab_min_logits=vmin[:T_active],
        vocab_max_logits=vmax[:T_active],
    )
    if rejection_sampling is not None:
        _rs_stats(stat, behave_mask, behave_kl, w, host_counts, loss_mask.shape)
    return loss, stat


# ----------------------------------------------------------------------------
# fused lm_head: hidden @ weight.T -> logp / entropy without the [T, V] logits
# ----------------------------------------------------------------------------
_LMHEAD_BACKWARD = {"recompute": 0, "carry": 1}  # aa_lmhead_backward_mode


def lm_head_chunk_tokens() -> int:
    """Tokens per chunk of the lm_head entry points (what ``kept_per_chunk`` counts over)."""
    return int(N.load().aa_lmhead_chunk_tokens())


def _lmhead_workspace(T: int, H: int, V: int, dev, forward_only: bool = False, extrema: bool = False) -> torch.Tensor:
    lib = N.load()
    if forward_only:
        n = lib.aa_lmhead_fwd_stats_workspace_bytes(T, H, V) if extrema else lib.aa_lmhead_fwd_workspace_bytes(T, H, V)
    else:
        n = lib.aa_lmhead_workspace_bytes(T, H, V)
    if n < 0:
        raise N.NativeLibraryError(
            f"the lm_head path needs a hidden size that is a multiple of 8, and sizes below 2^22 (got H={H}, V={V})"
        )
    return torch.empty(n, dtype=torch.uint8, device=dev)


class _LmHeadLogprobsEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature, want_minmax=False):
        ctx.set_materialize_grads(False)
        lib = N.load()
        T, H = hidden.shape
        V = weight.shape[0]
        dev = hidden.device
        f32 = dict(dtype=torch.float32, device=dev)
        logp, entropy, row_lse, row_ez = (torch.empty(T, **f32) for _ in range(4))
        vmax = torch.empty(T, **f32) if want_minmax else None
        vmin = torch.empty(T, **f32) if want_minmax else None
        ws = _lmhead_workspace(T, H, V, dev, forward_only=True, extrema=want_minmax)  # partials only: nothing of size T x V
        with torch.cuda.device(dev):
            N.check(
                lib.aa_lmhead_fwd(
                    _ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), 1.0 / float(temperature), _ptr(logp),
                    _ptr(entropy), _ptr(row_lse), _ptr(row_ez), _ptr(vmax), _ptr(vmin), _ptr(ws), ws.numel(),
                    _stream(dev),
                ),
                "aa_lmhead_fwd",
            )
        ctx.save_for_backward(hidden, weight, labels, row_lse, row_ez)
        ctx.temperature = float(temperature)
        if want_minmax:
            ctx.mark_non_differentiable(vmax, vmin)
        return logp, entropy, vmax, vmin

    @staticmethod
    def backward(ctx, g_logp, g_entropy, _g_vmax=None, _g_vmin=None):
        if g_logp is None and g_entropy is None:
            return None, None, None, None, None
        hidden, weight, labels, row_lse, row_ez = ctx.saved_tensors
        d_hidden, d_weight = _lmhead_recompute_backward(hidden, weight, labels, ctx.temperature, row_lse, row_ez,
                                                        g_logp, g_entropy)
        return d_hidden, d_weight, None, None, None


def _lmhead_recompute_backward(hidden, weight, labels, temperature, row_lse, row_ez, g_logp, g_entropy):
    """``aa_lmhead_bwd``: the logits tiles of the tokens with a gradient are formed again."""
    lib = N.load()
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    g_logp = torch.zeros(T, dtype=torch.float32, device=dev) if g_logp is None else _f32(g_logp)
    g_entropy = None if g_entropy is None else _f32(g_entropy)
    d_hidden = torch.empty_like(hidden)
    d_weight = torch.empty_like(weight)  # bf16: rounded once, after fp32 accumulation over the chunks
    ws = _lmhead_workspace(T, H, V, dev)
    # Rows whose upstream gradients are all zero (masked tokens) are left out of the gradient GEMMs; the device counts
    # them itself (no read-back: the host does not wait for the gradient to exist).
    has_grad = g_logp != 0 if g_entropy is None else (g_logp != 0) | (g_entropy != 0)
    chunk = int(lib.aa_lmhead_chunk_tokens())
    n_chunks = (T + chunk - 1) // chunk
    kept = (C.c_int64 * n_chunks)(*([N.AA_LMHEAD_COUNT_ON_DEVICE] * n_chunks))
    with torch.cuda.device(dev):
        N.check(
            lib.aa_lmhead_bwd(
                _ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), 1.0 / temperature, _ptr(row_lse),
                _ptr(row_ez), _ptr(g_logp), _ptr(g_entropy), _ptr(has_grad.view(torch.uint8)), kept,
                _ptr(d_hidden), _ptr(d_weight), _DTYPES[d_weight.dtype], _ptr(ws), ws.numel(), _stream(dev),
            ),
            "aa_lmhead_bwd",
        )
    return d_hidden, d_weight


class _LmHeadCarry(torch.autograd.Function):
    """The lm_head op whose forward also keeps ``p_v / p_label`` of the tokens that may get a gradient (bf16 rows, in a
    tensor that lives until the backward), so that the backward is two plain GEMMs (``aa_lmhead_fwd_carry`` /
    ``aa_lmhead_bwd_carry``)."""

    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature, grad_mask, kept_per_chunk, want_minmax):
        ctx.set_materialize_grads(False)
        lib = N.load()
        T, H = hidden.shape
        V = weight.shape[0]
        dev = hidden.device
        f32 = dict(dtype=torch.float32, device=dev)
        logp, entropy, row_lse, row_ez = (torch.empty(T, **f32) for _ in range(4))
        vmax = torch.empty(T, **f32) if want_minmax else None
        vmin = torch.empty(T, **f32) if want_minmax else None
        kept = None if kept_per_chunk is None else (C.c_int64 * len(kept_per_chunk))(*kept_per_chunk)
        if kept_per_chunk is None:
            rows = T
        else:  # a chunk whose count stays on the device keeps room for every one of its tokens
            chunk = lm_head_chunk_tokens()
            rows = sum(min(chunk, T - i * chunk) if k == N.AA_LMHEAD_COUNT_ON_DEVICE else k
                       for i, k in enumerate(kept_per_chunk))
        panel = torch.empty(max(rows, 1), int(lib.aa_lmhead_panel_pitch(V)), dtype=torch.bfloat16, device=dev)
        n = lib.aa_lmhead_carry_workspace_bytes(T, H, V)
        if n < 0:
            raise N.NativeLibraryError(
                f"the lm_head path needs a hidden size that is a multiple of 8, and sizes below 2^22 (got H={H}, V={V})")
        ws = torch.empty(n, dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            N.check(
                lib.aa_lmhead_fwd_carry(
                    _ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), 1.0 / float(temperature), _ptr(grad_mask), kept,
                    _ptr(logp), _ptr(entropy), _ptr(row_lse), _ptr(row_ez), _ptr(vmax), _ptr(vmin), _ptr(panel),
                    panel.shape[0], _ptr(ws), ws.numel(), _stream(dev),
                ),
                "aa_lmhead_fwd_carry",
            )
        ctx.save_for_backward(hidden, weight, labels, logp, row_lse, row_ez, panel, grad_mask)
        ctx.temperature = float(temperature)
        ctx.kept_per_chunk = kept_per_chunk
        if want_minmax:
            ctx.mark_non_differentiable(vmax, vmin)
        return logp, entropy, vmax, vmin

    @staticmethod
    def backward(ctx, g_logp, g_entropy, _g_vmax=None, _g_vmin=None):
        if g_logp is None and g_entropy is None:
            return (None,) * 7
        hidden, weight, labels, logp, row_lse, row_ez, panel, grad_mask = ctx.saved_tensors
        if g_entropy is not None:  # an entropy gradient is no multiple of the stored rows: form the logits again
            d_hidden, d_weight = _lmhead_recompute_backward(hidden, weight, labels, ctx.temperature, row_lse, row_ez,
                                                            g_logp, g_entropy)
            return (d_hidden, d_weight) + (None,) * 5
        # the backward patches the stored rows (and may overwrite a chunk of them): they serve one backward
        if getattr(ctx, "handed_out", False):
            raise RuntimeError("the stored rows of this lm_head forward were already used by a backward; run the forward "
                               "pass again instead of a second backward through a retained graph")
        ctx.handed_out = True
        lib = N.load()
        T, H = hidden.shape
        V = weight.shape[0]
        dev = hidden.device
        g_logp = _f32(g_logp)
        kept_per_chunk = ctx.kept_per_chunk
        kept = None if kept_per_chunk is None else (C.c_int64 * len(kept_per_chunk))(*kept_per_chunk)
        d_hidden = torch.empty_like(hidden)
        d_weight = torch.empty_like(weight)
        ws = torch.empty(lib.aa_lmhead_carry_workspace_bytes(T, H, V), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            N.check(
                lib.aa_lmhead_bwd_carry(
                    _ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), 1.0 / ctx.temperature, _ptr(logp), _ptr(row_lse),
                    _ptr(g_logp), _ptr(grad_mask), kept, _ptr(panel), panel.shape[0], _ptr(d_hidden), _ptr(d_weight),
                    _DTYPES[d_weight.dtype], _ptr(ws), ws.numel(), _stream(dev),
                ),
                "aa_lmhead_bwd_carry",
            )
        return (d_hidden, d_weight) + (None,) * 5


def lm_head_logprobs_entropy(
    hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0,
    token_mask: torch.Tensor | None = None, backward: str = "recompute", grad_token_mask: torch.Tensor | None = None,
    kept_per_chunk: list[int] | None = None, count_on_device: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``gather_logprobs_entropy(hidden @ weight.T, labels, temperature)`` without writing the ``[T, V]`` logits.
    Any vocabulary size; the hidden size has to be a multiple of 8.

    ``hidden`` is ``[T, H]`` and ``weight`` ``[V, H]`` (the lm_head), both bf16.  The forward forms 256 x 256 tiles of
    the logits in the accumulator registers of the library's bf16 MFMA tile GEMM (fp32 accumulation, not rounded to
    bf16 in between) and reduces each tile to softmax partials per token in the GEMM's epilogue; its only scratch
    memory is those partials (about ``24 * V / 256`` bytes per token of a chunk of at most 16384 tokens, 0.23 GB at
    ``V = 151936``).  Differentiable in ``hidden`` and ``weight``: the backward goes through the tokens in chunks of at
    most 16384, forms the chunk's logits tiles again, writes their gradient as bf16 rows (of the tokens whose upstream
    gradient is not zero) into a workspace panel ``[chunk, V]`` and contracts that panel with the weight and with the
    hidden states on the same tile GEMM (fp32 accumulation, the weight gradient is returned in the dtype of
    ``weight``).  The backward's workspace is that panel (``2 * chunk * V`` bytes), the hidden rows of the chunk's
    tokens with a gradient and a few fp32 planes of ``[chunk, H]``; the arrays are multiplied as they lie, nothing is
    transposed.
    The reference has no such op: it is the drop-in for its lm_head matmul followed by
    ``gather_logprobs_entropy`` (vocab_parallel.py:434-469).

    ``token_mask`` (``[T]``, optional, beyond the reference's semantics): only tokens whose entry is non-zero go
    through the lm_head; the others get log-prob 0 and entropy 0 (e.g. the forward-only ``compute_logp`` pass, whose
    results are multiplied by the loss mask anyway).

    ``backward="carry"`` (default ``"recompute"``): the forward also keeps ``p_v / p_label`` of the tokens that may get
    a gradient as bf16 rows until the backward, which is then two plain GEMMs instead of three (no second logits GEMM:
    about a fifth less time for forward + backward at the 8B shape).  For losses that need every log-prob before any
    gradient exists (sequence-level importance ratios, SAPO, anything custom).  The price is memory between the two
    passes: 2 bytes x V per such token.  ``grad_token_mask`` (``[T]``, e.g. the loss mask) names those tokens; tokens
    outside it get NO gradient, whatever the loss says; without it every token is kept.  The number of named tokens per
    chunk of ``lm_head_chunk_tokens()`` tokens sizes the stored rows: it is read back from the device unless the caller
    passes it as ``kept_per_chunk`` (counts that are too large are safe, too small ones drop tokens), or leaves it to
    the device with ``count_on_device=True``: nothing is read back then and the host does not wait, the stored rows
    take the room of every token (2 bytes x V x T) whatever the mask holds, and the kernels stop at the rows in use
    (same results, bit for bit).  A gradient
    with respect to the entropy cannot use the stored rows: such a backward forms the logits again, as ``"recompute"``
    does.  The stored rows serve one backward.
    """
    return _lm_head_impl(hidden, weight, labels, temperature, token_mask, False, backward, grad_token_mask,
                         kept_per_chunk, count_on_device)[:2]


def lm_head_logprobs_entropy_stats(
    hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0,
    token_mask: torch.Tensor | None = None, backward: str = "recompute", grad_token_mask: torch.Tensor | None = None,
    kept_per_chunk: list[int] | None = None, count_on_device: bool = False,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(logp, entropy, vocab_min_logits, vocab_max_logits)`` of ``hidden @ weight.T`` from the same tiles.

    The last two are what ``FSDPEngine._get_vocab_min_max_logits`` (areal/engine/fsdp_engine.py:1893-1906) reads from
    materialised logits and hands to the loss function; with no logits in memory the caller could not compute them.
    They come from the fp32 sums of the tiles, not from logits rounded to bf16 (the smallest exactly, the largest
    through the softmax exponent, i.e. to one rounding), and carry no gradient.  With ``token_mask`` the tokens left
    out of the lm_head get 0 for both.  The other arguments: see ``lm_head_logprobs_entropy``."""
    return _lm_head_impl(hidden, weight, labels, temperature, token_mask, True, backward, grad_token_mask,
                         kept_per_chunk, count_on_device)


def _lm_head_apply(hidden, weight, y, temperature, want_minmax, backward, grad_mask, kept_per_chunk,
                   count_on_device=False):
    """One of the two autograd functions on a contiguous batch; ``grad_mask``: bool / uint8 ``[T]`` or None."""
    needs_grad = torch.is_grad_enabled() and (hidden.requires_grad or weight.requires_grad)
    if backward != "carry" or not needs_grad:
        return _LmHeadLogprobsEntropy.apply(hidden, weight, y, float(temperature), want_minmax)
    T = hidden.shape[0]
    chunk = lm_head_chunk_tokens()
    n_chunks = (T + chunk - 1) // chunk
    m8 = kept = None
    if grad_mask is not None:
        m8 = _mask_u8(grad_mask)
        if kept_per_chunk is not None:
            kept = [max(0, min(int(v), chunk)) for v in kept_per_chunk]
            if len(kept) != n_chunks:
                raise ValueError(f"kept_per_chunk needs one count per chunk of {chunk} tokens")
        elif count_on_device:
            kept = [N.AA_LMHEAD_COUNT_ON_DEVICE] * n_chunks
        else:
            on = m8.ne(0)
            if n_chunks * chunk != T:
                on = torch.nn.functional.pad(on, (0, n_chunks * chunk - T))
            kept = _HostCounts(on.view(n_chunks, chunk).sum(1)).tolist()
    return _LmHeadCarry.apply(hidden, weight, y, float(temperature), m8, kept, want_minmax)


def _lm_head_impl(hidden, weight, labels, temperature, token_mask, want_minmax, backward="recompute",
                  grad_token_mask=None, kept_per_chunk=None, count_on_device=False):
    if backward not in _LMHEAD_BACKWARD:
        raise ValueError(f"backward must be one of {sorted(_LMHEAD_BACKWARD)}, got {backward!r}")
    _require_gpu(hidden, "hidden")
    if hidden.ndim != 2 or weight.ndim != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"expected hidden [T, H] and weight [V, H], got {tuple(hidden.shape)} and {tuple(weight.shape)}")
    if tuple(labels.shape) != (hidden.shape[0],):
        raise ValueError(f"labels shape {tuple(labels.shape)} != ({hidden.shape[0]},)")
    assert hidden.shape[0] > 0, "Input must have at least one token"
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("fused lm_head expects bf16 hidden states and weights")
    y = labels.to(device=hidden.device, dtype=torch.int64).contiguous()
    if token_mask is not None:
        if tuple(token_mask.shape) != (hidden.shape[0],):
            raise ValueError(f"token_mask shape {tuple(token_mask.shape)} != ({hidden.shape[0]},)")
        T, dev = hidden.shape[0], hidden.device
        idx = token_mask.to(dev).ne(0).nonzero().squeeze(-1)
        n_kept = idx.numel()
        if n_kept == 0:
            zero = (hidden[:1].float().sum() + weight[:1].float().sum()) * 0.0
            z = torch.zeros(T, dtype=torch.float32, device=dev) if want_minmax else None
            return zero.expand(T), zero.expand(T), z, z
        sub_mask = None if grad_token_mask is None else grad_token_mask.to(dev).reshape(-1).index_select(0, idx)
        lp, ent, vmax, vmin = _lm_head_apply(
            hidden.index_select(0, idx), weight.contiguous(), y.index_select(0, idx), temperature, want_minmax, backward,
            sub_mask, None, count_on_device)   # the caller's counts are per chunk of the whole batch, not of these tokens
        full = lambda v: torch.zeros(T, dtype=torch.float32, device=dev).index_copy(0, idx, v)
        return full(lp), full(ent), (full(vmin) if want_minmax else None), (full(vmax) if want_minmax else None)
    if grad_token_mask is not None and tuple(grad_token_mask.shape) != (hidden.shape[0],):
        raise ValueError(f"grad_token_mask shape {tuple(grad_token_mask.shape)} != ({hidden.shape[0]},)")
    lp, ent, vmax, vmin = _lm_head_apply(hidden.contiguous(), weight.contiguous(), y, temperature, want_minmax, backward,
                                         None if grad_token_mask is None else grad_token_mask.to(hidden.device),
                                         kept_per_chunk, count_on_device)
    return lp, ent, vmin, vmax


def lm_head_logprobs_entropy_static(
    hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0,
    out: tuple[torch.Tensor, torch.Tensor] | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Forward of ``lm_head_logprobs_entropy`` through ``aa_lmhead_fwd_static``: no workspace, nothing allocated by
    the library (its softmax partials live in a 32 MiB device array of its own).  For callers that cannot allocate:
    with ``out = (logp, entropy)`` given (float32 ``[T]``) this function allocates nothing either.  No autograd.
    Calls that overlap on one GPU share that array and race; a vocabulary above ``aa_lmhead_fwd_static_max_vocab()``
    is refused.  The reference has no counterpart."""
    _require_gpu(hidden, "hidden")
    if hidden.ndim != 2 or weight.ndim != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"expected hidden [T, H] and weight [V, H], got {tuple(hidden.shape)} and {tuple(weight.shape)}")
    T, H = hidden.shape
    V = weight.shape[0]
    if tuple(labels.shape) != (T,) or labels.dtype != torch.int64 or not labels.is_contiguous():
        raise ValueError("labels must be a contiguous int64 tensor of shape [T]")
    assert T > 0, "Input must have at least one token"
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("fused lm_head expects bf16 hidden states and weights")
    if not hidden.is_contiguous() or not weight.is_contiguous():
        raise ValueError("hidden and weight must be contiguous")
    lib = N.load()
    if V > lib.aa_lmhead_fwd_static_max_vocab():
        raise ValueError(f"vocabulary {V} is beyond what aa_lmhead_fwd_static takes ({lib.aa_lmhead_fwd_static_max_vocab()})")
    dev = hidden.device
    if out is None:
        out = (torch.empty(T, dtype=torch.float32, device=dev), torch.empty(T, dtype=torch.float32, device=dev))
    logp, entropy = out
    for t in out:
        if t.dtype != torch.float32 or tuple(t.shape) != (T,) or not t.is_contiguous() or t.device != dev:
            raise ValueError("out must hold two contiguous float32 tensors of shape [T] on the device of hidden")
    with torch.cuda.device(dev):
        N.check(
            lib.aa_lmhead_fwd_static(_ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), 1.0 / float(temperature), _ptr(logp),
                                     _ptr(entropy), None, None, _stream(dev)),
            "aa_lmhead_fwd_static",
        )
    return logp, entropy


class _FusedLmHeadPpo(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature, T_active, prox, adv, mask_eff, behave_w, params, n_valid,
                grad_scale, kept_per_chunk, backward_mode):
        ctx.set_materialize_grads(False)  # no zero-filled gradients for the outputs that have none
        lib = N.load()
        kept = None if kept_per_chunk is None else (C.c_int64 * len(kept_per_chunk))(*kept_per_chunk)
        T, H = hidden.shape
        V = weight.shape[0]
        dev = hidden.device
        f32 = dict(dtype=torch.float32, device=dev)
        logp = torch.empty(T, **f32)
        entropy = torch.empty(T, **f32)
        vmax = torch.empty(T, **f32)
        vmin = torch.empty(T, **f32)
        stat_loss = torch.empty(T_active, **f32)
        ratio = torch.empty(T_active, **f32)
        flags = torch.empty(T_active, dtype=torch.uint8, device=dev)
        loss = torch.empty((), **f32)
        d_hidden = torch.empty_like(hidden)
        d_weight = torch.empty_like(weight)  # bf16: rounded once, after fp32 accumulation over the chunks
        ws = _lmhead_workspace(T, H, V, dev)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(
                lib.aa_lmhead_ppo_fused(
                    _ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), 1.0 / float(temperature), T_active, _ptr(prox),
                    _ptr(adv), _ptr(mask_eff), _ptr(behave_w), C.byref(params), _ptr(n_valid), _ptr(grad_scale), kept,
                    int(backward_mode), _ptr(logp), _ptr(entropy), _ptr(stat_loss), _ptr(ratio), _ptr(flags),
                    _ptr(vmax), _ptr(vmin), _ptr(d_hidden), _ptr(d_weight), _DTYPES[d_weight.dtype], _ptr(ws),
                    ws.numel(), st,
                ),
                "aa_lmhead_ppo_fused",
            )
            _finish_fused_loss(lib, params, stat_loss, logp, mask_eff, T_active, n_valid, grad_scale, loss, st)
        ctx.save_for_backward(d_hidden, d_weight)
        ctx.mark_non_differentiable(logp, entropy, stat_loss, ratio, flags, vmax, vmin)
        return loss, logp, entropy, stat_loss, ratio, flags, vmax, vmin

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        if g_loss is None:
            return (None,) * 14
        _hand_out_once(ctx)
        lib = N.load()
        d_hidden, d_weight = ctx.saved_tensors
        dev = d_hidden.device
        g = _f32(g_loss).reshape(1)
        with torch.cuda.device(dev):  # both gradients were written with the loss; a factor of 1 is a no-op
            for t in (d_hidden, d_weight):
                N.check(lib.aa_scale_inplace(_ptr(t), _DTYPES[t.dtype], t.numel(), _ptr(g), _stream(dev)),
                        "aa_scale_inplace")
        return (d_hidden, d_weight) + (None,) * 12


def fused_lm_head_ppo_loss(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip: float,
    loss_mask: torch.Tensor,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling: Any | None = None,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
    temperature: float = 1.0,
    loss_scale: torch.Tensor | float | None = None,
    skip_masked_tokens: bool = True,
    forward_masked_tokens: bool = True,
    kept_per_chunk: list[int] | None = None,
    backward: str = "carry",
    carry_rows_limit_bytes: int = 16 << 30,
    count_on_device: bool = True,
) -> tuple[torch.Tensor, dict]:
    """lm_head + ``gather_logprobs_entropy`` + ``ppo_actor_loss_fn`` (+ backward) for one micro-batch.

    ``hidden`` is ``[T_pad, H]`` (the final hidden states of the batch-padded micro-batch), ``weight`` the ``[V, H]``
    lm_head, both bf16; the other arguments are those of ``fused_logprobs_ppo_loss``.  The logits are formed as
    256 x 256 tiles in the accumulator registers of the library's bf16 MFMA tile GEMM and reduced to softmax partials
    in its epilogue; they are never written to memory.  Tokens are processed in chunks of at most 16384;
    ``loss.backward()`` hands back ``d(hidden)`` and ``d(weight)`` written during the forward pass (the loss is
    known by then).  With ``importance_sampling_level="sequence"`` (GSPO) every log-prob of a sequence is needed before
    any gradient exists, so the call runs ``lm_head_logprobs_entropy`` and the unfused loss; with ``backward="carry"``
    that op keeps the bf16 rows of the tokens with a mask from its forward to its backward (two GEMMs instead of
    three), as long as they take no more than ``carry_rows_limit_bytes`` (2 bytes x V per such token; default 16 GiB),
    and forms the logits again otherwise.

    ``backward`` chooses how the bf16 ``d(loss)/d(logits)`` rows of a chunk (``[tokens with gradient, V]`` in the
    workspace, which the two gradient GEMMs contract) are obtained.  ``"recompute"``: the logits tiles of those tokens
    are formed a second time once the loss is known, as ``lm_head_logprobs_entropy``'s backward does (a third more
    matrix work).  ``"carry"`` (default, the faster of the two by measurement): the forward tiles also write
    ``p_v / p_label`` of those tokens in bf16 into the rows (the label's logit is known before the tiles run); once
    the loss is known the gradient row is that row times one factor per token, which the two gradient GEMMs apply
    themselves, so there is neither a second logits GEMM nor a pass over the rows.  A chunk that holds a token whose
    label has a log-prob below -80, or whose factor is below 2^-100 in magnitude (outside the stored range), is redone
    by recompute, decided on the device.  Both
    modes use the same workspace (``2 * chunk * V`` bytes for the rows).

    ``skip_masked_tokens``: a token whose (effective) loss mask is zero has a zero gradient row, so the two gradient
    GEMMs run on the other tokens only; the results are those of the dense computation.  ``False`` multiplies the
    zero rows through, as the reference's autograd does.  How many tokens of a chunk take part is counted on the
    device (``count_on_device=True``, the default): the kernels are queued for every token that could and stop at
    the rows in use, so the host neither needs the mask nor waits for the device; the results are, bit for bit, those
    of the same counts given by the host, in the same time.  With ``count_on_device=False`` the
    host reads the per-chunk counts back (one small device-to-host copy that waits for the mask only) and sizes the
    GEMMs itself.  A caller that already knows the counts on the host (the number of tokens with a
    non-zero effective mask in each chunk of ``aa_lmhead_chunk_tokens()`` tokens, e.g. from the CPU copy of
    ``loss_mask`` when there is no rejection sampling) can pass them as ``kept_per_chunk``; nothing is read back then
    either.  A count that is too small drops the tokens beyond it from the gradient; a count that is too large (e.g.
    counts of ``loss_mask`` while rejection sampling shrinks the mask on the device) is safe: the surplus rows are
    cleared on the device and add nothing.

    ``stat`` also holds ``vocab_min_logits`` / ``vocab_max_logits`` (what the engine would read from materialised
    logits, areal/engine/fsdp_engine.py:1893-1906), from the fp32 sums of the tiles.

    ``forward_masked_tokens=False`` (token level only) goes one step further than the reference's semantics: tokens
    whose effective mask is zero are not run through the lm_head at all, so their entries of ``stat["logprobs"]``,
    ``stat["entropy"]``, ``stat["loss"]``, ``stat["importance_weight"]`` and ``stat["approx_kl"]`` are zero instead
    of the values the reference computes there (and every consumer masks out).  Loss, gradients and the entries of
    the other tokens are unchanged.
    """
    if importance_sampling_level not in ("token", "sequence"):
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. Must be 'token' or 'sequence'."
        )
    if backward not in _LMHEAD_BACKWARD:
        raise ValueError(f"backward must be one of {sorted(_LMHEAD_BACKWARD)}, got {backward!r}")
    _require_gpu(hidden, "hidden")
    if hidden.ndim != 2 or weight.ndim != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"expected hidden [T, H] and weight [V, H], got {tuple(hidden.shape)} and {tuple(weight.shape)}")
    if tuple(labels.shape) != (hidden.shape[0],):
        raise ValueError(f"labels shape {tuple(labels.shape)} != ({hidden.shape[0]},)")
    assert hidden.shape[0] > 0, "Input must have at least one token"
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("fused lm_head expects bf16 hidden states and weights")
    T_active = loss_mask.shape[0]
    if loss_mask.ndim != 1 or T_active > hidden.shape[0]:
        raise ValueError(f"loss_mask shape {tuple(loss_mask.shape)} does not fit hidden {tuple(hidden.shape)}")
    for name, t in (("proximal_logprobs", proximal_logprobs), ("old_logprobs", old_logprobs), ("advantages", advantages)):
        if t.shape != loss_mask.shape:
            raise ValueError(f"{name} shape {tuple(t.shape)} != loss_mask shape {tuple(loss_mask.shape)}")
    dev = hidden.device
    scale_t = None
    if loss_scale is not None:
        scale_t = torch.as_tensor(loss_scale, dtype=torch.float32, device=dev).reshape(1)
    y = labels.to(device=dev, dtype=torch.int64).contiguous()

    forward_only = not (torch.is_grad_enabled() and (hidden.requires_grad or weight.requires_grad))
    if importance_sampling_level == "sequence" or forward_only:
        # forward-only: forward GEMM + loss.  Sequence level: every log-prob of a sequence is needed before any gradient
        # exists, so the op and the loss run one after the other; in carry mode the op keeps the rows of the tokens with
        # a mask for its backward (2 bytes x V per such token until then) unless that is more than the caller allows
        grad_mask = kept_seq = None
        op_backward = "recompute"
        if not forward_only and backward == "carry":
            pad = hidden.shape[0] - T_active
            grad_mask = loss_mask.to(dev).reshape(-1).ne(0)
            if pad:
                grad_mask = torch.nn.functional.pad(grad_mask, (0, pad))
            if kept_per_chunk is not None:
                kept_seq = [int(v) for v in kept_per_chunk]
            rows_bound = sum(kept_seq) if kept_seq is not None else hidden.shape[0]
            if 2 * rows_bound * weight.shape[0] <= carry_rows_limit_bytes:
                op_backward = "carry"
        logp, entropy, vmin, vmax = lm_head_logprobs_entropy_stats(
            hidden, weight, y, temperature, backward=op_backward,
            grad_token_mask=grad_mask if op_backward == "carry" else None,
            kept_per_chunk=kept_seq if op_backward == "carry" else None,
            count_on_device=count_on_device)
        logp, entropy = logp[:T_active], entropy[:T_active]
        loss, stat = ppo_actor_loss_fn(
            logp, proximal_logprobs, old_logprobs, advantages, eps_clip, loss_mask, eps_clip_higher, c_clip,
            rejection_sampling, importance_sampling_level, cu_seqlens,
        )
        if scale_t is not None:
            loss = loss * scale_t.squeeze(0)
        stat.update(logprobs=logp.detach(), entropy=entropy.detach(), vocab_min_logits=vmin[:T_active],
                    vocab_max_logits=vmax[:T_active])
        return loss, stat

    prox = _f32(proximal_logprobs.detach())
    old = _f32(old_logprobs.detach())
    adv = _f32(advantages.detach())
    m8 = _mask_u8(loss_mask)
    params = _ppo_params(eps_clip, eps_clip_higher, c_clip, rejection_sampling is not None)
    w = counts = None
    mask_eff = m8
    if rejection_sampling is not None:
        _validate_rs(rejection_sampling)
        mask_eff, w, counts = _rejection_sampling_device(prox, old, m8, loss_mask.shape, cu_seqlens, rejection_sampling)
        host_counts = _HostCounts(counts)
        if rejection_sampling.action != "mask":
            mask_eff = m8
        n_valid = counts
    else:
        n_valid = _count_nonzero(m8)
    if not forward_masked_tokens:
        # only the tokens with a mask go through the lm_head: gather them (autograd scatters d(hidden) back), run the
        # step on the closed-up batch with an all-true mask, and put the per-token results back at their tokens
        idx = mask_eff.nonzero().squeeze(-1)
        n_kept = idx.numel()
        full = lambda v, dtype=torch.float32: torch.zeros(T_active, dtype=dtype, device=dev).index_copy_(0, idx, v)
        if n_kept == 0:
            loss = (hidden[:1].float().sum() + weight[:1].float().sum()) * 0.0
            z = torch.zeros(T_active, dtype=torch.float32, device=dev)
            zb = torch.zeros(T_active, dtype=torch.bool, device=dev)
            stat = dict(loss=z, importance_weight=z.clone(), approx_kl=z.clone(), clip_mask=zb, dual_clip_mask=zb.clone(),
                        logprobs=z.clone(), entropy=z.clone(), vocab_min_logits=z.clone(), vocab_max_logits=z.clone())
        else:
            ones = torch.ones(n_kept, dtype=torch.uint8, device=dev)
            chunk = int(N.load().aa_lmhead_chunk_tokens())
            kept = [max(0, min(chunk, n_kept - c)) for c in range(0, n_kept, chunk)]
            loss, logp, entropy, stat_loss, ratio, flags, vmax, vmin = _FusedLmHeadPpo.apply(
                hidden.index_select(0, idx), weight.contiguous(), y.index_select(0, idx), float(temperature), n_kept,
                prox.index_select(0, idx), adv.index_select(0, idx), ones,
                None if w is None else w.index_select(0, idx), params, n_valid, scale_t, kept, _LMHEAD_BACKWARD[backward],
            )
            logp, entropy = logp[:n_kept], entropy[:n_kept]
            clip, dual = _flag_bits(flags)
            stat = dict(
                loss=full(stat_loss), importance_weight=full(ratio), approx_kl=full(logp - prox.index_select(0, idx)),
                clip_mask=full(clip, torch.bool), dual_clip_mask=full(dual, torch.bool),
                logprobs=full(logp), entropy=full(entropy),
                vocab_min_logits=full(vmin[:n_kept]), vocab_max_logits=full(vmax[:n_kept]),
            )
        if rejection_sampling is not None:
            behave_mask = (w > 0) & mask_eff.bool()
            _rs_stats(stat, behave_mask, torch.where(behave_mask, prox - old, 0.0), w, host_counts, loss_mask.shape)
        return loss, stat
    kept = None
    if skip_masked_tokens and kept_per_chunk is not None:
        chunk = int(N.load().aa_lmhead_chunk_tokens())
        kept = [int(v) for v in kept_per_chunk]
        if len(kept) != (hidden.shape[0] + chunk - 1) // chunk:
            raise ValueError(f"kept_per_chunk needs one count per chunk of {chunk} tokens")
    elif skip_masked_tokens:
        kept = _device_or_read_back_counts(hidden.shape[0], T_active, mask_eff, count_on_device)
    loss, logp, entropy, stat_loss, ratio, flags, vmax, vmin = _FusedLmHeadPpo.apply(
        hidden.contiguous(), weight.contiguous(), y, float(temperature), T_active, prox, adv, mask_eff, w, params,
        n_valid, scale_t, kept, _LMHEAD_BACKWARD[backward],
    )
    logp_a = logp[:T_active]
    approx_kl, clip, dual, behave_mask, behave_kl = _stat_outputs(logp_a, prox, old, flags, w, mask_eff)
    stat = dict(
        loss=stat_loss,
        importance_weight=ratio,
        approx_kl=approx_kl,
        clip_mask=clip,
        dual_clip_mask=dual,
        logprobs=logp_a,
        entropy=entropy[:T_active],
        vocab_min_logits=vmin[:T_active],
        vocab_max_logits=vmax[:T_active],
    )
    if rejection_sampling is not None:
        _rs_stats(stat, behave_mask, behave_kl, w, host_counts, loss_mask.shape)
    return loss, stat


# ----------------------------------------------------------------------------
# sibling losses: SAPO, clipped value loss of the critic
# ----------------------------------------------------------------------------
class _SapoLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logp, old, adv, mask, cu, B, seq_level, tau_pos, tau_neg, n_valid):
        lib = N.load()
        dev = logp.device
        n = logp.numel()
        f32 = dict(dtype=torch.float32, device=dev)
        stat_loss, ratio, g_logp = (torch.empty(n, **f32) for _ in range(3))
        gates = torch.empty(3, n, **f32)
        loss = torch.empty((), **f32)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(
                lib.aa_sapo_loss(_ptr(logp), _ptr(old), _ptr(adv), _ptr(mask), n, _ptr(cu), B, 1 if seq_level else 0,
                                 float(tau_pos), float(tau_neg), _ptr(n_valid), _ptr(stat_loss), _ptr(ratio),
                                 _ptr(gates), _ptr(g_logp), st),
                "aa_sapo_loss",
            )
            N.check(lib.aa_masked_sum(_ptr(stat_loss), _ptr(mask), n, _ptr(n_valid), None, _ptr(loss), st),
                    "aa_masked_sum")
        ctx.save_for_backward(g_logp)
        ctx.mark_non_differentiable(stat_loss, ratio, gates)
        return loss, stat_loss, ratio, gates

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        if g_loss is None:  # the loss was not used (gradients are not materialised, see forward)
            return (None,) * 10
        (g_logp,) = ctx.saved_tensors
        return (g_logp * g_loss,) + (None,) * 9


def sapo_loss_fn(
    logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    tau_pos: float,
    tau_neg: float,
    loss_mask: torch.Tensor,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
) -> tuple[torch.Tensor, dict]:
    """SAPO loss with asymmetric sigmoid gates; functional.py:562-638, same stat keys."""
    if tau_pos <= 0 or tau_neg <= 0:
        raise ValueError("SAPO temperatures (tau_pos, tau_neg) must be positive.")
    if importance_sampling_level not in ("token", "sequence"):
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. Must be 'token' or 'sequence'."
        )
    _require_gpu(logprobs, "logprobs")
    shape = logprobs.shape
    seq_level = importance_sampling_level == "sequence"
    cu, B = None, 0
    if seq_level:
        cu, B = _segments(
            shape,
            cu_seqlens,
            "cu_seqlens is required for 1D tensors (packed format). For a single sequence, use "
            "cu_seqlens=torch.tensor([0, seq_len], dtype=torch.int32).",
        )
        if cu is not None:
            cu = cu.to(logprobs.device)
    lp = _f32(logprobs).reshape(-1)
    old = _f32(old_logprobs.detach()).reshape(-1)
    adv = _f32(advantages.detach()).reshape(-1)
    m8 = _mask_u8(loss_mask).reshape(-1)
    n_valid = _count_nonzero(m8)
    loss, stat_loss, ratio, gates = _SapoLoss.apply(lp, old, adv, m8, cu, B, seq_level, tau_pos, tau_neg, n_valid)
    zeros = torch.zeros(shape, dtype=torch.bool, device=lp.device)
    stat = dict(
        loss=stat_loss.view(shape),
        importance_weight=ratio.view(shape),
        approx_kl=(lp.detach() - old).view(shape),
        clip_mask=zeros,
        dual_clip_mask=zeros.clone(),
        sapo_soft_gate=gates[0].view(shape),
        sapo_scaled_gate_pos=gates[1].view(shape),
        sapo_scaled_gate_neg=gates[2].view(shape),
    )
    return loss, stat


class _CriticLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, value, old, target, mask, eps, loss_type, n_valid):
        lib = N.load()
        dev = value.device
        n = value.numel()
        f32 = dict(dtype=torch.float32, device=dev)
        stat_loss, g_value = torch.empty(n, **f32), torch.empty(n, **f32)
        clip = torch.empty(n, dtype=torch.uint8, device=dev)
        total = torch.empty((), **f32)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(
                lib.aa_critic_loss(_ptr(value), _ptr(old), _ptr(target), _ptr(mask), n, float(eps), loss_type,
                                   _ptr(n_valid), _ptr(stat_loss), _ptr(clip), _ptr(g_value), st),
                "aa_critic_loss",
            )
            N.check(lib.aa_masked_sum(_ptr(stat_loss), _ptr(mask), n, None, None, _ptr(total), st), "aa_masked_sum")
        loss = total / n_valid[0].to(torch.float32)  # no floor: an empty mask gives NaN, as in the reference
        ctx.save_for_backward(g_value)
        ctx.mark_non_differentiable(stat_loss, clip)
        return loss, stat_loss, clip

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        (g_value,) = ctx.saved_tensors
        return (g_value * g_loss,) + (None,) * 6


def ppo_critic_loss_fn(
    value: torch.Tensor,
    old_value: torch.Tensor,
    target_value: torch.Tensor,
    value_eps_clip: float,
    loss_mask: torch.Tensor | None = None,
    loss_fn_type: str = "mse",
) -> tuple[torch.Tensor, dict]:
    """Clipped value loss of the PPO critic; functional.py:704-778 (stat keys ``clip_mask``, ``loss``)."""
    assert value.dtype == torch.float32
    assert old_value.dtype == torch.float32
    assert target_value.dtype == torch.float32
    if loss_fn_type not in ("mse", "huber"):
        raise NotImplementedError(f"Unknown loss fn type: {loss_fn_type}")
    _require_gpu(value, "value")
    shape = value.shape
    v = value.contiguous().reshape(-1)
    o = old_value.detach().contiguous().reshape(-1)
    t = target_value.detach().contiguous().reshape(-1)
    if loss_mask is not None:
        m8 = _mask_u8(loss_mask).reshape(-1)
        n_valid = _count_nonzero(m8)
    else:
        m8 = None
        n_valid = torch.full((1,), v.numel(), dtype=torch.int32, device=v.device)
    loss, stat_loss, clip = _CriticLoss.apply(v, o, t, m8, value_eps_clip, 0 if loss_fn_type == "mse" else 1, n_valid)
    return loss, dict(clip_mask=clip.bool().view(shape), loss=stat_loss.view(shape))
