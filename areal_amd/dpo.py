"""Pairwise preference losses over a packed batch of interleaved (chosen, rejected) sequences: DPO and the
reward-model loss.

Host-side mirror of ``dpo_pair_logratios`` / ``dpo_preference_loss`` (areal/utils/functional/functional.py:641-703)
and of the loss assembled from them in ``compute_dpo_loss`` (areal/trainer/dpo/dpo_engine.py:147-213); of
``compute_rw_loss`` (areal/trainer/rw/rw_engine.py:115-146).
"""
from __future__ import annotations

import torch

from . import _native as N
from .functional import _DTYPES, _f32, _mask_u8, _ptr, _require_gpu, _stream

_LOSS_TYPES = {"sigmoid": 0, "ipo": 1}


def _loss_type_id(loss_type: str) -> int:
    if loss_type not in _LOSS_TYPES:
        raise ValueError(f"Unsupported DPO loss_type: {loss_type!r}")
    return _LOSS_TYPES[loss_type]


def _packed_inputs(logprobs, ref_logprobs, cu_seqlens, loss_mask):
    _require_gpu(logprobs, "logprobs")
    dev = logprobs.device
    if logprobs.dim() != 1 or ref_logprobs.shape != logprobs.shape or loss_mask.shape != logprobs.shape:
        raise ValueError("logprobs, ref_logprobs and loss_mask must be 1-D and of the same length")
    if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 1:
        raise ValueError("cu_seqlens must be 1-D with at least one entry")
    lp = logprobs if logprobs.dtype == torch.float32 and logprobs.is_contiguous() else logprobs.float().contiguous()
    ref = _f32(ref_logprobs.detach().to(dev))
    m8 = _mask_u8(loss_mask.to(dev))
    cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    return lp, ref, m8, cu


def _launch_bwd(g_sums, scale, m8, cu, n_seqs, T, dev):
    d_logp = torch.empty(T, dtype=torch.float32, device=dev)
    if T:
        lib = N.load()
        with torch.cuda.device(dev):
            N.check(lib.aa_dpo_seq_sums_bwd(_ptr(g_sums), _ptr(scale) if scale is not None else None, _ptr(m8),
                                            _ptr(cu), n_seqs, T, _ptr(d_logp), _stream(dev)), "aa_dpo_seq_sums_bwd")
    return d_logp


class _SeqSums(torch.autograd.Function):
    """Per-sequence fp64 sums under the shifted mask; differentiable in the policy log-probs."""

    @staticmethod
    def forward(ctx, lp, ref, m8, cu):
        lib = N.load()
        dev = lp.device
        n_seqs, T = cu.numel() - 1, lp.numel()
        policy, refs, lens = torch.empty(3, n_seqs, dtype=torch.float64, device=dev).unbind(0)
        if n_seqs:
            with torch.cuda.device(dev):
                N.check(lib.aa_dpo_seq_sums(_ptr(lp), _ptr(ref), _ptr(m8), _ptr(cu), n_seqs, T, _ptr(policy),
                                            _ptr(refs), _ptr(lens), _stream(dev)), "aa_dpo_seq_sums")
        ctx.save_for_backward(m8, cu)
        ctx.mark_non_differentiable(refs, lens)
        return policy, refs, lens

    @staticmethod
    def backward(ctx, g_policy, _g_ref, _g_lens):
        m8, cu = ctx.saved_tensors
        g = g_policy.to(torch.float64).contiguous()
        return _launch_bwd(g, None, m8, cu, cu.numel() - 1, m8.numel(), m8.device), None, None, None


def dpo_pair_logratios(logprobs: torch.Tensor, ref_logprobs: torch.Tensor, cu_seqlens: torch.Tensor,
                       loss_mask: torch.Tensor, valid_pairs: torch.Tensor):
    """Per-sequence masked log-prob sums of a packed batch, paired up; functional.py:641-687.

    Sequences are interleaved ``[chosen_0, rejected_0, chosen_1, ...]``; ``loss_mask`` is shifted by one inside each
    sequence to align with next-token log-probs and the last position of a sequence never counts.  Returns
    ``(policy_logps, ref_logps, completion_lens)``, fp64, each ``[K, 2]`` with ``K = valid_pairs.sum()``, column 0
    chosen and column 1 rejected.  Differentiable in ``logprobs`` only (``ref_logprobs`` is treated as data).
    """
    lp, ref, m8, cu = _packed_inputs(logprobs, ref_logprobs, cu_seqlens, loss_mask)
    if (cu.numel() - 1) % 2:
        raise ValueError("a DPO batch holds an even number of sequences")
    policy, refs, lens = _SeqSums.apply(lp, ref, m8, cu)
    vp = valid_pairs.to(lp.device)
    return policy.view(-1, 2)[vp], refs.view(-1, 2)[vp], lens.view(-1, 2)[vp]


class _PreferenceLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, beta, loss_type):
        lib = N.load()
        dev = x.device
        loss = torch.empty_like(x)
        dloss = torch.empty_like(x)
        if x.numel():
            with torch.cuda.device(dev):
                N.check(lib.aa_dpo_preference_loss(_ptr(x), x.numel(), float(beta), loss_type, _ptr(loss), _ptr(dloss),
                                                   _stream(dev)), "aa_dpo_preference_loss")
        ctx.save_for_backward(dloss)
        return loss

    @staticmethod
    def backward(ctx, g):
        (dloss,) = ctx.saved_tensors
        return g * dloss, None, None


def dpo_preference_loss(logits: torch.Tensor, *, beta: float, loss_type: str = "sigmoid") -> torch.Tensor:
    """Per-pair preference loss from DPO log-ratio logits, float32; functional.py:689-703.

    ``"sigmoid"``: ``-logsigmoid(beta * logits)``; ``"ipo"``: ``(logits - 1 / (2 beta)) ** 2`` on logits that the
    caller has already averaged per token.
    """
    lt = _loss_type_id(loss_type)
    _require_gpu(logits, "logits")
    x = logits.float().contiguous()
    return _PreferenceLoss.apply(x.reshape(-1), float(beta), lt).view(logits.shape)


class _DpoLoss(torch.autograd.Function):
    """Sums, pairing, loss and mean in two launches; the backward is one launch."""

    @staticmethod
    def forward(ctx, lp, ref, m8, cu, beta, loss_type):
        lib = N.load()
        dev = lp.device
        n_seqs, T = cu.numel() - 1, lp.numel()
        n_pairs = n_seqs // 2
        # every element below is written by the two kernels
        policy, refs, lens, g_sums = torch.empty(4, n_seqs, dtype=torch.float64, device=dev).unbind(0)
        pair_loss, chosen, rejected = torch.empty(3, n_pairs, dtype=torch.float32, device=dev).unbind(0)
        valid = torch.empty(n_pairs, dtype=torch.bool, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        n_valid = torch.empty((), dtype=torch.int32, device=dev)
        with torch.cuda.device(dev):
            st = _stream(dev)
            if n_seqs:
                N.check(lib.aa_dpo_seq_sums(_ptr(lp), _ptr(ref), _ptr(m8), _ptr(cu), n_seqs, T, _ptr(policy),
                                            _ptr(refs), _ptr(lens), st), "aa_dpo_seq_sums")
            N.check(lib.aa_dpo_pair_loss(_ptr(policy), _ptr(refs), _ptr(lens), _ptr(cu), n_pairs, float(beta),
                                         loss_type, _ptr(loss), _ptr(n_valid), _ptr(pair_loss), _ptr(chosen),
                                         _ptr(rejected), _ptr(valid), _ptr(g_sums), st), "aa_dpo_pair_loss")
        ctx.save_for_backward(g_sums, m8, cu)
        outs = (pair_loss, chosen, rejected, valid, n_valid)
        ctx.mark_non_differentiable(*outs)
        return (loss,) + outs

    @staticmethod
    def backward(ctx, g_loss, *_):
        g_sums, m8, cu = ctx.saved_tensors
        scale = g_loss.to(torch.float32).contiguous()
        return _launch_bwd(g_sums, scale, m8, cu, cu.numel() - 1, m8.numel(), m8.device), None, None, None, None, None


def dpo_loss(logprobs: torch.Tensor, ref_logprobs: torch.Tensor, cu_seqlens: torch.Tensor, loss_mask: torch.Tensor, *,
             beta: float, loss_type: str = "sigmoid") -> tuple[torch.Tensor, dict]:
    """Mean preference loss over the valid pairs of a packed batch; dpo_engine.py:147-213 without its logging.

    A pair is valid when both of its sequences are non-empty (dpo_engine.py:22-24); with no valid pair the loss is 0.
    Nothing is read back to the host.  Returns ``(loss, stat)`` with per pair (zeros where invalid) ``loss``,
    ``chosen_reward``, ``rejected_reward`` and the bool ``valid_pairs``, and ``n_pairs`` (int32 scalar on the
    device): what the reference records under the ``n_pairs`` denominator.
    """
    lt = _loss_type_id(loss_type)
    lp, ref, m8, cu = _packed_inputs(logprobs, ref_logprobs, cu_seqlens, loss_mask)
    if (cu.numel() - 1) % 2:
        raise ValueError("a DPO batch holds an even number of sequences")
    loss, pair_loss, chosen, rejected, valid, n_valid = _DpoLoss.apply(lp, ref, m8, cu, float(beta), lt)
    stat = dict(loss=pair_loss, chosen_reward=chosen, rejected_reward=rejected, valid_pairs=valid, n_pairs=n_valid)
    return loss, stat


class _RwLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, scores, cu):
        lib = N.load()
        dev = scores.device
        T, n_pairs = scores.numel(), (cu.numel() - 1) // 2
        pair_loss, pos, neg = torch.empty(3, n_pairs, dtype=torch.float32, device=dev).unbind(0)
        valid = torch.empty(n_pairs, dtype=torch.bool, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        n_valid = torch.empty((), dtype=torch.int32, device=dev)
        g = torch.empty(T, dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            N.check(lib.aa_rw_pair_loss(_ptr(scores), T, _ptr(cu), n_pairs, _ptr(loss), _ptr(n_valid), _ptr(pair_loss),
                                        _ptr(pos), _ptr(neg), _ptr(valid), _ptr(g), _stream(dev)), "aa_rw_pair_loss")
        ctx.save_for_backward(g)
        outs = (pair_loss, pos, neg, valid, n_valid)
        ctx.mark_non_differentiable(*outs)
        return (loss,) + outs

    @staticmethod
    def backward(ctx, g_loss, *_):
        (g,) = ctx.saved_tensors
        out = g.clone()   # [T] floats: keeps the saved gradient intact for a second backward (retain_graph)
        dev = g.device
        up = _f32(g_loss).reshape(1)
        if out.numel():
            with torch.cuda.device(dev):
                N.check(N.load().aa_scale_inplace(_ptr(out), _DTYPES[out.dtype], out.numel(), _ptr(up), _stream(dev)),
                        "aa_scale_inplace")
        return out, None


def rw_pair_loss(scores: torch.Tensor, cu_seqlens: torch.Tensor) -> tuple[torch.Tensor, dict]:
    """Mean of ``-logsigmoid(score_chosen - score_rejected)`` over the valid pairs of a packed batch, a sequence's
    score being the one at its last token; rw_engine.py:115-146 without its logging.  With no valid pair the loss
    is 0.  Nothing is read back.  Returns ``(loss, stat)`` with per pair (zeros where invalid) ``loss``,
    ``pos_score``, ``neg_score``, the bool ``valid_pairs`` and ``n_pairs`` (int32 scalar on the device)."""
    _require_gpu(scores, "scores")
    if scores.dim() != 1 or cu_seqlens.dim() != 1 or cu_seqlens.numel() < 1 or (cu_seqlens.numel() - 1) % 2:
        raise ValueError("expected 1-D scores and cu_seqlens over an even number of sequences")
    s = scores if scores.dtype == torch.float32 and scores.is_contiguous() else scores.float().contiguous()
    cu = cu_seqlens.to(device=s.device, dtype=torch.int32).contiguous()
    loss, pair_loss, pos, neg, valid, n_valid = _RwLoss.apply(s, cu)
    return loss, dict(loss=pair_loss, pos_score=pos, neg_score=neg, valid_pairs=valid, n_pairs=n_valid)
