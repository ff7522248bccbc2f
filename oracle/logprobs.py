"""Oracle of the log-prob / entropy op (test infrastructure, CPU only).

Follows areal/utils/functional/vocab_parallel.py:
  :15-20   log_softmax of the fp32-cast logits divided by the temperature, then gather
  :23-29   the same plus entropy = -sum(p * log p)
  :41-61   the op is applied to chunks of at most ``chunk_size`` rows of dim 0 and
           the pieces are concatenated (the result does not depend on chunking)
  :339-370 closed form of both gradients (used here as an independent check of autograd)
"""
from __future__ import annotations

import torch


def _row_chunks(n: int, chunk_size: int):
    assert n > 0, "Input logits must have at least one element"
    start = 0
    while start < n:
        stop = min(start + chunk_size, n)
        yield start, stop
        start = stop


def logprobs(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0, chunk_size: int = 1024):
    """fp32 log-prob of each label; vocab_parallel.py:15-20 applied per chunk (:41-61)."""
    pieces = []
    for a, b in _row_chunks(logits.shape[0], chunk_size):
        lsm = torch.log_softmax(logits[a:b].float() / temperature, dim=-1)
        pieces.append(torch.gather(lsm, -1, labels[a:b].unsqueeze(-1)).squeeze(-1))
    return torch.cat(pieces)


def logprobs_entropy(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0, chunk_size: int = 1024):
    """(log-prob of each label, entropy of each row) in fp32; vocab_parallel.py:23-29 per chunk."""
    lp_pieces, ent_pieces = [], []
    for a, b in _row_chunks(logits.shape[0], chunk_size):
        lsm = torch.log_softmax(logits[a:b].float() / temperature, dim=-1)
        ent_pieces.append(-(lsm.exp() * lsm).sum(dim=-1))
        lp_pieces.append(torch.gather(lsm, -1, labels[a:b].unsqueeze(-1)).squeeze(-1))
    return torch.cat(lp_pieces), torch.cat(ent_pieces)


def logprobs_entropy_f64(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0):
    """Same quantities with every step in float64 (the yardstick for tolerances)."""
    z = logits.double() / float(temperature)
    lsm = torch.log_softmax(z, dim=-1)
    lp = torch.gather(lsm, -1, labels.unsqueeze(-1)).squeeze(-1)
    ent = -(lsm.exp() * lsm).sum(dim=-1)
    return lp, ent


def logprobs_entropy_grad_closed_form(
    logits: torch.Tensor,
    labels: torch.Tensor,
    g_logp: torch.Tensor,
    g_entropy: torch.Tensor | None,
    temperature: float = 1.0,
) -> torch.Tensor:
    """d/d(logits) of sum(g_logp * logp) + sum(g_entropy * entropy), float64.

    The closed form the reference's vocab-parallel variant uses
    (vocab_parallel.py:339-370): with z = logits / T and p = softmax(z),
      grad_z = g_logp * (onehot - p) + g_entropy * p * (E_p[z] - z)
    and grad_logits = grad_z / T.
    """
    z = logits.double() / float(temperature)
    p = torch.softmax(z, dim=-1)
    onehot = torch.zeros_like(p)
    onehot.scatter_(-1, labels.unsqueeze(-1), 1.0)
    grad_z = g_logp.double().unsqueeze(-1) * (onehot - p)
    if g_entropy is not None:
        ez = (p * z).sum(dim=-1, keepdim=True)
        grad_z = grad_z + g_entropy.double().unsqueeze(-1) * p * (ez - z)
    return grad_z / float(temperature)
