"""CPU oracle of the supervised fine-tuning loss over a packed batch.  TEST INFRASTRUCTURE ONLY.

Restates ``compute_packed_sft_loss`` (areal/trainer/sft/lm_engine.py:81-131) in plain PyTorch on the CPU, with the
logged tensors returned instead of recorded.  How it is pinned is listed in ``oracle/PINNING.md``.
"""
from __future__ import annotations

import torch


def packed_sft_loss(logprobs, loss_mask, cu_seqlens):
    """(loss, stat); lm_engine.py:90-131."""
    loss_mask = loss_mask.bool()
    logprobs = torch.where(loss_mask, logprobs, 0)                                  # :93
    loss = -logprobs.sum() / (1e-5 + loss_mask.count_nonzero())                     # :96
    with torch.no_grad():
        batch_size = cu_seqlens.shape[0] - 1
        seqlogp = torch.zeros(batch_size, dtype=torch.float64)
        n_seqs = torch.zeros(batch_size, dtype=torch.bool)
        for i in range(batch_size):                                                 # :101-112
            m = loss_mask[cu_seqlens[i]: cu_seqlens[i + 1]]
            logp = logprobs[cu_seqlens[i]: cu_seqlens[i + 1]]
            valid_tokens = int(m.count_nonzero().item())
            if valid_tokens == 0:
                continue
            n_seqs[i] = True
            seqlogp[i] = torch.where(m, logp.detach(), 0.0).sum() / valid_tokens
    stat = dict(ppl=(-seqlogp).exp().float(), loss=-logprobs.detach(), seqlogp=seqlogp, n_seqs=n_seqs)   # :121-122
    return loss, stat
