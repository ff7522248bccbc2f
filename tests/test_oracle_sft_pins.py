"""Pins of oracle/sft.py.  No test of the reference calls compute_packed_sft_loss with known values
(tests/fp8/model_hooks.py:128 only re-implements it), so the restatement is pinned by what the definition fixes:
closed forms, a scalar Python restatement, and the closed-form gradient."""
import math

import numpy as np
import torch

from oracle.sft import packed_sft_loss


def test_closed_forms():
    # every selected token has log-prob -c: loss = c n / (n + 1e-5), every sequence has perplexity e^c
    c = 0.75
    cu = torch.tensor([0, 4, 9, 9, 12])
    mask = torch.tensor([0, 1, 1, 1, 0, 0, 1, 1, 1, 0, 0, 0], dtype=torch.bool)      # last sequence: nothing selected
    lp = torch.full((12,), -c)
    lp[~mask] = -50.0                                                               # must not matter
    loss, stat = packed_sft_loss(lp, mask, cu)
    n = int(mask.sum())
    assert abs(float(loss) - c * n / (n + 1e-5)) < 1e-6
    assert stat["n_seqs"].tolist() == [True, True, False, False]
    assert np.allclose(stat["ppl"].numpy(), [math.exp(c), math.exp(c), 1.0, 1.0], rtol=1e-6)   # skipped: exp(-0)
    assert torch.equal(stat["loss"], torch.where(mask, torch.tensor(c), torch.tensor(0.0)))
    # nothing selected at all: 0 / 1e-5
    loss, stat = packed_sft_loss(lp, torch.zeros(12, dtype=torch.bool), cu)
    assert float(loss) == 0.0 and not stat["n_seqs"].any()


def test_against_scalar_restatement_and_gradient():
    rng = np.random.default_rng(5)
    lens = [5, 1, 0, 9, 3]
    cu = [0] + list(np.cumsum(lens))
    T = cu[-1]
    lp = rng.normal(-1.3, 0.8, T)
    mask = rng.random(T) < 0.6
    n = int(mask.sum())
    # "1e-5 + count" is a Python float plus an integer tensor: torch forms it in float32 (15.00001 -> 15.00000954)
    denom = float(np.float32(1e-5) + np.float32(n))
    want = -sum(lp[t] for t in range(T) if mask[t]) / denom
    seq = []
    for s in range(len(lens)):
        sel = [lp[t] for t in range(cu[s], cu[s + 1]) if mask[t]]
        seq.append(sum(sel) / len(sel) if sel else 0.0)
    x = torch.tensor(lp, requires_grad=True)
    loss, stat = packed_sft_loss(x, torch.tensor(mask), torch.tensor(cu))
    assert abs(float(loss.detach()) - want) < 1e-12
    assert np.allclose(stat["seqlogp"].numpy(), seq, atol=1e-12)
    assert np.allclose(stat["ppl"].numpy(), np.exp(-np.array(seq)), rtol=1e-6)
    assert stat["n_seqs"].tolist() == [any(mask[cu[s]:cu[s + 1]]) for s in range(len(lens))]
    loss.backward()
    assert np.allclose(x.grad.numpy(), np.where(mask, -1.0 / denom, 0.0), atol=1e-15)
