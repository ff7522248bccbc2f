"""Pins of oracle/dpo.py: the known answers of the reference's own tests (tests/test_dpo.py, transcribed as data),
a scalar Python restatement from the published definitions with a different indexing of the shift, and central
differences for the gradient."""
import math

import numpy as np
import pytest
import torch

from oracle import dpo as D

LOG2 = math.log(2.0)


def _loss(lp, ref, cu, mask, beta, loss_type="sigmoid"):
    t = lambda a, dt: torch.tensor(a, dtype=dt)
    return D.compute_dpo_loss(t(lp, torch.float32), t(ref, torch.float32), t(cu, torch.int32), t(mask, torch.bool),
                              beta, loss_type)


def test_reference_shift_alignment_cases():
    # tests/test_dpo.py:232-281: nothing leaks across the sequence boundary -> both sums 0 -> loss = log 2
    lp = [100.0, 0, 0, 0, 100.0, 0, 0, 0]
    loss, _ = _loss(lp, [0.0] * 8, [0, 4, 8], [0, 0, 1, 1, 0, 0, 0, 1], 0.1)
    assert abs(float(loss) - LOG2) < 1e-5
    # :283-318: the last position of a sequence is never counted, whatever its mask
    lp = [0.0, 0.0, 0.0, 1e6] * 2
    loss, _ = _loss(lp, [0.0] * 8, [0, 4, 8], [1] * 8, 0.1)
    assert abs(float(loss) - LOG2) < 1e-5
    # :320-347: two pairs with identical chosen and rejected content
    seq = [0.0, 0.0, -1.0, -2.0, -3.0]
    loss, _ = _loss(seq * 4, [0.0] * 20, [0, 5, 10, 15, 20], [0, 0, 1, 1, 1] * 4, 0.5)
    assert abs(float(loss) - LOG2) < 1e-5


def test_reference_ordering_and_masking_cases():
    cu, ones, zeros = [0, 4, 8], [1] * 8, [0.0] * 8
    # :58-78 chosen preferred -> lower loss
    good, _ = _loss([-0.1] * 4 + [-5.0] * 4, zeros, cu, ones, 0.1)
    bad, _ = _loss([-5.0] * 4 + [-0.1] * 4, zeros, cu, ones, 0.1)
    assert float(good) < float(bad)
    # :103-133 reference agreeing with the policy -> log 2; disagreeing -> lower
    lp = [-1.0] * 4 + [-2.0] * 4
    same, _ = _loss(lp, lp, cu, ones, 0.1)
    opp, _ = _loss(lp, [-2.0] * 4 + [-1.0] * 4, cu, ones, 0.1)
    assert abs(float(same) - LOG2) < 1e-6 and float(opp) < float(same)
    # :151-190 prompt tokens do not matter
    mask = [0, 0, 0, 0, 1, 1, 0, 0, 0, 0, 1, 1]
    a, _ = _loss([-10.0] * 4 + [-1.0] * 2 + [-10.0] * 4 + [-2.0] * 2, [0.0] * 12, [0, 6, 12], mask, 0.1)
    b, _ = _loss([-0.1] * 4 + [-1.0] * 2 + [-0.1] * 4 + [-2.0] * 2, [0.0] * 12, [0, 6, 12], mask, 0.1)
    assert abs(float(a) - float(b)) < 1e-5
    # :135-149, 505-518 all sequences empty -> 0
    for lt in ("sigmoid", "ipo"):
        loss, _ = _loss([], [], [0, 0, 0], [], 0.1, lt)
        assert float(loss) == 0.0
    # :208-226 valid pairs and the loss weight
    assert D.valid_pairs(torch.tensor([0, 5, 10, 15, 20])).tolist() == [True, True]
    assert D.valid_pairs(torch.tensor([0, 5, 10, 15, 15])).tolist() == [True, False]
    with pytest.raises(ValueError, match="Unsupported DPO loss_type"):
        _loss(zeros, zeros, cu, ones, 0.1, "nonexistent")


def test_reference_ipo_cases():
    cu, ones, zeros = [0, 4, 8], [1] * 8, [0.0] * 8
    # :400-422 per-token average equal to 1 / (2 beta) -> loss 0
    beta = 0.1
    lp = [5.0] * 3 + [0.0] * 5
    loss, _ = _loss(lp, zeros, cu, ones, beta, "ipo")
    assert abs(float(loss)) < 1e-4
    # :436-462 same per-token averages at different lengths -> same loss
    a, _ = _loss([-1.0] * 3 + [0.0] + [-2.0] * 3 + [0.0], zeros, cu, ones, 0.1, "ipo")
    b, _ = _loss([-1.0] * 7 + [0.0] + [-2.0] * 7 + [0.0], [0.0] * 16, [0, 8, 16], [1] * 16, 0.1, "ipo")
    assert abs(float(a) - float(b)) < 1e-5
    assert abs(float(a) - (1.0 - 5.0) ** 2) < 1e-5          # average gap 1, target 5
    # :464-486 chosen preferred -> closer to the target
    good, _ = _loss([-0.1] * 4 + [-5.0] * 4, zeros, cu, ones, 0.5, "ipo")
    bad, _ = _loss([-5.0] * 4 + [-0.1] * 4, zeros, cu, ones, 0.5, "ipo")
    assert float(good) < float(bad)


def _scalar_dpo(lp, ref, cu, mask, beta, loss_type):
    """From the definitions: a response token j (mask[j] set, not the first token of its sequence) is predicted at
    position j - 1; a sequence's score is the sum of those log-probs."""
    n = len(cu) - 1
    pol, rf, ln = [0.0] * n, [0.0] * n, [0] * n
    for s in range(n):
        for j in range(cu[s] + 1, cu[s + 1]):
            if mask[j]:
                pol[s] += lp[j - 1]
                rf[s] += ref[j - 1]
                ln[s] += 1
    losses, chosen, rejected = [], [], []
    for p in range(n // 2):
        c, r = 2 * p, 2 * p + 1
        if cu[c + 1] == cu[c] or cu[r + 1] == cu[r]:
            continue
        if loss_type == "ipo":
            x = (pol[c] - rf[c]) / max(ln[c], 1) - (pol[r] - rf[r]) / max(ln[r], 1)
            losses.append((x - 1 / (2 * beta)) ** 2)
        else:
            x = (pol[c] - rf[c]) - (pol[r] - rf[r])
            z = beta * x
            losses.append(math.log1p(math.exp(-z)) if z > 0 else -z + math.log1p(math.exp(z)))
        chosen.append(beta * (pol[c] - rf[c]))
        rejected.append(beta * (pol[r] - rf[r]))
    return (sum(losses) / len(losses) if losses else 0.0), losses, chosen, rejected, pol, rf, ln


@pytest.mark.parametrize("loss_type", ["sigmoid", "ipo"])
def test_against_scalar_restatement_and_central_differences(loss_type):
    rng = np.random.default_rng(11)
    lens = [7, 3, 0, 5, 1, 4, 6, 2, 9, 0]               # pair 1 and pair 4 have an empty side; one length-1 sequence
    cu = [0] + list(np.cumsum(lens))
    T = cu[-1]
    lp = rng.normal(-1.2, 0.6, T)
    ref = lp + rng.normal(0, 0.3, T)
    mask = rng.random(T) < 0.6
    beta = 0.3
    want, losses, chosen, rejected, pol, rf, ln = _scalar_dpo(lp, ref, cu, mask, beta, loss_type)

    t64 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float64)
    valid = D.valid_pairs(torch.tensor(cu))
    assert valid.tolist() == [True, False, True, True, False]
    got = D.pair_logratios(t64(lp), t64(ref), torch.tensor(cu), torch.tensor(mask), valid)
    keep = [i for i in range(len(lens)) if valid[i // 2]]
    assert torch.allclose(got[0].reshape(-1), t64([pol[i] for i in keep]), atol=1e-12)
    assert torch.allclose(got[1].reshape(-1), t64([rf[i] for i in keep]), atol=1e-12)
    assert got[2].reshape(-1).tolist() == [float(ln[i]) for i in keep]

    x = t64(lp).requires_grad_(True)
    loss, stat = D.compute_dpo_loss(x, t64(ref), torch.tensor(cu), torch.tensor(mask), beta, loss_type)
    assert abs(float(loss.detach()) - want) < 1e-5 * max(1.0, abs(want))      # the loss itself is float32
    assert np.allclose(stat["loss"].numpy(), losses, rtol=1e-5, atol=1e-6)
    assert np.allclose(stat["chosen_reward"].numpy(), chosen, rtol=1e-6, atol=1e-6)
    assert np.allclose(stat["rejected_reward"].numpy(), rejected, rtol=1e-6, atol=1e-6)
    loss.backward()
    for i in range(T):
        up, dn = lp.copy(), lp.copy()
        up[i] += 1e-5
        dn[i] -= 1e-5
        fd = (_scalar_dpo(up, ref, cu, mask, beta, loss_type)[0] - _scalar_dpo(dn, ref, cu, mask, beta, loss_type)[0]) / 2e-5
        assert abs(float(x.grad[i]) - fd) < 2e-5 * max(1.0, abs(fd)), (i, float(x.grad[i]), fd)


def test_preference_loss_closed_forms():
    x = torch.tensor([0.0, 3.0, -3.0, 200.0, -200.0], dtype=torch.float64)
    got = D.preference_loss(x, 0.5, "sigmoid")
    assert got.dtype == torch.float32
    want = [LOG2, math.log1p(math.exp(-1.5)), 1.5 + math.log1p(math.exp(-1.5)), 0.0, 100.0]
    assert np.allclose(got.numpy(), want, rtol=1e-6, atol=1e-30)
    got = D.preference_loss(x, 0.25, "ipo")
    assert np.allclose(got.numpy(), [(v - 2.0) ** 2 for v in x.tolist()], rtol=1e-6)


def test_reward_model_loss_reference_cases():
    """tests/test_eval_dispatch.py:325-371: lengths [5, 4, 0, 0], scores 3 and 1 at the two last tokens -> the loss
    is -logsigmoid(2) over the one valid pair; only empty pairs -> 0."""
    cu = torch.tensor([0, 5, 9, 9, 9])
    scores = torch.tensor([0.0, 0.0, 0.0, 0.0, 3.0, 0.0, 0.0, 0.0, 1.0])
    loss, stat = D.compute_rw_loss(scores, cu)
    want = math.log1p(math.exp(-2.0))
    assert abs(float(loss) - want) < 1e-6
    assert stat["valid_pairs"].tolist() == [True, False]
    assert stat["pos_score"].tolist() == [3.0] and stat["neg_score"].tolist() == [1.0]
    assert stat["correct_ratio"].tolist() == [1.0] and abs(float(stat["loss"][0]) - want) < 1e-6
    loss, stat = D.compute_rw_loss(torch.tensor([], dtype=torch.float32), torch.tensor([0, 0, 0]))
    assert float(loss) == 0.0 and stat["valid_pairs"].tolist() == [False]
    # equal scores -> log 2; gradient of the mean: -sigmoid(-(pos - neg)) / K at the chosen token, + at the rejected
    cu = torch.tensor([0, 2, 5, 6, 8])
    s = torch.tensor([9.0, 0.5, 9.0, 9.0, 0.5, 1.0, 9.0, -1.0], requires_grad=True)
    loss, _ = D.compute_rw_loss(s, cu)
    want = (LOG2 + math.log1p(math.exp(-2.0))) / 2
    assert abs(float(loss.detach()) - want) < 1e-6
    loss.backward()
    sig = lambda z: 1 / (1 + math.exp(-z))
    g = [0.0, -0.5 * sig(0.0), 0.0, 0.0, 0.5 * sig(0.0), -0.5 * sig(-2.0), 0.0, 0.5 * sig(-2.0)]
    assert np.allclose(s.grad.numpy(), g, atol=1e-7)
