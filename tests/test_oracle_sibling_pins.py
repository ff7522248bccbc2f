"""Pins of oracle/siblings.py: the reference's own known answers (transcribed as data from tests/test_functional.py
and tests/test_prox_approx.py), hand-computed values, and brute force from the definitions."""
import math

import numpy as np
import pytest
import torch

from oracle import siblings as S


def test_sapo_known_value_and_gate_selection():
    # tests/test_functional.py:923-954: ratio 1, advantage 1, tau 1 -> gate 2, loss -2
    one = torch.tensor([[1.0, 1.0]])
    loss, stat = S.sapo_loss(one, one, one, 1.0, 1.0, torch.ones(1, 2, dtype=torch.bool))
    assert abs(float(loss) + 2.0) < 1e-5 and torch.allclose(stat["sapo_soft_gate"], torch.full((1, 2), 2.0), atol=1e-5)
    # tests/test_functional.py:956-1000: the gate follows the sign of the advantage
    lp, old = torch.tensor([[0.5, 0.5]]), torch.zeros(1, 2)
    m = torch.ones(1, 2, dtype=torch.bool)
    _, st = S.sapo_loss(lp, old, torch.tensor([[1.0, 2.0]]), 1.0, 2.0, m)
    assert torch.allclose(st["sapo_soft_gate"], st["sapo_scaled_gate_pos"])
    _, st = S.sapo_loss(lp, old, torch.tensor([[-1.0, -2.0]]), 1.0, 2.0, m)
    assert torch.allclose(st["sapo_soft_gate"], st["sapo_scaled_gate_neg"])
    assert not st["clip_mask"].any() and not st["dual_clip_mask"].any()
    with pytest.raises(ValueError, match="must be positive"):
        S.sapo_loss(lp, old, lp, 0.0, 1.0, m)


def test_sapo_scalar_brute_force_and_gradient():
    rng = np.random.default_rng(0)
    n = 40
    lp, old, adv = rng.normal(size=n) * 0.3, rng.normal(size=n) * 0.3, rng.normal(size=n)
    mask = rng.random(n) < 0.7
    tp, tn = 1.3, 0.8
    total = 0.0
    grad = np.zeros(n)
    for i in range(n):
        r = math.exp(lp[i] - old[i])
        tau = tp if adv[i] > 0 else tn
        g = 1.0 / (1.0 + math.exp(-tau * (r - 1.0)))
        if mask[i]:
            total += -(4.0 / tau) * g * adv[i]
            grad[i] = -4.0 * adv[i] * g * (1 - g) * r / mask.sum()
    x = torch.tensor(lp, requires_grad=True)
    loss, _ = S.sapo_loss(x, torch.tensor(old), torch.tensor(adv), tp, tn, torch.tensor(mask))
    loss.backward()
    assert abs(float(loss.detach()) - total / mask.sum()) < 1e-12
    assert np.allclose(x.grad.numpy(), grad, atol=1e-12)


def test_critic_loss_hand_values():
    # value moved by +0.5 from old with eps 0.2: clipped value = old + 0.2
    value, old, target = torch.tensor([1.5, 1.0, 0.0]), torch.tensor([1.0, 1.0, 1.0]), torch.tensor([2.0, 3.0, 0.5])
    loss, stat = S.critic_loss(value, old, target, 0.2)
    # token 0: orig 0.5*0.25=0.125, clipped 0.5*(1.2-2)^2=0.32 -> 0.32, clipped wins
    # token 1: no move: orig = clipped = 2.0 -> not flagged
    # token 2: value 0, clipped 0.8: orig 0.125, clipped 0.045 -> 0.125
    assert torch.allclose(stat["loss"], torch.tensor([0.32, 2.0, 0.125]), atol=1e-6)
    assert stat["clip_mask"].tolist() == [True, False, False]
    assert abs(float(loss) - (0.32 + 2.0 + 0.125) / 3) < 1e-6
    mask = torch.tensor([True, False, True])
    loss, stat = S.critic_loss(value, old, target, 0.2, mask)
    assert abs(float(loss) - (0.32 + 0.125) / 2) < 1e-6 and stat["clip_mask"].tolist() == [True, False, False]
    # huber with delta 10: quadratic below, linear above
    loss, stat = S.critic_loss(torch.tensor([0.0, 0.0]), torch.tensor([0.0, 0.0]), torch.tensor([3.0, 25.0]), 0.2,
                               loss_fn_type="huber")
    assert torch.allclose(stat["loss"], torch.tensor([4.5, 10.0 * (25.0 - 5.0)]))
    with pytest.raises(NotImplementedError):
        S.critic_loss(value, old, target, 0.2, loss_fn_type="l1")


def test_prox_approx_reference_known_answers():
    f = lambda v: torch.tensor(v, dtype=torch.float32)
    i = lambda v: torch.tensor(v, dtype=torch.int32)
    # tests/test_prox_approx.py:24-44
    a = S.prox_logp_approximations(f([[-1.0, -2.0, -3.0]]), f([[-1.5, -2.5, -3.5]]), i([[0, 0, 0]]), 2)
    assert torch.allclose(a["loglinear"], f([[-1.25, -2.25, -3.25]]), atol=1e-4)
    # :46-63 rollout returns the behaviour log-probs
    a = S.prox_logp_approximations(f([[-1.0, -2.0]]), f([[-5.0, -6.0]]), i([[0, 1]]), 5)
    assert torch.allclose(a["rollout"], f([[-1.0, -2.0]]))
    # :65-82 alpha = 0 when behaviour version = proximal version
    a = S.prox_logp_approximations(f([[-1.0]]), f([[-2.0]]), i([[4]]), 5)
    assert torch.allclose(a["loglinear"], f([[-1.0]]), atol=1e-4)
    # :84-106 mixed versions
    a = S.prox_logp_approximations(f([[-1.0], [-2.0]]), f([[-1.5], [-2.2]]), i([[0], [2]]), 4)
    assert torch.allclose(a["loglinear"], f([[-1.375], [-2.1]]), atol=1e-4)
    # :108-127 linear in probability space
    a = S.prox_logp_approximations(f([[-0.693]]), f([[-1.386]]), i([[0]]), 2)
    assert torch.allclose(a["linear"], torch.log(f([[0.375]])), atol=1e-3)
    # :150-166 equal versions: no division by zero, alpha 0
    a = S.prox_logp_approximations(f([[-1.0]]), f([[-2.0]]), i([[3]]), 3)
    assert torch.allclose(a["loglinear"], f([[-1.0]]), atol=1e-4)
    # :168-187 prompt tokens (negative version) are not interpolated
    a = S.prox_logp_approximations(f([[-1.0, -2.0, -3.0]]), f([[-1.5, -2.5, -3.5]]), i([[-1, 0, 1]]), 3)
    assert float(a["loglinear"][0, 0]) == -1.0 and torch.isfinite(a["loglinear"]).all()
    assert list(S.prox_logp_approximations(f([[-1.0]]), f([[-2.0]]), i([[0]]), 2, method="linear")) == ["linear"]


def _m2po_brute(m2, mask, thr):
    """Remove the largest valid value while the mean of the valid rest is not below the threshold (keep one)."""
    keep = [i for i in range(len(m2)) if mask[i]]
    while len(keep) > 1 and np.mean([m2[i] for i in keep], dtype=np.float64) >= thr:
        worst = max(keep, key=lambda i: (m2[i], -i))  # ties: the lower index goes first
        keep.remove(worst)
    out = np.zeros(len(m2), dtype=bool)
    out[keep] = True
    return out


@pytest.mark.parametrize("thr", [0.02, 0.1, 0.5, 1e-9, 100.0])
def test_m2po_against_brute_force(thr):
    rng = np.random.default_rng(4)
    old = rng.normal(size=(6, 11)).astype(np.float32) * 0.5
    prox = old + rng.normal(size=(6, 11)).astype(np.float32) * 0.4
    mask = rng.random((6, 11)) < 0.7
    got = S.m2po_mask(torch.tensor(old), torch.tensor(prox), torch.tensor(mask), thr).numpy()
    d = (old - prox).reshape(-1)
    want = _m2po_brute((d * d).tolist(), mask.reshape(-1).tolist(), thr).reshape(6, 11)
    assert (got == want).all()
    assert got.sum() >= 1 and not (got & ~mask).any()


def test_m2po_edge_cases():
    old, prox = torch.zeros(5), torch.tensor([0.0, 1.0, 2.0, 3.0, 4.0])
    none = torch.zeros(5, dtype=torch.bool)
    assert torch.equal(S.m2po_mask(old, prox, none, 0.1), none)           # nothing selected: unchanged
    allm = torch.ones(5, dtype=torch.bool)
    # squares 0, 1, 4, 9, 16; means of suffixes (desc): 6, 3.5, 1.67, 0.5, 0 -> threshold 2 drops 16 and 9
    assert S.m2po_mask(old, prox, allm, 2.0).tolist() == [True, True, True, False, False]
    # nothing qualifies: one token (the smallest) survives
    assert S.m2po_mask(old + 5, prox, allm, 0.0).tolist() == [False, False, False, False, True]


def test_distillation_loss_against_scalar_definitions():
    """No test of the reference covers actor.py:482-511, so the restatement is pinned by what the formulas fix:
    scalar Python loops over the definitions, special cases with a closed form, and central differences for the
    gradients (with the reward of the pure form held fixed, as `.detach()` there prescribes)."""
    rng = np.random.default_rng(3)
    n = 23
    lp = rng.normal(-1.5, 0.7, n)
    old = lp + rng.normal(0, 0.2, n)
    teacher = lp + rng.normal(0, 0.5, n)
    mask = rng.random(n) < 0.6
    cnt = max(int(mask.sum()), 1)
    t = lambda a: torch.tensor(a, dtype=torch.float64)
    base = torch.tensor(0.37, dtype=torch.float64)

    # joint form: rl_w * loss + kd_w * mean over valid tokens of (logp - teacher)
    want = 0.8 * 0.37 + 0.01 * sum((lp[i] - teacher[i]) for i in range(n) if mask[i]) / cnt
    x = t(lp).requires_grad_(True)
    loss, stat = S.distillation_loss(base, x, t(old), t(teacher), torch.tensor(mask), 0.8, 0.01)
    assert abs(float(loss.detach()) - want) < 1e-12
    loss.backward()
    assert torch.allclose(x.grad, t(np.where(mask, 0.01 / cnt, 0.0)), atol=1e-15)   # constant gradient per valid token
    assert torch.allclose(stat.detach(), t(np.where(mask, lp - teacher, 0.0)))
    # student == teacher: the penalty vanishes
    loss0, _ = S.distillation_loss(base, t(teacher), t(old), t(teacher), torch.tensor(mask), 0.8, 0.01)
    assert abs(float(loss0) - 0.8 * 0.37) < 1e-15

    # pure form: -kd_w * mean over valid tokens of exp(logp - old) * (teacher - logp), the RL loss dropped
    def pure(lp_w, lp_r):  # importance weight from lp_w, reward from lp_r
        return -0.01 * sum(math.exp(lp_w[i] - old[i]) * (teacher[i] - lp_r[i]) for i in range(n) if mask[i]) / cnt
    x = t(lp).requires_grad_(True)
    loss, stat = S.distillation_loss(base, x, t(old), t(teacher), torch.tensor(mask), 0, 0.01)
    assert abs(float(loss.detach()) - pure(lp, lp)) < 1e-12
    loss.backward()
    for i in range(n):
        up, dn = lp.copy(), lp.copy()
        up[i] += 1e-6
        dn[i] -= 1e-6
        fd = (pure(up, lp) - pure(dn, lp)) / 2e-6            # the reward does not move
        assert abs(float(x.grad[i]) - fd) < 1e-8
    assert torch.allclose(stat.detach(), t(np.where(mask, -np.exp(lp - old) * (teacher - lp), 0.0)))
    # on-policy (logp == old): importance weights are 1, the loss is -kd_w * mean(teacher - logp)
    loss1, _ = S.distillation_loss(base, t(old), t(old), t(teacher), torch.tensor(mask), 0, 0.01)
    assert abs(float(loss1) + 0.01 * float((teacher - old)[mask].sum()) / cnt) < 1e-12
    # an all-masked batch divides by 1
    lossm, _ = S.distillation_loss(base, t(lp), t(old), t(teacher), torch.zeros(n, dtype=torch.bool), 0, 0.01)
    assert float(lossm) == 0.0


def test_proximal_logging_tensors_hand_cases():
    """No test of the reference checks the values logged under compute_logp / version_stats (tests/test_prox_approx.py
    :795-935 checks which names appear); the values are pinned by hand arithmetic and the names by those tests."""
    ln2 = math.log(2.0)
    old = torch.tensor([-1.0, -2.0, -1.0, -3.0])
    new = torch.tensor([-1.0 + ln2, -2.0, -1.5, -3.0])
    gt = torch.tensor([-1.0, -1.5, -1.25, -3.0])
    ver = torch.tensor([3, 4, 2, -1], dtype=torch.int32)       # current 5: alpha = 1/2, 0, 2/3, 0 (prompt)
    mask = torch.tensor([True, True, True, False])
    # recompute: ground truth and the KL estimators only
    out, stale = S.proximal_logging_tensors(old, new, gt, ver, 5, mask, "recompute")
    assert sorted(out) == ["kl_div_direct", "kl_div_dual", "kl_div_taylor", "prox_logp_gt"]
    assert torch.allclose(out["kl_div_direct"], torch.tensor([-ln2, 0.0, 0.5, 0.0]))
    assert torch.allclose(out["kl_div_taylor"], torch.tensor([ln2 * ln2 / 2, 0.0, 0.125, 0.0]))
    assert torch.allclose(out["kl_div_dual"], torch.tensor([2 - 1 - ln2, 0.0, math.exp(-0.5) - 1 + 0.5, 0.0]))
    assert stale["sample_staleness_proximal"].tolist() == [1.0, 0.0, 2.0]
    assert stale["sample_staleness_theta"].tolist() == [2.0, 1.0, 3.0]
    # no versions: the reference returns before the estimators
    out, stale = S.proximal_logging_tensors(old, new, gt, None, 5, mask, "metrics")
    assert list(out) == ["prox_logp_gt"] and stale == {}
    out, stale = S.proximal_logging_tensors(old, new, None, ver, None, mask, "loglinear")
    assert out == {} and stale == {}
    # loglinear: three tensors, no error metrics (tests/test_prox_approx.py:795-817)
    out, _ = S.proximal_logging_tensors(old, new, None, ver, 5, mask, "loglinear")
    assert sorted(k for k in out if "/" in k) == ["loglinear/approx_logp", "loglinear/behave_imp_weight",
                                                  "loglinear/importance_weight"]
    approx = torch.tensor([-1.0 + ln2 / 2, -2.0, -1.0 - 0.5 * 2 / 3, -3.0])
    assert torch.allclose(out["loglinear/approx_logp"], approx)
    assert torch.allclose(out["loglinear/behave_imp_weight"], torch.tensor([math.sqrt(2.0), 1.0, math.exp(-1 / 3), 1.0]))
    assert torch.allclose(out["loglinear/importance_weight"], torch.tensor([math.sqrt(2.0), 1.0, math.exp(-1 / 6), 1.0]))
    # metrics with ground truth: every method with all ten names (tests/test_prox_approx.py:905-935)
    out, _ = S.proximal_logging_tensors(old, new, gt, ver, 5, mask, "metrics")
    for method in ("loglinear", "linear", "rollout"):
        for key in ("approx_logp", "behave_imp_weight", "importance_weight", "abs_error", "rel_error", "squared_error",
                    "behave_imp_weight_abs_error", "behave_imp_weight_rel_error", "importance_weight_abs_error",
                    "importance_weight_rel_error"):
            assert f"{method}/{key}" in out
    # rollout approximates by the behaviour log-prob: errors are those of old against the ground truth
    assert torch.allclose(out["rollout/abs_error"], torch.tensor([0.0, 0.5, 0.25, 0.0]))
    assert torch.allclose(out["rollout/rel_error"], torch.tensor([0.0, 0.5 / 1.5, 0.25 / 1.25, 0.0]), atol=1e-7)
    assert torch.allclose(out["rollout/squared_error"], torch.tensor([0.0, 0.25, 0.0625, 0.0]))
    # behave weight: truth exp(gt - old), approximation 1
    want = torch.tensor([0.0, math.exp(0.5) - 1, 1 - math.exp(-0.25), 0.0])
    assert torch.allclose(out["rollout/behave_imp_weight_abs_error"], want, atol=1e-7)
    assert torch.allclose(out["rollout/behave_imp_weight_rel_error"],
                          want / torch.tensor([1.0, math.exp(0.5), math.exp(-0.25), 1.0]), atol=1e-6)
    # importance weight: truth exp(new - gt), approximation exp(new - old)
    t = torch.tensor([2.0, math.exp(-0.5), math.exp(-0.25), 1.0])
    a = torch.tensor([2.0, 1.0, math.exp(-0.5), 1.0])
    assert torch.allclose(out["rollout/importance_weight_abs_error"], (t - a).abs(), atol=1e-6)
    # nothing generated under the mask: no staleness
    _, stale = S.proximal_logging_tensors(old, new, gt, ver, 5, torch.tensor([False, False, False, True]), "recompute")
    assert stale == {}
