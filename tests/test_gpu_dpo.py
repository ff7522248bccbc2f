"""GPU parity of the DPO ops (per-sequence fp64 sums under the shifted mask, the preference loss, the whole loss and
its gradient) against the CPU oracle, and the cases of the reference's own tests (tests/test_dpo.py) run through the
library."""
import math

import pytest
import torch

import areal_amd
from areal_amd import engine_glue as G
from helpers import cosine
from oracle import dpo as D

pytestmark = pytest.mark.gpu
LOG2 = math.log(2.0)


def _batch(lens, seed, p_mask=0.6):
    g = torch.Generator().manual_seed(seed)
    cu = torch.tensor([0] + lens, dtype=torch.int64).cumsum(0).to(torch.int32)
    T = int(cu[-1])
    lp = -torch.rand(T, generator=g) * 3
    ref = lp + 0.3 * torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < p_mask
    return lp, ref, cu, mask


LENS = {
    "small": [7, 3, 0, 5, 1, 4, 6, 2, 9, 0],
    "one_long_pair": [5000, 3111],
    "ragged": [1, 1, 300, 2, 0, 0, 257, 256, 255, 1024, 33, 2048],
}


@pytest.mark.parametrize("name", list(LENS))
def test_pair_logratios_match_oracle(device, name):
    lp, ref, cu, mask = _batch(LENS[name], 5)
    valid = D.valid_pairs(cu.long())
    want = D.pair_logratios(lp, ref, cu, mask, valid)
    got = areal_amd.dpo_pair_logratios(lp.to(device), ref.to(device), cu.to(device), mask.to(device), valid.to(device))
    for g, w in zip(got[:2], want[:2]):
        assert g.dtype == torch.float64 and g.shape == w.shape
        # fp64 sums of the same fp32 values in another order
        assert torch.allclose(g.cpu(), w, rtol=1e-13, atol=1e-11)
    assert torch.equal(got[2].cpu(), want[2])


@pytest.mark.parametrize("loss_type", ["sigmoid", "ipo"])
@pytest.mark.parametrize("name", list(LENS))
def test_dpo_loss_and_gradient_match_oracle(device, name, loss_type):
    lp, ref, cu, mask = _batch(LENS[name], 9)
    beta = 0.1 if name == "one_long_pair" and loss_type == "sigmoid" else 0.4
    x = lp.clone().requires_grad_(True)
    w_loss, w_stat = D.compute_dpo_loss(x, ref, cu, mask, beta, loss_type)
    (3.0 * w_loss).backward()
    y = lp.to(device).requires_grad_(True)
    loss, stat = areal_amd.dpo_loss(y, ref.to(device), cu.to(device), mask.to(device), beta=beta, loss_type=loss_type)
    (3.0 * loss).backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=2e-6, abs=1e-7)
    valid = stat["valid_pairs"].cpu()
    assert torch.equal(valid, w_stat["valid_pairs"]) and int(stat["n_pairs"]) == int(valid.sum())
    for k in ("loss", "chosen_reward", "rejected_reward"):
        assert torch.allclose(stat[k].cpu()[valid], w_stat[k], rtol=2e-6, atol=1e-6), k
        assert not stat[k].cpu()[~valid].any()
    assert torch.allclose(y.grad.cpu(), x.grad, rtol=1e-5, atol=1e-9) and cosine(y.grad.cpu(), x.grad) > 0.999999
    # the composition of the two mirrored functions, as the reference's loss function composes them, gives the same
    z = lp.to(device).requires_grad_(True)
    vp = valid.to(device)
    pol, rf, ln = areal_amd.dpo_pair_logratios(z, ref.to(device), cu.to(device), mask.to(device), vp)
    if loss_type == "ipo":
        logits = (pol[:, 0] - rf[:, 0]) / ln[:, 0].clamp(min=1) - (pol[:, 1] - rf[:, 1]) / ln[:, 1].clamp(min=1)
    else:
        logits = (pol[:, 0] - pol[:, 1]) - (rf[:, 0] - rf[:, 1])
    per_pair = areal_amd.dpo_preference_loss(logits, beta=beta, loss_type=loss_type)
    assert per_pair.dtype == torch.float32
    (3.0 * per_pair.mean()).backward()
    assert float(per_pair.detach().mean()) == pytest.approx(float(loss.detach()), rel=2e-6, abs=1e-7)
    assert torch.allclose(z.grad, y.grad, rtol=1e-5, atol=1e-9)


def test_preference_loss_values_and_gradient(device):
    x = torch.tensor([0.0, 3.0, -3.0, 200.0, -200.0, 1e-4, 17.5, -88.0], dtype=torch.float64)
    for lt, beta in (("sigmoid", 0.5), ("sigmoid", 2.0), ("ipo", 0.25)):
        a = x.clone().requires_grad_(True)
        want = D.preference_loss(a, beta, lt)
        want.sum().backward()
        b = x.to(device).requires_grad_(True)
        got = areal_amd.dpo_preference_loss(b, beta=beta, loss_type=lt)
        got.sum().backward()
        assert got.dtype == torch.float32
        assert torch.allclose(got.detach().cpu(), want.detach(), rtol=1e-6, atol=1e-30), (lt, beta)
        assert b.grad.dtype == torch.float64 and torch.allclose(b.grad.cpu(), a.grad, rtol=1e-6, atol=1e-30)
    with pytest.raises(ValueError, match="Unsupported DPO loss_type"):
        areal_amd.dpo_preference_loss(x.to(device), beta=0.1, loss_type="hinge")


def _glue(device, lp, ref, cu, mask, beta, loss_type="sigmoid"):
    t = lambda a, dt: torch.tensor(a, dtype=dt, device=device)
    inp = {"cu_seqlens": t(cu, torch.int32), "loss_mask": t(mask, torch.bool), "ref_logprobs": t(ref, torch.float32)}
    loss, stat = G.compute_dpo_loss(t(lp, torch.float32), None, inp, beta=beta, loss_type=loss_type)
    return float(loss), stat


def test_reference_cases_through_the_loss_function(device):
    """The known answers of tests/test_dpo.py (shift alignment :232-347, ordering :58-133, masking :151-190, empty
    batch :135-149, IPO :400-518, helper functions :205-226)."""
    cu, ones, zeros = [0, 4, 8], [1] * 8, [0.0] * 8
    loss, _ = _glue(device, [100.0, 0, 0, 0, 100.0, 0, 0, 0], zeros, cu, [0, 0, 1, 1, 0, 0, 0, 1], 0.1)
    assert abs(loss - LOG2) < 1e-5
    loss, _ = _glue(device, [0.0, 0.0, 0.0, 1e6] * 2, zeros, cu, ones, 0.1)
    assert abs(loss - LOG2) < 1e-5
    loss, _ = _glue(device, [0.0, 0.0, -1.0, -2.0, -3.0] * 4, [0.0] * 20, [0, 5, 10, 15, 20], [0, 0, 1, 1, 1] * 4, 0.5)
    assert abs(loss - LOG2) < 1e-5
    good, st = _glue(device, [-0.1] * 4 + [-5.0] * 4, zeros, cu, ones, 0.1)
    bad, _ = _glue(device, [-5.0] * 4 + [-0.1] * 4, zeros, cu, ones, 0.1)
    assert good < bad and st["reward_accuracy"].tolist() == [1.0]
    assert st["reward_margin"].item() == pytest.approx(0.1 * 3 * 4.9, rel=1e-6)
    lp = [-1.0] * 4 + [-2.0] * 4
    same, _ = _glue(device, lp, lp, cu, ones, 0.1)
    opp, _ = _glue(device, lp, [-2.0] * 4 + [-1.0] * 4, cu, ones, 0.1)
    assert abs(same - LOG2) < 1e-6 and opp < same
    mask = [0, 0, 0, 0, 1, 1, 0, 0, 0, 0, 1, 1]
    a, _ = _glue(device, [-10.0] * 4 + [-1.0] * 2 + [-10.0] * 4 + [-2.0] * 2, [0.0] * 12, [0, 6, 12], mask, 0.1)
    b, _ = _glue(device, [-0.1] * 4 + [-1.0] * 2 + [-0.1] * 4 + [-2.0] * 2, [0.0] * 12, [0, 6, 12], mask, 0.1)
    assert abs(a - b) < 1e-5
    for lt in ("sigmoid", "ipo"):
        loss, st = _glue(device, [], [], [0, 0, 0], [], 0.1, lt)
        assert loss == 0.0 and int(st["n_pairs"]) == 0
    # IPO
    loss, _ = _glue(device, [5.0] * 3 + [0.0] * 5, zeros, cu, ones, 0.1, "ipo")
    assert abs(loss) < 1e-4
    a, _ = _glue(device, [-1.0] * 3 + [0.0] + [-2.0] * 3 + [0.0], zeros, cu, ones, 0.1, "ipo")
    b, _ = _glue(device, [-1.0] * 7 + [0.0] + [-2.0] * 7 + [0.0], [0.0] * 16, [0, 8, 16], [1] * 16, 0.1, "ipo")
    assert abs(a - b) < 1e-5 and abs(a - 16.0) < 1e-4
    with pytest.raises(ValueError, match="Unsupported DPO loss_type"):
        _glue(device, zeros, zeros, cu, ones, 0.1, "nonexistent")
    with pytest.raises(KeyError):
        G.compute_dpo_loss(torch.zeros(8, device=device), None,
                           {"cu_seqlens": torch.tensor(cu), "loss_mask": torch.ones(8, dtype=torch.bool)}, beta=0.1)
    x = {"cu_seqlens": torch.tensor([0, 5, 10, 15, 15], dtype=torch.int32, device=device)}
    assert G.dpo_valid_pairs(x).tolist() == [True, False] and float(G.dpo_loss_weight(x)) == 1.0
    # backward through the loss function on a leaf (:349-367, :488-497)
    for lt in ("sigmoid", "ipo"):
        leaf = torch.randn(8, device=device, requires_grad=True)
        inp = {"cu_seqlens": torch.tensor(cu, device=device), "loss_mask": torch.ones(8, dtype=torch.bool, device=device),
               "ref_logprobs": torch.zeros(8, device=device)}
        loss, _ = G.compute_dpo_loss(leaf, None, inp, beta=0.1, loss_type=lt)
        loss.backward()
        assert torch.isfinite(leaf.grad).all() and leaf.grad[3] == 0 and leaf.grad[7] == 0


def test_long_sequences_keep_fp64_accuracy(device):
    """Two 60 000-token sequences whose sums differ by far less than an fp32 sum's error (the case the reference
    gives for its fp64 accumulation, functional.py:655-657): the pair's logit must keep the sign."""
    L = 60000
    g = torch.Generator().manual_seed(2)
    base = -torch.rand(L, generator=g) * 8 - 0.5
    chosen, rejected = base.clone(), base.clone()
    chosen[100] += 1e-3                       # chosen ahead by 1e-3 in a sum of about -270 000
    lp = torch.cat([chosen, rejected])
    ref = torch.cat([base, base])
    cu = torch.tensor([0, L, 2 * L], dtype=torch.int32)
    mask = torch.ones(2 * L, dtype=torch.bool)
    w_loss, w_stat = D.compute_dpo_loss(lp, ref, cu, mask, 1.0)
    loss, stat = areal_amd.dpo_loss(lp.to(device), ref.to(device), cu.to(device), mask.to(device), beta=1.0)
    exact = float(chosen[100].double() - base[100].double())
    assert stat["chosen_reward"].item() == pytest.approx(exact, rel=1e-6) and stat["rejected_reward"].item() == 0.0
    assert float(loss) == pytest.approx(float(w_loss), rel=1e-6) and float(loss) < LOG2


@pytest.mark.parametrize("name", list(LENS))
def test_reward_model_loss_matches_oracle(device, name):
    lens = LENS[name]
    g = torch.Generator().manual_seed(4)
    cu = torch.tensor([0] + lens, dtype=torch.int64).cumsum(0)
    T = int(cu[-1])
    scores = torch.randn(T, generator=g) * 2
    x = scores.clone().requires_grad_(True)
    w_loss, w_stat = D.compute_rw_loss(x, cu)
    (1.7 * w_loss).backward()
    y = scores.to(device).requires_grad_(True)
    loss, stat = G.compute_rw_loss(y, {"cu_seqlens": cu.to(torch.int32).to(device)})
    (1.7 * loss).backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=2e-6)
    valid = stat["valid_pairs"].cpu()
    assert torch.equal(valid, w_stat["valid_pairs"]) and int(stat["n_pairs"]) == int(valid.sum())
    for k in ("loss", "pos_score", "neg_score", "correct_ratio"):
        assert torch.allclose(stat[k].cpu()[valid], w_stat[k], rtol=2e-6, atol=1e-7), k
    assert torch.allclose(y.grad.cpu(), x.grad, rtol=1e-5, atol=1e-9)
    assert int((y.grad != 0).sum()) == 2 * int(valid.sum())


def test_reward_model_loss_reference_cases(device):
    """tests/test_eval_dispatch.py:325-371."""
    inp = {"cu_seqlens": torch.tensor([0, 5, 9, 9, 9], dtype=torch.int32, device=device)}
    scores = torch.tensor([0.0, 0.0, 0.0, 0.0, 3.0, 0.0, 0.0, 0.0, 1.0], device=device)
    loss, stat = G.compute_rw_loss(scores, inp)
    assert float(loss) == pytest.approx(math.log1p(math.exp(-2.0)), rel=1e-5)
    assert int(stat["n_pairs"]) == 1 and float(G.rw_loss_weight(inp)) == 1.0
    assert stat["pos_score"].tolist() == [3.0, 0.0] and stat["neg_score"].tolist() == [1.0, 0.0]
    assert stat["correct_ratio"].tolist() == [1.0, 0.0]
    loss, stat = G.compute_rw_loss(torch.zeros(0, device=device),
                                   {"cu_seqlens": torch.tensor([0, 0, 0], dtype=torch.int32, device=device)})
    assert float(loss) == 0.0 and int(stat["n_pairs"]) == 0
    # bf16 scores, as a value head emits them
    s16 = torch.randn(9, device=device).bfloat16().requires_grad_(True)
    loss, _ = G.compute_rw_loss(s16, inp)
    loss.backward()
    assert s16.grad.dtype == torch.bfloat16 and int((s16.grad != 0).sum()) == 2
