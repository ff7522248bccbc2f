"""Pins of the advantage-pipeline oracle (oracle/advantages.py): the reference's own known-answer cases for
Normalization (transcribed as data), numpy closed forms, a brute-force leave-one-out, and for GAE (which the
reference has no test for) the textbook double sum on the compressed sequence of unmasked tokens."""
import json
import math
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import advantages as O

GOLD = json.loads((Path(__file__).parent / "golden" / "reference_norm_known_answers.json").read_text())


def _case_tensors(c):
    x = torch.tensor(c["x"], dtype=torch.float32)
    mask = torch.ones_like(x) if c["mask"] == "ones" else torch.tensor(c["mask"], dtype=torch.float32)
    return x, mask


@pytest.mark.parametrize("c", GOLD["cases"], ids=[c["name"] for c in GOLD["cases"]])
def test_normalization_reference_known_answers(c):
    x, mask = _case_tensors(c)
    out = O.normalization(x, mask, **c["cfg"])
    assert out.dtype == torch.float32 and out.shape == x.shape
    atol = c.get("atol", 1e-6)
    if "expected" in c:
        assert torch.allclose(out, torch.tensor(c["expected"], dtype=torch.float32), atol=atol)
    for key, val in c.get("expected_at", {}).items():
        i, j = (int(t) for t in key.split(","))
        assert abs(float(out[i, j]) - val) <= atol, (key, float(out[i, j]), val)
    p = c.get("properties", {})
    if "mean_abs_below" in p:
        assert abs(float(out.mean())) < p["mean_abs_below"]
    if "nonmasked_mean_abs_below" in p:
        nm = out[mask.bool()]
        assert abs(float(nm.mean())) < p["nonmasked_mean_abs_below"]
        assert abs(float(nm.std()) - 1.0) < p["nonmasked_unbiased_std_minus_one_abs_below"]


def test_normalization_unbiased_ratio():
    # tests/test_adv_norm_config.py:708-737: ratio of spreads = sqrt(n / (n - 1))
    x = torch.tensor([[1.0], [2.0], [3.0]])
    b = O.normalization(x, torch.ones_like(x), std_unbiased=False)
    u = O.normalization(x, torch.ones_like(x), std_unbiased=True)
    assert abs(float(b.std() / u.std()) - math.sqrt(1.5)) < 1e-4


@pytest.mark.parametrize("unbiased", [False, True])
def test_normalization_matches_numpy_closed_forms(unbiased):
    rng = np.random.default_rng(0)
    x = rng.normal(size=(12, 7)).astype(np.float32)
    m = (rng.random((12, 7)) < 0.6).astype(np.float32)
    ddof = 1 if unbiased else 0
    # batch level
    sel = x[m > 0].astype(np.float64)
    want = (x - sel.mean()) * m / (sel.std(ddof=ddof) + 1e-5)
    got = O.normalization(torch.tensor(x), torch.tensor(m), std_unbiased=unbiased)
    assert np.allclose(got.numpy(), want, atol=2e-6)
    # group level, groups of 3 rows
    want = np.zeros_like(x, dtype=np.float64)
    for g in range(4):
        s = slice(3 * g, 3 * g + 3)
        sel = x[s][m[s] > 0].astype(np.float64)
        want[s] = (x[s] - sel.mean()) * m[s] / (sel.std(ddof=ddof) + 1e-5)
    got = O.normalization(torch.tensor(x), torch.tensor(m), mean_level="group", std_level="group", group_size=3,
                          std_unbiased=unbiased)
    assert np.allclose(got.numpy(), want, atol=5e-6)
    # no mask
    want = (x - x.astype(np.float64).mean()) / (x.astype(np.float64).std(ddof=ddof) + 1e-5)
    got = O.normalization(torch.tensor(x), None, std_unbiased=unbiased)
    assert np.allclose(got.numpy(), want, atol=2e-6)


def test_normalization_leave_one_out_brute_force_and_leftover_rows():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(7, 5)).astype(np.float32)
    m = (rng.random((7, 5)) < 0.7).astype(np.float32)
    got = O.normalization(torch.tensor(x), torch.tensor(m), mean_level="group", std_level=None, group_size=3,
                          mean_leave1out=True).numpy()
    for g in range(2):
        rows = range(3 * g, 3 * g + 3)
        idx = [(i, j) for i in rows for j in range(5) if m[i, j] > 0]
        for (i, j) in idx:
            others = [x[a, b] for (a, b) in idx if (a, b) != (i, j)]
            assert abs(got[i, j] - (x[i, j] - np.mean(others))) < 1e-5
    # the row past the last full group keeps mean 0 and (std none) scale 1: x * mask
    assert np.allclose(got[6], x[6] * m[6], atol=1e-7)
    # with a group-level std the leftover row is divided by eps alone
    got = O.normalization(torch.tensor(x), torch.tensor(m), mean_level=None, std_level="group", group_size=3,
                          eps=1e-5).numpy()
    assert np.allclose(got[6], x[6] * m[6] / np.float32(1e-5), rtol=1e-6)


def test_normalization_all_masked_returns_input():
    x = torch.randn(4, 3)
    assert torch.equal(O.normalization(x, torch.zeros_like(x)), x)


# ---------------------------------------------------------------------------------------------------------------
def _gae_textbook(r, v, m, no_eos, gamma, lam):
    """Advantages at the unmasked tokens t <= L-2 from the definition sum_k (gamma lam)^k delta_k over the compressed
    sequence of unmasked tokens (a token's successor value is the value of the next unmasked token, or
    v[L-1] * no_eos after the last one)."""
    L = len(r)
    idx = [t for t in range(L - 1) if m[t] > 0]
    out = {}
    deltas = []
    for k, t in enumerate(idx):
        nxt = v[idx[k + 1]] if k + 1 < len(idx) else v[L - 1] * no_eos
        deltas.append(r[t] + gamma * nxt - v[t])
    for k, t in enumerate(idx):
        out[t] = sum((gamma * lam) ** (j - k) * deltas[j] for j in range(k, len(idx)))
    return out


@pytest.mark.parametrize("gamma,lam", [(1.0, 1.0), (0.99, 0.95), (0.9, 0.0)])
def test_gae_against_textbook_definition(gamma, lam):
    rng = np.random.default_rng(3)
    bs, L = 5, 23
    r = rng.normal(size=(bs, L))
    v = rng.normal(size=(bs, L))
    m = (rng.random((bs, L)) < 0.6).astype(np.float64)
    no_eos = np.array([1, 0, 1, 0, 1], dtype=np.float64)
    adv, ret = O.gae(torch.tensor(r), torch.tensor(v), torch.tensor(m), torch.tensor(no_eos), gamma, lam)
    assert float(adv[:, L - 1].abs().max()) == 0.0
    assert torch.allclose(ret, adv + torch.tensor(v))
    for b in range(bs):
        want = _gae_textbook(r[b], v[b], m[b], no_eos[b], gamma, lam)
        carried = 0.0
        for t in reversed(range(L - 1)):
            if t in want:
                carried = want[t]
            assert abs(float(adv[b, t]) - carried) < 1e-9, (b, t)  # masked tokens repeat the value to their right


def test_gae_special_cases():
    L = 9
    r = torch.arange(1.0, L + 1).reshape(1, L)
    z = torch.zeros(1, L)
    ones = torch.ones(1, L)
    # no values, gamma = lambda = 1: reverse cumulative sum of the rewards up to L-2
    adv, _ = O.gae(r, z, ones, torch.zeros(1), 1.0, 1.0)
    want = torch.flip(torch.cumsum(torch.flip(r[:, : L - 1], [1]), 1), [1])
    assert torch.allclose(adv[:, : L - 1], want)
    # lambda = 0: one-step TD residual
    v = torch.linspace(-1, 1, L).reshape(1, L)
    adv, _ = O.gae(r, v, ones, torch.ones(1), 0.9, 0.0)
    assert torch.allclose(adv[:, : L - 1], r[:, : L - 1] + 0.9 * v[:, 1:] - v[:, : L - 1], atol=1e-6)


def test_masked_moments_against_numpy():
    rng = np.random.default_rng(5)
    vals = [torch.tensor(rng.normal(size=50).astype(np.float32)) for _ in range(3)]
    mask = torch.tensor(rng.random(50) < 0.5)
    out = O.masked_moments(vals, mask)
    for k, v in enumerate(vals):
        sel = v.numpy()[mask.numpy()]
        assert np.allclose(out[k].numpy(), [sel.sum(), sel.min(), sel.max(), len(sel)], rtol=1e-6)
    empty = O.masked_moments(vals[:1], torch.zeros(50, dtype=torch.bool))
    assert float(empty[0, 0]) == 0.0 and math.isinf(float(empty[0, 1])) and float(empty[0, 3]) == 0.0


def test_kl_rewards_hand_case():
    # two sequences of a padded [2, 5] batch: lengths 4 and 5 (the second fills the row: no EOS seen)
    old = torch.tensor([[-1.0, -2.0, -3.0, -4.0, 0.0], [-1.0, -1.0, -1.0, -1.0, -1.0]])
    ref = torch.tensor([[-1.5, -2.0, -2.0, -4.0, 0.0], [-1.0, -2.0, -1.0, -1.0, -3.0]])
    mask = torch.ones(2, 5)
    seqlens = torch.tensor([4, 5])
    score = torch.tensor([2.0, -1.0])
    rewards, kl = O.kl_rewards(old, ref, mask, seqlens, score, kl_ctl=0.1)
    assert torch.allclose(kl, -0.1 * (old - ref))                                  # k1: the plain difference
    want = kl.clone()
    want[0, 3] = 0.0
    want[0, 2] += 2.0          # score one step before the last token
    want[1, 4] = 0.0
    want[1, 3] += -1.0
    assert torch.allclose(rewards, want)
    rewards, _ = O.kl_rewards(old, ref, mask, seqlens, score, kl_ctl=0.1, mask_no_eos_with_zero=True)
    want[1, 3] -= -1.0         # the sequence that fills the row gets no score
    assert torch.allclose(rewards, want)
    # k2 and the clamp at 10
    _, kl2 = O.kl_rewards(old * 10, ref, mask, seqlens, score, kl_ctl=1.0, kl_estimator="k2")
    d = old * 10 - ref
    assert torch.allclose(kl2, -(d * d / 2).clamp(max=10.0))


def test_compute_advantages_grpo_shape_by_hand():
    # no critic, no KL, gamma = lambda = 1: every unmasked token before the score gets the (clipped, scaled) score
    bs, L = 2, 6
    am = torch.tensor([[1, 1, 1, 1, 1, 0], [1, 1, 1, 0, 0, 0]])
    lm = torch.tensor([[0, 0, 1, 1, 1, 0], [0, 1, 1, 0, 0, 0]])
    logprobs_in = -torch.rand(bs, L)
    data = dict(input_ids=torch.zeros(bs, L, dtype=torch.long), attention_mask=am, loss_mask=lm,
                logprobs=logprobs_in.clone(), rewards=torch.tensor([30.0, -0.5]))
    out = O.compute_advantages(data, reward_scaling=0.5, reward_clip=5.0)
    rolled = torch.roll(lm.float(), -1, -1)
    assert torch.equal(out["loss_mask"], rolled)
    # sequence 0: score min(30 * 0.5, 5) = 5 placed at position 3; rolled mask = positions 1, 2, 3
    assert out["advantages"][0].tolist() == [5.0, 5.0, 5.0, 5.0, 0.0, 0.0]
    # sequence 1: score -0.25 at position 1; rolled mask = positions 0, 1
    assert out["advantages"][1].tolist() == [-0.25, -0.25, 0.0, 0.0, 0.0, 0.0]
    assert torch.equal(out["returns"], out["advantages"]) and torch.equal(out["tot_rewards"][0, 3], torch.tensor(5.0))
    # the reference multiplies old_logp by the rolled mask in place (actor.py:195) after storing that same tensor as
    # data["prox_logp"] (:191): both come out masked
    assert torch.equal(out["prox_logp"], torch.roll(logprobs_in, -1, -1) * rolled)
    assert out["prox_logp"] is out["logprobs"]


def test_overlong_penalty_hand_cases():
    """functional.py:782-803 has no test in the reference; the restatement is pinned by hand-computed cases of the
    DAPO length penalty: nothing up to max_len - overlong tokens, then a linear ramp of factor per overlong tokens."""
    L = 12
    lens = [3, 6, 7, 9, 12]                     # max_len 10, overlong 4: expected length 6
    mask = torch.tensor([[1.0] * n + [0.0] * (L - n) for n in lens])
    data = dict(rewards=torch.tensor([1.0, 1.0, 1.0, -2.0, 0.5]), loss_mask=mask, input_ids=torch.zeros(5, L))
    out = O.overlong_penalty(data, overlong_tokens=4, overlong_penalty_factor=2.0, max_response_length=10)
    # excess 0, 0, 1, 3, 6 tokens -> penalty 0, 0, 0.5, 1.5, 3.0
    assert torch.allclose(out["rewards"], torch.tensor([1.0, 1.0, 0.5, -3.5, -2.5]))


def test_masked_normalization_against_numpy_moments():
    """No test of the reference covers functional.py:16-53; pinned by numpy's mean / std (with and without Bessel's
    correction) over the selection, by hand values, and by the fate of masked positions (whitened as zeros)."""
    from oracle.advantages import masked_normalization

    rng = np.random.default_rng(4)
    x = rng.normal(2.0, 3.0, (6, 50))
    t = torch.tensor(x)
    # no mask, all axes: numpy mean and population / sample std
    for unbiased, ddof in ((False, 0), (True, 1)):
        got = masked_normalization(t, None, None, unbiased, 1e-5).numpy()
        want = (x - x.mean()) / (x.std(ddof=ddof) + 1e-5)
        assert got.dtype == np.float32 and np.allclose(got, want, rtol=1e-6, atol=1e-6)
    # hand value: [1, 2, 3, 4] -> mean 2.5, population std sqrt(1.25)
    got = masked_normalization(torch.tensor([1.0, 2.0, 3.0, 4.0]), eps=0.0).tolist()
    assert np.allclose(got, [(v - 2.5) / math.sqrt(1.25) for v in (1, 2, 3, 4)], rtol=1e-6)
    # mask, per row (dim=1): moments over the selected entries; masked entries are whitened as zeros
    m = rng.random((6, 50)) < 0.6
    got = masked_normalization(t, torch.tensor(m), 1, True, 1e-5).numpy()
    for r in range(6):
        sel = x[r][m[r]]
        mean, std = sel.mean(), sel.std(ddof=1)
        assert np.allclose(got[r][m[r]], (sel - mean) / (std + 1e-5), rtol=1e-5, atol=1e-6)
        assert np.allclose(got[r][~m[r]], (0.0 - mean) / (std + 1e-5), rtol=1e-5, atol=1e-6)
    # a float mask weighs the entries: v = x * w, F = sum(w)
    w = rng.random(50)
    got = masked_normalization(t[0], torch.tensor(w), None, False, 0.0).numpy()
    v = x[0] * w
    mean = v.sum() / w.sum()
    var = (v * v).sum() / w.sum() - mean * mean
    assert np.allclose(got, (v - mean) / math.sqrt(var), rtol=1e-5, atol=1e-6)
