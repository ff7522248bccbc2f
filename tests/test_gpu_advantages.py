"""GPU parity of the advantage pipeline (GAE scan, Normalization, masked moments) against the CPU oracle and the
reference's own known-answer cases."""
import itertools
import json
from pathlib import Path

import pytest
import torch

import areal_amd
from areal_amd import NormConfig, Normalization
from oracle import advantages as O

pytestmark = pytest.mark.gpu

GOLD = json.loads((Path(__file__).parent / "golden" / "reference_norm_known_answers.json").read_text())


@pytest.mark.parametrize("c", GOLD["cases"], ids=[c["name"] for c in GOLD["cases"]])
def test_normalization_reference_known_answers(device, c):
    x = torch.tensor(c["x"], dtype=torch.float32)
    mask = torch.ones_like(x) if c["mask"] == "ones" else torch.tensor(c["mask"], dtype=torch.float32)
    out = Normalization(NormConfig(**c["cfg"]))(x.to(device), mask.to(device)).cpu()
    assert out.dtype == torch.float32 and out.shape == x.shape
    atol = c.get("atol", 1e-6)
    if "expected" in c:
        assert torch.allclose(out, torch.tensor(c["expected"], dtype=torch.float32), atol=atol)
    for key, val in c.get("expected_at", {}).items():
        i, j = (int(t) for t in key.split(","))
        assert abs(float(out[i, j]) - val) <= atol
    p = c.get("properties", {})
    if "mean_abs_below" in p:
        assert abs(float(out.mean())) < p["mean_abs_below"]
    if "nonmasked_mean_abs_below" in p:
        nm = out[mask.bool()]
        assert abs(float(nm.mean())) < p["nonmasked_mean_abs_below"]
        assert abs(float(nm.std()) - 1.0) < p["nonmasked_unbiased_std_minus_one_abs_below"]


LEVELS = [None, "batch", "group"]


@pytest.mark.parametrize("mean_level,std_level", list(itertools.product(LEVELS, LEVELS)))
@pytest.mark.parametrize("loo,unbiased", [(False, True), (True, False), (True, True)])
def test_normalization_matches_oracle(device, mean_level, std_level, loo, unbiased):
    g = torch.Generator().manual_seed(hash((str(mean_level), str(std_level), loo, unbiased)) % 1000)
    for shape, gs, with_mask in [((14, 37), 4, True), ((12, 5), 3, False), ((9,), 2, False), ((6, 3, 4), 1, True),
                                 ((5, 8), 8, True)]:
        x = torch.randn(*shape, generator=g) * 2.0 + 0.5
        mask = (torch.rand(*shape, generator=g) < 0.6).float() if with_mask else None
        cfg = dict(mean_level=mean_level, mean_leave1out=loo, std_level=std_level, std_unbiased=unbiased, eps=1e-5,
                   group_size=gs)
        want = O.normalization(x, mask, **cfg)
        got = Normalization(NormConfig(**cfg))(x.to(device), None if mask is None else mask.to(device)).cpu()
        assert got.shape == want.shape and got.dtype == torch.float32
        scale = float(want.abs().max()) + 1.0
        assert float((got - want).abs().max()) <= 2e-6 * scale, (shape, gs, cfg)


def test_normalization_edge_cases(device):
    x = torch.randn(4, 6)
    zero = torch.zeros_like(x)
    out = Normalization(NormConfig())(x.to(device), zero.to(device))
    assert torch.equal(out.cpu(), x)  # nothing active: the input comes back
    with pytest.raises(ValueError, match="group_size must be a positive integer"):
        NormConfig(mean_level="group", std_level="batch", group_size=0)
    with pytest.raises(ValueError, match="mean_level must be"):
        NormConfig(mean_level="bad")
    with pytest.raises(areal_amd.NativeLibraryError):
        Normalization(NormConfig())(x)  # CPU tensors are refused
    # bf16 input is accepted and comes back float32
    out = Normalization(NormConfig())(x.bfloat16().to(device))
    assert out.dtype == torch.float32
    assert torch.allclose(out.cpu(), O.normalization(x.bfloat16().float()), atol=1e-5)


def test_normalization_full_size(device):
    bs, L = 512, 4096
    g = torch.Generator().manual_seed(0)
    x = torch.randn(bs, L, generator=g)
    mask = (torch.rand(bs, L, generator=g) < 0.7).float()
    for cfg in (dict(), dict(mean_level="group", std_level="group", group_size=16),
                dict(mean_level="batch", std_level="group", group_size=8, mean_leave1out=True)):
        want = O.normalization(x, mask, **cfg)
        norm = Normalization(NormConfig(**cfg))
        got = norm(x.to(device), mask.to(device))
        assert float((got.cpu() - want).abs().max()) < 1e-5
        assert torch.equal(got, norm(x.to(device), mask.to(device)))  # fixed summation order


@pytest.mark.parametrize("bs,L", [(1, 1), (3, 2), (5, 63), (4, 64), (7, 65), (6, 66), (9, 129), (2, 1000), (3, 4096),
                                   (2, 4097), (2, 4098), (2, 9001), (1, 20000)])
@pytest.mark.parametrize("gamma,lam", [(1.0, 1.0), (0.99, 0.95)])
def test_gae_matches_oracle(device, bs, L, gamma, lam):
    g = torch.Generator().manual_seed(bs * 1000 + L)
    r = torch.randn(bs, L, generator=g)
    v = torch.randn(bs, L, generator=g)
    m = (torch.rand(bs, L, generator=g) < 0.6).float()
    ne = torch.rand(bs, generator=g) < 0.5
    want_a, want_r = O.gae(r.double(), v.double(), m.double(), ne.double(), gamma, lam)
    adv, ret = areal_amd.gae_advantages(r.to(device), v.to(device), m.to(device), ne.to(device), gamma, lam)
    scale = float(want_a.abs().max()) + 1.0
    assert float((adv.cpu().double() - want_a).abs().max()) < 2e-5 * scale
    assert float((ret.cpu().double() - want_r).abs().max()) < 2e-5 * scale
    # the fp32 loop of the reference agrees to the same bar
    ref_a, _ = O.gae(r, v, m, ne.float(), gamma, lam)
    assert float((adv.cpu() - ref_a).abs().max()) < 4e-5 * scale
    # no critic: values = None stands for zeros
    adv0, ret0 = areal_amd.gae_advantages(r.to(device), None, m.to(device), None, gamma, lam)
    want0, _ = O.gae(r.double(), torch.zeros(bs, L).double(), m.double(), torch.zeros(bs).double(), gamma, lam)
    assert float((adv0.cpu().double() - want0).abs().max()) < 2e-5 * (float(want0.abs().max()) + 1.0)
    assert torch.equal(adv0, ret0)


def test_gae_full_size_and_grpo_shape(device):
    bs, L = 512, 4096
    g = torch.Generator().manual_seed(1)
    lens = torch.randint(L // 4, L + 1, (bs,), generator=g)
    pos = torch.arange(L)[None, :]
    m = ((pos >= (lens[:, None] * 0.3).long()) & (pos < lens[:, None] - 1)).float()
    r = torch.zeros(bs, L)
    r[torch.arange(bs), (lens - 2).clamp(min=0)] = torch.randn(bs, generator=g)   # one terminal reward per sequence
    r = r - 0.01 * torch.rand(bs, L, generator=g) * m                             # plus KL penalties
    v = torch.randn(bs, L, generator=g) * 0.1
    ne = lens == L
    want_a, want_r = O.gae(r, v, m, ne.float(), 1.0, 1.0)
    adv, ret = areal_amd.gae_advantages(r.to(device), v.to(device), m.to(device), ne.to(device), 1.0, 1.0)
    assert float((adv.cpu() - want_a).abs().max()) < 1e-4 and float((ret.cpu() - want_r).abs().max()) < 1e-4
    adv2, _ = areal_amd.gae_advantages(r.to(device), v.to(device), m.to(device), ne.to(device), 1.0, 1.0)
    assert torch.equal(adv, adv2)


def test_masked_moments(device):
    g = torch.Generator().manual_seed(2)
    n = 10007
    vals = {f"s{k}": torch.randn(n, generator=g) * (k + 1) for k in range(5)}
    vals["flag"] = (torch.rand(n, generator=g) < 0.3).float()
    mask = torch.rand(n, generator=g) < 0.4
    got = areal_amd.masked_moments({k: v.to(device) for k, v in vals.items()}, mask.to(device))
    want = O.masked_moments(list(vals.values()), mask)
    for i, k in enumerate(vals):
        assert float(got[k]["sum"]) == pytest.approx(float(want[i, 0]), rel=1e-5, abs=1e-4)
        assert float(got[k]["min"]) == float(want[i, 1]) and float(got[k]["max"]) == float(want[i, 2])
        assert float(got[k]["count"]) == float(want[i, 3])
        assert float(got[k]["avg"]) == pytest.approx(float(want[i, 0] / want[i, 3]), rel=1e-5, abs=1e-6)
    empty = areal_amd.masked_moments({"a": vals["s0"].to(device)}, torch.zeros(n, dtype=torch.bool, device=device))
    assert float(empty["a"]["count"]) == 0.0 and float(empty["a"]["min"]) == float("inf")
    with pytest.raises(ValueError):
        areal_amd.masked_moments({"a": vals["s0"][:5].to(device)}, mask.to(device))


@pytest.mark.parametrize("est", ["k1", "k2", "k3"])
@pytest.mark.parametrize("no_eos_zero", [False, True])
def test_kl_rewards_match_oracle(device, est, no_eos_zero):
    g = torch.Generator().manual_seed(11)
    bs, L = 9, 40
    seqlens = torch.tensor([40, 1, 2, 17, 40, 5, 39, 3, 40])
    old, ref = -torch.rand(bs, L, generator=g) * 12, -torch.rand(bs, L, generator=g) * 3
    mask = (torch.rand(bs, L, generator=g) < 0.6).float()
    score = torch.randn(bs, generator=g)
    want_r, want_k = O.kl_rewards(old * mask, ref * mask, mask, seqlens, score, 0.2, est, no_eos_zero)
    r, k = areal_amd.kl_regularized_rewards((old * mask).to(device), (ref * mask).to(device), mask.to(device),
                                            seqlens.to(device), score.to(device), 0.2, est, no_eos_zero)
    assert torch.allclose(k.cpu(), want_k, rtol=1e-5, atol=1e-6) and torch.allclose(r.cpu(), want_r, rtol=1e-5, atol=1e-6)
    r0, _ = areal_amd.kl_regularized_rewards((old * mask).to(device), None, mask.to(device), seqlens.to(device),
                                             score.to(device), 0.2, est, no_eos_zero)
    w0, _ = O.kl_rewards(old * mask, torch.zeros(bs, L), mask, seqlens, score, 0.2, est, no_eos_zero)
    assert torch.allclose(r0.cpu(), w0, rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError, match="Invalid KL estimator"):
        areal_amd.kl_regularized_rewards(old.to(device), None, mask.to(device), seqlens.to(device), score.to(device), 0.1, "k9")


@pytest.mark.parametrize("case", ["grpo", "critic_kl", "recompute", "overlong"])
def test_compute_advantages_matches_oracle(device, case):
    from areal_amd.engine_glue import compute_advantages

    g = torch.Generator().manual_seed(21)
    bs, L = 16, 96
    lens = torch.randint(4, L + 1, (bs,), generator=g)
    lens[0] = L
    pos = torch.arange(L)[None, :]
    am = (pos < lens[:, None]).long()
    lm = ((pos >= (lens[:, None] * 0.4).long()) & (pos < lens[:, None])).long()
    data = dict(input_ids=torch.randint(0, 100, (bs, L), generator=g), attention_mask=am, loss_mask=lm,
                logprobs=-torch.rand(bs, L, generator=g) * 2, rewards=torch.randn(bs, generator=g) * 3)
    if case == "grpo":
        kw = dict(reward_scaling=2.0, reward_bias=-0.5, reward_clip=4.0,
                  reward_norm=dict(mean_level="group", std_level="group", group_size=4),
                  adv_norm=dict(mean_level="batch", std_level="batch"))
    elif case == "critic_kl":
        data["values"] = torch.randn(bs, L, generator=g) * 0.3
        data["ref_logp"] = -torch.rand(bs, L, generator=g) * 2
        kw = dict(kl_ctl=0.1, kl_estimator="k3", discount=0.99, gae_lambda=0.95, mask_no_eos_with_zero=True,
                  use_decoupled_loss=True, adv_norm=dict(mean_level="batch", std_level=None, mean_leave1out=True))
    elif case == "overlong":
        kw = dict(overlong_tokens=16, overlong_penalty_factor=0.7, max_new_tokens=48,
                  adv_norm=dict(mean_level="batch", std_level="batch"))
    else:
        data["prox_logp"] = -torch.rand(bs, L, generator=g) * 2
        kw = dict(recompute_logprob=True, use_decoupled_loss=False)
    want = O.compute_advantages({k: (v.clone() if torch.is_tensor(v) else v) for k, v in data.items()}, **kw)
    gkw = dict(kw)
    for name in ("reward_norm", "adv_norm"):
        if gkw.get(name) is not None:
            gkw[name] = Normalization(NormConfig(**gkw[name]))
    got = compute_advantages({k: (v.to(device) if torch.is_tensor(v) else v) for k, v in data.items()}, **gkw)
    for key in ("advantages", "returns", "kl_rewards", "tot_rewards", "loss_mask", "logprobs"):
        scale = float(want[key].abs().max()) + 1.0
        assert float((got[key].cpu() - want[key]).abs().max()) < 2e-5 * scale, key
    rolled_mask = torch.roll(lm.float(), shifts=-1, dims=-1)
    if case != "critic_kl":
        # the reference masks old_logp in place (actor.py:195), and data["prox_logp"] is that very tensor
        assert torch.allclose(got["prox_logp"].cpu(), want["prox_logp"])
        assert got["prox_logp"] is got["logprobs"]
        assert float((got["prox_logp"].cpu() * (1 - rolled_mask)).abs().max()) == 0.0
    else:
        # ... and data["ref_logp"] likewise (actor.py:194)
        assert torch.equal(want["ref_logp"], data["ref_logp"] * rolled_mask)
        assert torch.equal(got["ref_logp"].cpu(), want["ref_logp"])


def test_overlong_penalty_matches_oracle_and_updates_in_place(device):
    g = torch.Generator().manual_seed(8)
    bs, L = 37, 300
    lens = torch.randint(1, L + 1, (bs,), generator=g)
    mask = (torch.arange(L)[None, :] < lens[:, None]).float()
    rewards = torch.randn(bs, generator=g)
    want = O.overlong_penalty(dict(rewards=rewards.clone(), loss_mask=mask, input_ids=torch.zeros(bs, L)), 40, 1.3, 200)
    r_dev = rewards.to(device)
    data = dict(rewards=r_dev, loss_mask=mask.to(device), input_ids=torch.zeros(bs, L, device=device))
    got = areal_amd.reward_overlong_penalty(data, 40, 1.3, 200)
    assert got["rewards"] is r_dev and torch.equal(r_dev.cpu(), want["rewards"])
    assert bool((want["rewards"] <= rewards).all()) and bool((want["rewards"] < rewards).any())


@pytest.mark.parametrize("shape,dim", [((2_000_003,), None), ((64, 4096), None), ((64, 4096), 1), ((64, 4096), 0),
                                       ((5, 7, 33), (0, 2)), ((3, 1), None), ((1,), None)])
@pytest.mark.parametrize("masked,unbiased", [(False, False), (True, True), (True, False)])
def test_masked_normalization_matches_oracle(device, shape, dim, masked, unbiased):
    g = torch.Generator().manual_seed(13)
    x = torch.randn(shape, generator=g) * 3 + 1.5
    mask = (torch.rand(shape, generator=g) < 0.7) if masked else None
    want = O.masked_normalization(x, mask, dim, unbiased, 1e-5)
    got = areal_amd.masked_normalization(x.to(device), None if mask is None else mask.to(device), dim, unbiased, 1e-5)
    assert got.dtype == torch.float32 and got.shape == x.shape
    # a single value (or a single selected value with Bessel's correction) divides by zero in both
    assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-6, equal_nan=True)


def test_masked_normalization_weights_and_broadcast_mask(device):
    g = torch.Generator().manual_seed(14)
    x = torch.randn(16, 300, generator=g)
    w = torch.rand(16, 1, generator=g)                      # a float mask that broadcasts over the row
    want = O.masked_normalization(x, w.expand_as(x), 1, False, 1e-3)
    got = areal_amd.masked_normalization(x.to(device), w.to(device), dim=1, eps=1e-3)
    assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-6)
    got16 = areal_amd.masked_normalization(x.to(device).bfloat16(), None, dim=-1)
    assert torch.allclose(got16.cpu(), O.masked_normalization(x.bfloat16(), None, 1), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("estimator", ["k1", "k2", "k3"])
@pytest.mark.parametrize("clamp", [True, False])
def test_kl_estimator_matches_oracle(device, estimator, clamp):
    from oracle import kl_estimate

    g = torch.Generator().manual_seed(2)
    a = -torch.rand(4, 333, generator=g) * 5
    b = a + torch.randn(4, 333, generator=g) * 3          # differences large enough for the clamp to bind
    b[0, 0] = a[0, 0] - 40.0                              # k3 overflows the clamp by far
    want = kl_estimate(a, b, estimator)
    if clamp:
        want = want.clamp(min=-10, max=10)                # data.py:1654-1655
    got = areal_amd.KLEstimator(estimator, clamp)(a.to(device), b.to(device))
    assert got.shape == a.shape and torch.allclose(got.cpu(), want, rtol=2e-6, atol=1e-6)
    # the numbers the reference's tests quote (tests/test_rejection_sampling.py:507-546): log-ratios 0.5, -0.5, 2.0
    d = torch.tensor([0.5, -0.5, 2.0], device=device)
    val = areal_amd.KLEstimator(estimator, clamp)(d, torch.zeros(3, device=device)).tolist()
    quoted = {"k1": [0.5, -0.5, 2.0], "k2": [0.125, 0.125, 2.0], "k3": [0.1065, 0.1487, 1.1353]}[estimator]
    assert val == pytest.approx(quoted, abs=1e-4)
    with pytest.raises(ValueError, match="Invalid KL estimator"):
        areal_amd.KLEstimator("k4")
