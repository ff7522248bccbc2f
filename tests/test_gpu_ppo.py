"""GPU parity of apply_rejection_sampling and ppo_actor_loss_fn against the oracle and against the
reference's own known-answer cases."""
import itertools
import math

import pytest
import torch

import areal_amd
import oracle
from areal_amd import RejectionSamplingConfig
from helpers import cosine
from test_oracle_pins import _ppo_case_tensors, _run_rs_case, check_ppo_expectations, check_rs_expectations

pytestmark = pytest.mark.gpu


def _to(dev, *ts):
    return [None if t is None else t.to(dev) for t in ts]


def test_rejection_sampling_reference_known_answers(device, known_answers):
    def fn(prox, old, mask, cu, cfg):
        return areal_amd.apply_rejection_sampling(*_to(device, prox, old, mask, cu), cfg)

    for case in known_answers["rejection_sampling"]:
        check_rs_expectations(case, _run_rs_case(case, fn, RejectionSamplingConfig))


def test_ppo_loss_reference_known_answers(device, known_answers):
    for case in known_answers["ppo_actor_loss"]:
        lp, prox, old, adv, mask, cu = _to(device, *_ppo_case_tensors(case))
        loss, stat = areal_amd.ppo_actor_loss_fn(
            lp, prox, old, adv, case["eps_clip"], mask, importance_sampling_level=case["level"], cu_seqlens=cu
        )
        check_ppo_expectations(case, loss.cpu(), {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in stat.items()})


def _random_packed(seed, n_seqs=9, lo=1, hi=40, all_masked_seq=True):
    g = torch.Generator().manual_seed(seed)
    lengths = torch.randint(lo, hi + 1, (n_seqs,), generator=g).tolist()
    T = sum(lengths)
    cu = torch.tensor([0] + list(itertools.accumulate(lengths)), dtype=torch.int32)
    prox = -2 + 0.5 * torch.randn(T, generator=g)
    old = prox + 0.6 * torch.randn(T, generator=g)
    lp = prox + 0.3 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < 0.7
    if all_masked_seq:
        mask[int(cu[2]) : int(cu[3])] = False
    return lengths, cu, lp, prox, old, adv, mask


RS_GRID = [
    dict(level=lv, action=ac, metric=me, agg=ag, upper=up, lower=lo)
    for lv in ("token", "sequence")
    for ac, me in (("mask", "ratio"), ("mask", "kl_k1"), ("mask", "kl_k2"), ("mask", "kl_k3"), ("clamp", "ratio"))
    for ag in (("mean",) if lv == "token" else ("sum", "mean", "max"))
    for up, lo in (((1.6, None), (1.6, 0.7)) if me == "ratio" else ((0.15, None), (0.15, -0.2)))
]


@pytest.mark.parametrize("kw", RS_GRID, ids=lambda k: "-".join(str(v) for v in k.values()))
def test_rejection_sampling_matches_oracle_packed_and_padded(device, kw):
    cfg = RejectionSamplingConfig(**kw)
    _, cu, _, prox, old, _, mask = _random_packed(seed=17)
    prox[5] = float("-inf"); old[5] = float("-inf")  # NaN difference is sanitised (functional.py:231-233)
    for mask_t in (mask, mask.float()):
        want = oracle.rejection_sampling(prox, old, mask_t, cu, cfg)
        got = areal_amd.apply_rejection_sampling(*_to(device, prox, old, mask_t, cu), cfg)
        assert got.loss_mask.dtype == mask_t.dtype
        assert torch.equal(got.loss_mask.cpu(), want.loss_mask)                      # masks: bit-exact
        assert torch.allclose(got.behave_imp_weight.cpu(), want.behave_imp_weight, rtol=2e-6, atol=1e-7)
        assert got.filtered_fraction == pytest.approx(want.filtered_fraction, abs=1e-12)
    # 2-D padded layout
    g = torch.Generator().manual_seed(23)
    p2 = -2 + 0.5 * torch.randn(6, 11, generator=g)
    o2 = p2 + 0.6 * torch.randn(6, 11, generator=g)
    m2 = torch.rand(6, 11, generator=g) < 0.6
    m2[4] = False
    want = oracle.rejection_sampling(p2, o2, m2, None, cfg)
    got = areal_amd.apply_rejection_sampling(*_to(device, p2, o2, m2), None, cfg)
    assert torch.equal(got.loss_mask.cpu(), want.loss_mask)
    assert torch.allclose(got.behave_imp_weight.cpu(), want.behave_imp_weight, rtol=2e-6, atol=1e-7)
    assert got.filtered_fraction == pytest.approx(want.filtered_fraction, abs=1e-12)


PPO_GRID = [
    dict(eps_clip=0.2),
    dict(eps_clip=0.2, eps_clip_higher=0.28, c_clip=3.0),
    dict(eps_clip=0.1, c_clip=1.2),
    dict(eps_clip=0.2, rs=dict(level="token", metric="ratio", upper=1.5)),
    dict(eps_clip=0.2, c_clip=3.0, eps_clip_higher=0.28, rs=dict(level="token", action="clamp", metric="ratio", upper=1.5)),
    dict(eps_clip=0.2, rs=dict(level="sequence", agg="mean", metric="kl_k2", upper=0.2)),
    dict(eps_clip=0.2, rs=dict(level="sequence", action="clamp", agg="max", metric="ratio", upper=1.4, lower=0.8)),
]


@pytest.mark.parametrize("level", ["token", "sequence"])
@pytest.mark.parametrize("kw", PPO_GRID, ids=lambda k: "-".join(f"{a}={b}" for a, b in k.items() if a != "rs") + ("-rs" if "rs" in k else ""))
def test_ppo_loss_and_gradient_match_oracle(device, kw, level):
    kw = dict(kw)
    rs = kw.pop("rs", None)
    cfg = RejectionSamplingConfig(**rs) if rs else None
    _, cu, lp, prox, old, adv, mask = _random_packed(seed=29)
    for packed in (True, False):
        if packed:
            args, cu_arg = (lp, prox, old, adv, mask), cu
        else:
            n = (lp.numel() // 7) * 7
            args, cu_arg = tuple(t[:n].reshape(-1, 7) for t in (lp, prox, old, adv, mask)), None
        lp_o = args[0].clone().requires_grad_(True)
        want_loss, want = oracle.ppo_actor_loss(
            lp_o, args[1], args[2], args[3], loss_mask=args[4], rejection_sampling_cfg=cfg,
            importance_sampling_level=level, cu_seqlens=cu_arg, **kw
        )
        want_loss.backward()
        lp_d = args[0].to(device).requires_grad_(True)
        got_loss, got = areal_amd.ppo_actor_loss_fn(
            lp_d, *_to(device, args[1], args[2], args[3]), loss_mask=args[4].to(device), rejection_sampling=cfg,
            importance_sampling_level=level, cu_seqlens=None if cu_arg is None else cu_arg.to(device), **kw
        )
        (got_loss * 1.0).backward()
        assert got_loss.ndim == 0 and got_loss.dtype == torch.float32
        assert float(got_loss.detach()) == pytest.approx(float(want_loss.detach()), rel=1e-3, abs=1e-6)   # stated tolerance
        assert float(got_loss.detach()) == pytest.approx(float(want_loss.detach()), rel=2e-5, abs=1e-6)   # what it delivers
        assert set(got) == set(want)
        for k in ("clip_mask", "dual_clip_mask") + (("behave_mask",) if cfg else ()):
            assert got[k].dtype == torch.bool and torch.equal(got[k].cpu(), want[k]), k
        for k in ("loss", "importance_weight", "approx_kl") + (("behave_approx_kl", "behave_imp_weight") if cfg else ()):
            assert got[k].dtype == torch.float32 and got[k].shape == args[0].shape
            assert torch.allclose(got[k].cpu(), want[k], rtol=1e-5, atol=1e-6), k
        if cfg:
            assert got["filtered_fraction"] == pytest.approx(want["filtered_fraction"], abs=1e-12)
        assert torch.allclose(lp_d.grad.cpu(), lp_o.grad, rtol=2e-5, atol=1e-7)
        assert cosine(lp_d.grad.cpu(), lp_o.grad) > 0.99999


def test_gradient_ties_match_autograd(device):
    """Exact ties: ratio on a clip bound, zero advantage, dual-clip equality."""
    lo, hi = 1.0 - 0.25, 1.0 + 0.25   # exactly representable
    ratios = torch.tensor([lo, hi, 1.0, 2.0, 0.5, 4.0, 3.0, 1.0])
    adv = torch.tensor([1.0, -1.0, 0.0, 1.0, -1.0, -1.0, -1.0, 2.0])
    lp = ratios.log()
    # make exp(lp) land exactly on the intended ratios where that matters
    prox = torch.zeros_like(lp)
    mask = torch.ones_like(lp, dtype=torch.bool)
    lp_o = lp.clone().requires_grad_(True)
    want_loss, want = oracle.ppo_actor_loss(lp_o, prox, prox, adv, 0.25, mask, None, 3.0)
    want_loss.backward()
    lp_d = lp.to(device).requires_grad_(True)
    got_loss, got = areal_amd.ppo_actor_loss_fn(lp_d, *_to(device, prox, prox, adv), 0.25, mask.to(device), None, 3.0)
    got_loss.backward()
    same_ratio = got["importance_weight"].cpu() == want["importance_weight"]
    assert same_ratio[2] and same_ratio[7]
    # compare wherever both sides computed the same ratio bit for bit (exp may differ by an ulp elsewhere)
    assert torch.allclose(lp_d.grad.cpu()[same_ratio], lp_o.grad[same_ratio], rtol=1e-6, atol=1e-8)
    assert torch.equal(got["clip_mask"].cpu()[same_ratio], want["clip_mask"][same_ratio])
    assert torch.equal(got["dual_clip_mask"].cpu()[same_ratio], want["dual_clip_mask"][same_ratio])


def test_edge_cases(device):
    z = torch.randn(2, 4, device=device)
    none = torch.zeros(2, 4, dtype=torch.bool, device=device)
    loss, stat = areal_amd.ppo_actor_loss_fn(z.clone().requires_grad_(True), z, z, z, 0.2, none)
    assert float(loss.detach()) == 0.0 and float(stat["importance_weight"].abs().sum()) == 0.0
    assert "behave_imp_weight" not in stat and "filtered_fraction" not in stat
    with pytest.raises(ValueError, match="cu_seqlens is required for 1D tensors"):
        areal_amd.ppo_actor_loss_fn(z[0], z[0], z[0], z[0], 0.2, ~none[0], importance_sampling_level="sequence")
    with pytest.raises(AssertionError):
        areal_amd.ppo_actor_loss_fn(z, z, z, z, 0.2, ~none, c_clip=1.0)
    # sequences of length one, and a batch of one
    cu = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device=device)
    t = torch.randn(3, device=device)
    loss, stat = areal_amd.ppo_actor_loss_fn(t, t - 0.1, t, torch.ones(3, device=device), 0.2,
                                             torch.ones(3, dtype=torch.bool, device=device),
                                             importance_sampling_level="sequence", cu_seqlens=cu)
    assert torch.allclose(stat["importance_weight"], torch.full((3,), math.exp(0.1), device=device), atol=1e-5)


def test_masked_positions_and_denominator_keep_reference_semantics(device):
    """stat['loss'] keeps its pre-mask value, the ratio is zero where masked, and the denominator is the
    ORIGINAL mask count even when rejection sampling drops tokens (functional.py:479-483)."""
    _, cu, lp, prox, old, adv, mask = _random_packed(seed=31)
    cfg = RejectionSamplingConfig(level="token", metric="ratio", upper=1.3)
    loss, stat = areal_amd.ppo_actor_loss_fn(*_to(device, lp, prox, old, adv), 0.2, mask.to(device), rejection_sampling=cfg)
    kept = stat["behave_mask"].cpu()
    assert kept.sum() < mask.sum()
    manual = float(stat["loss"].cpu()[kept].double().sum()) / int(mask.sum())
    assert float(loss) == pytest.approx(manual, rel=1e-5)
    assert float(stat["importance_weight"].cpu()[~kept].abs().sum()) == 0.0


def test_empty_batches_do_not_raise(device):
    """Zero tokens (a data-parallel rank without work): empty results, zero counts, no launch over null pointers."""
    from areal_amd import RejectionSamplingConfig

    e = torch.zeros(0, device=device)
    eb = torch.zeros(0, dtype=torch.bool, device=device)
    cu0 = torch.zeros(1, dtype=torch.int32, device=device)
    for level in ("token", "sequence"):
        res = areal_amd.apply_rejection_sampling(e, e, eb, cu0, RejectionSamplingConfig(level=level, metric="ratio",
                                                                                         upper=2.0))
        assert res.loss_mask.numel() == 0 and res.filtered_fraction == 0.0
    loss, stat = areal_amd.ppo_actor_loss_fn(e.clone().requires_grad_(True), e, e, e, 0.2, eb)
    assert float(loss.detach()) == 0.0 and stat["importance_weight"].numel() == 0
    adv, ret = areal_amd.gae_advantages(torch.zeros(0, 8, device=device), torch.zeros(0, 8, device=device),
                                        torch.zeros(0, 8, device=device), eb, 1.0, 0.95)
    assert adv.shape == (0, 8) and ret.shape == (0, 8)
