"""GPU parity of the sibling losses (SAPO, clipped value loss) and the actor-side filters (proximal log-prob
approximations, M2PO masking) against the CPU oracle and the reference's known answers."""
import pytest
import torch

import areal_amd
from helpers import cosine
from oracle import siblings as S

pytestmark = pytest.mark.gpu


def _tok(n, seed):
    g = torch.Generator().manual_seed(seed)
    lp = -torch.rand(n, generator=g) * 3
    old = lp + 0.3 * torch.randn(n, generator=g)
    adv = torch.randn(n, generator=g)
    mask = torch.rand(n, generator=g) < 0.7
    return lp, old, adv, mask


@pytest.mark.parametrize("level", ["token", "sequence"])
@pytest.mark.parametrize("tau_pos,tau_neg", [(1.0, 1.05), (2.5, 0.7)])
def test_sapo_matches_oracle(device, level, tau_pos, tau_neg):
    n = 777
    lp, old, adv, mask = _tok(n, 3)
    adv[5] = 0.0
    cu = torch.tensor([0, 100, 101, 400, 777], dtype=torch.int32)
    mask[100:101] = False  # a sequence with no valid token
    x = lp.clone().requires_grad_(True)
    w_loss, w_stat = S.sapo_loss(x, old, adv, tau_pos, tau_neg, mask, level, cu)
    w_loss.backward()
    y = lp.to(device).requires_grad_(True)
    loss, stat = areal_amd.sapo_loss_fn(y, old.to(device), adv.to(device), tau_pos, tau_neg, mask.to(device), level,
                                        cu.to(device))
    loss.backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=1e-5, abs=1e-7)
    for k in ("loss", "importance_weight", "approx_kl", "sapo_soft_gate", "sapo_scaled_gate_pos",
              "sapo_scaled_gate_neg"):
        assert torch.allclose(stat[k].cpu(), w_stat[k], rtol=2e-5, atol=2e-6), k
    assert not stat["clip_mask"].any() and stat["clip_mask"].dtype == torch.bool
    assert torch.allclose(y.grad.cpu(), x.grad, rtol=1e-4, atol=1e-8) and cosine(y.grad.cpu(), x.grad) > 0.999999


def test_sapo_known_value_2d_and_errors(device):
    one = torch.ones(1, 2, device=device)
    loss, stat = areal_amd.sapo_loss_fn(one, one, one, 1.0, 1.0, torch.ones(1, 2, dtype=torch.bool, device=device))
    assert abs(float(loss) + 2.0) < 1e-5 and stat["sapo_soft_gate"].shape == (1, 2)
    assert torch.allclose(stat["sapo_soft_gate"].cpu(), torch.full((1, 2), 2.0), atol=1e-5)
    with pytest.raises(ValueError, match="must be positive"):
        areal_amd.sapo_loss_fn(one, one, one, 1.0, -1.0, one.bool())
    with pytest.raises(ValueError, match="Invalid importance_sampling_level"):
        areal_amd.sapo_loss_fn(one, one, one, 1.0, 1.0, one.bool(), importance_sampling_level="x")
    # 2-D sequence level: rows are the sequences
    g = torch.Generator().manual_seed(1)
    lp, old, adv = torch.randn(4, 8, generator=g), torch.randn(4, 8, generator=g), torch.randn(4, 8, generator=g)
    mask = torch.rand(4, 8, generator=g) < 0.8
    w_loss, _ = S.sapo_loss(lp, old, adv, 1.0, 1.05, mask, "sequence")
    loss, _ = areal_amd.sapo_loss_fn(lp.to(device), old.to(device), adv.to(device), 1.0, 1.05, mask.to(device),
                                     "sequence")
    assert float(loss) == pytest.approx(float(w_loss), rel=1e-5, abs=1e-7)


@pytest.mark.parametrize("kind", ["mse", "huber"])
@pytest.mark.parametrize("with_mask", [True, False])
def test_critic_loss_matches_oracle(device, kind, with_mask):
    g = torch.Generator().manual_seed(9)
    shape = (6, 50)
    old = torch.randn(*shape, generator=g) * (8.0 if kind == "huber" else 1.0)
    value = old + 0.3 * torch.randn(*shape, generator=g)
    target = old + torch.randn(*shape, generator=g) * (12.0 if kind == "huber" else 1.0)
    value[0, :5] = old[0, :5]                 # ties: original == clipped
    value[1, :3] = old[1, :3] + 0.2           # exactly on the clip boundary
    mask = torch.rand(*shape, generator=g) < 0.6 if with_mask else None
    x = value.clone().requires_grad_(True)
    w_loss, w_stat = S.critic_loss(x, old, target, 0.2, mask, kind)
    w_loss.backward()
    y = value.to(device).requires_grad_(True)
    loss, stat = areal_amd.ppo_critic_loss_fn(y, old.to(device), target.to(device), 0.2,
                                              None if mask is None else mask.to(device), kind)
    loss.backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=1e-5)
    assert torch.allclose(stat["loss"].cpu(), w_stat["loss"], rtol=1e-6, atol=1e-7)
    assert torch.equal(stat["clip_mask"].cpu(), w_stat["clip_mask"])
    assert torch.allclose(y.grad.cpu(), x.grad, rtol=1e-5, atol=1e-9)


def test_critic_loss_edge_cases(device):
    v = torch.randn(8, device=device)
    loss, _ = areal_amd.ppo_critic_loss_fn(v, v.clone(), v + 1, 0.2, torch.zeros(8, dtype=torch.bool, device=device))
    assert torch.isnan(loss)  # 0 / 0, as in the reference
    with pytest.raises(NotImplementedError):
        areal_amd.ppo_critic_loss_fn(v, v, v, 0.2, None, "l1")
    with pytest.raises(AssertionError):
        areal_amd.ppo_critic_loss_fn(v.double(), v, v, 0.2)


def test_prox_approx_matches_oracle_and_known_answers(device):
    f = lambda v: torch.tensor(v, dtype=torch.float32)
    a = areal_amd.compute_prox_logp_approximations(f([[-1.0], [-2.0]]).to(device), f([[-1.5], [-2.2]]).to(device),
                                                   torch.tensor([[0], [2]], dtype=torch.int32).to(device), 4)
    assert torch.allclose(a["loglinear"].cpu(), f([[-1.375], [-2.1]]), atol=1e-4)   # tests/test_prox_approx.py:84-106
    assert set(a) == {"loglinear", "linear", "rollout"} and a["linear"].shape == (2, 1)
    g = torch.Generator().manual_seed(2)
    old, new = -torch.rand(5, 40, generator=g) * 4, -torch.rand(5, 40, generator=g) * 4
    ver = torch.randint(-1, 12, (5, 40), generator=g)
    for cur in (0, 3, 10, 12):
        want = S.prox_logp_approximations(old, new, ver, cur)
        got = areal_amd.compute_prox_logp_approximations(old.to(device), new.to(device), ver.to(device), cur)
        for k in want:
            assert torch.allclose(got[k].cpu(), want[k], rtol=1e-5, atol=1e-6), (cur, k)
    only = areal_amd.compute_prox_logp_approximations(old.to(device), new.to(device), ver.to(device), 5, "loglinear")
    assert list(only) == ["loglinear"]


@pytest.mark.parametrize("n,thr", [(1, 0.1), (77, 0.05), (5000, 0.02), (5000, 1e-9), (5000, 50.0), (200000, 0.04)])
def test_m2po_matches_oracle(device, n, thr):
    g = torch.Generator().manual_seed(n)
    old = torch.randn(n, generator=g) * 0.5
    prox = old + torch.randn(n, generator=g) * 0.3
    mask = torch.rand(n, generator=g) < 0.7
    if n > 10:
        prox[3] = old[3] + 0.7
        prox[7] = old[7] + 0.7  # a tie
    want = S.m2po_mask(old, prox, mask, thr)
    got = areal_amd.apply_m2po_masking(old.to(device), prox.to(device), mask.to(device), thr).cpu()
    assert got.dtype == torch.bool and got.shape == mask.shape
    diff = int((got != want).sum())
    # float32 suffix sums in another order may move the cut by a token or two on long inputs
    assert diff <= (0 if n <= 5000 else 2), diff
    assert not (got & ~mask).any() and (int(got.sum()) >= 1 or not mask.any())
    # the mean second momentum of what is kept is below the threshold (or a single token is left)
    d = (old - prox)[got]
    assert int(got.sum()) <= 1 or float((d * d).double().mean()) < thr * (1 + 1e-5)


def test_m2po_2d_and_empty(device):
    old, prox = torch.zeros(2, 5), torch.tensor([[0.0, 1.0, 2.0, 3.0, 4.0]] * 2)
    allm = torch.ones(2, 5, dtype=torch.bool)
    got = areal_amd.apply_m2po_masking(old.to(device), prox.to(device), allm.to(device), 2.0).cpu()
    assert torch.equal(got, S.m2po_mask(old, prox, allm, 2.0)) and got.shape == (2, 5)
    none = torch.zeros(2, 5, dtype=torch.bool)
    assert not areal_amd.apply_m2po_masking(old.to(device), prox.to(device), none.to(device), 2.0).any()


@pytest.mark.parametrize("variant", ["ppo_rs", "sapo", "loglinear_m2po"])
def test_grpo_loss_fn_matches_composed_oracle(device, variant):
    """The actor's loss function (actor.py:408-480) against the same composition of oracle pieces."""
    from areal_amd import RejectionSamplingConfig
    from areal_amd.engine_glue import grpo_loss_fn
    from oracle import ppo as OP

    n = 600
    lp, old, adv, mask = _tok(n, 13)
    g = torch.Generator().manual_seed(14)
    prox = lp + 0.1 * torch.randn(n, generator=g)
    ent = torch.rand(n, generator=g)
    ver = torch.randint(-1, 4, (n,), generator=g)
    cu = torch.tensor([0, 200, 600], dtype=torch.int32)
    data = dict(logprobs=old, advantages=adv, loss_mask=mask, prox_logp=prox, cu_seqlens=cu, versions=ver)
    kw = dict(eps_clip=0.2, eps_clip_higher=0.28, c_clip=3.0)
    x = lp.clone().requires_grad_(True)
    if variant == "ppo_rs":
        rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", upper=1.25)
        kw.update(rejection_sampling=rs, use_decoupled_loss=True)
        w_loss, w_stat = OP.ppo_actor_loss(x, prox, old, adv, 0.2, mask, 0.28, 3.0, rs, "token", cu)
        w_mask = mask
    elif variant == "sapo":
        kw.update(use_sapo_loss=True, sapo_tau_pos=1.0, sapo_tau_neg=1.05)
        w_loss, w_stat = S.sapo_loss(x, old, adv, 1.0, 1.05, mask)
        w_mask = mask
    else:
        data["prox_logp"] = None
        kw.update(prox_logp_method="loglinear", current_version=4, m2_threshold=0.05, use_decoupled_loss=True)
        w_prox = S.prox_logp_approximations(old, lp, ver, 4, "loglinear")["loglinear"]
        w_mask = S.m2po_mask(old, w_prox, mask, 0.05)
        w_loss, w_stat = OP.ppo_actor_loss(x, w_prox, old, adv, 0.2, w_mask, 0.28, 3.0, None, "token", cu)
    w_loss.backward()
    y = lp.to(device).requires_grad_(True)
    d_dev = {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in data.items()}
    loss, stat = grpo_loss_fn(y, ent.to(device), d_dev, **kw)
    loss.backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=1e-4, abs=1e-7)
    assert torch.allclose(y.grad.cpu(), x.grad, rtol=1e-4, atol=1e-8)
    assert torch.equal(stat["loss_mask"].cpu(), w_mask)
    red = stat["reduced"]
    sel = w_mask
    assert float(red["importance_weight"]["avg"]) == pytest.approx(float(w_stat["importance_weight"][sel].mean()), rel=1e-4)
    assert float(red["actor_loss"]["sum"]) == pytest.approx(float(w_stat["loss"][sel].sum()), rel=1e-4, abs=1e-5)
    assert float(red["entropy"]["max"]) == float(ent[sel].max()) and float(red["new_logp"]["count"]) == float(sel.sum())
    if variant == "ppo_rs":
        assert float(red["rs_filtered_fraction"]) == pytest.approx(float(w_stat["filtered_fraction"]), abs=1e-6)
        assert float(red["behave_imp_weight"]["count"]) == float(w_stat["behave_mask"].sum())
        assert float(red["clipped_new_logp"]["count"]) == float(w_stat["clip_mask"].sum())
    if variant == "sapo":
        assert "sapo_soft_gate" in red and "clipped_new_logp" not in red
        with pytest.raises(ValueError, match="SAPO is not compatible"):
            grpo_loss_fn(y, ent.to(device), d_dev, **dict(kw, use_decoupled_loss=True))
    with pytest.raises(ValueError, match="compute_logp\\(\\) was skipped incorrectly"):
        grpo_loss_fn(y, ent.to(device), dict(d_dev, prox_logp=None), 0.2, None, None)


@pytest.mark.parametrize("rl_weight", [0, 0.8])
def test_grpo_loss_fn_joint_distillation(device, rl_weight):
    """teacher_logp in the micro-batch (actor.py:482-511): pure reverse-KL distillation and the joint RL + KD loss."""
    from areal_amd.engine_glue import grpo_loss_fn
    from oracle import ppo as OP

    n = 500
    lp, old, adv, mask = _tok(n, 21)
    g = torch.Generator().manual_seed(22)
    prox = lp + 0.1 * torch.randn(n, generator=g)
    teacher = lp + 0.4 * torch.randn(n, generator=g)
    ent = torch.rand(n, generator=g)
    cu = torch.tensor([0, 150, 500], dtype=torch.int32)
    data = dict(logprobs=old, advantages=adv, loss_mask=mask, prox_logp=prox, cu_seqlens=cu, teacher_logp=teacher,
                rl_loss_weight=rl_weight, distill_loss_weight=0.02)
    x = lp.clone().requires_grad_(True)
    w_loss, _ = OP.ppo_actor_loss(x, prox, old, adv, 0.2, mask, None, None, None, "token", cu)
    w_loss, w_rkl = S.distillation_loss(w_loss, x, old, teacher, mask, rl_weight, 0.02)
    w_loss.backward()
    y = lp.to(device).requires_grad_(True)
    d_dev = {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in data.items()}
    loss, stat = grpo_loss_fn(y, ent.to(device), d_dev, 0.2, None, None, use_decoupled_loss=True)
    loss.backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=1e-4, abs=1e-7)
    assert torch.allclose(y.grad.cpu(), x.grad, rtol=1e-4, atol=1e-9)
    assert float(stat["reduced"]["rkl_loss"]["sum"]) == pytest.approx(float(w_rkl.detach()[mask].sum()), rel=1e-4, abs=1e-6)


def test_distillation_terms_shapes_and_empty_mask(device):
    lp = torch.randn(3, 7, device=device) - 2
    teacher = lp + 0.1
    none = torch.zeros(3, 7, dtype=torch.bool, device=device)
    x = lp.clone().requires_grad_(True)
    mean, term = areal_amd.distillation_terms(x, lp, teacher, none, pure=True)
    mean.backward()
    assert float(mean.detach()) == 0.0 and term.shape == (3, 7) and float(term.abs().max()) == 0.0
    assert float(x.grad.abs().max()) == 0.0
    allm = ~none
    mean, term = areal_amd.distillation_terms(lp, None, teacher, allm, pure=False)
    assert float(mean) == pytest.approx(-0.1, rel=1e-5) and torch.allclose(term, lp - teacher)
    with pytest.raises(ValueError, match="same shape"):
        areal_amd.distillation_terms(lp, None, teacher[:2], allm, pure=False)


def test_loss_adapters_count_logical_tokens(device):
    """tests/test_ppo_stats.py:54-111: with cu_seqlens = [0, 4] and two local tokens, n_tokens is 4 for the actor's
    and the critic's loss function; the critic adapter against the oracle's value loss."""
    from areal_amd.engine_glue import critic_loss_fn, grpo_loss_fn

    cu = torch.tensor([0, 4], dtype=torch.int32, device=device)
    z2 = torch.zeros(2, device=device)
    data = dict(input_ids=torch.tensor([11, 12], device=device), cu_seqlens=cu, logprobs=z2, advantages=z2 + 1,
                loss_mask=torch.ones(2, dtype=torch.bool, device=device), prox_logp=z2,
                versions=torch.zeros(2, dtype=torch.int32, device=device))
    _, stat = grpo_loss_fn(z2.clone().requires_grad_(True), z2, data, 0.2, None, None)
    assert stat["reduced"]["n_tokens"] == 4
    g = torch.Generator().manual_seed(2)
    n = 300
    value, old, target = (torch.randn(n, generator=g) for _ in range(3))
    mask = torch.rand(n, generator=g) < 0.7
    cdata = dict(input_ids=torch.zeros(n, dtype=torch.long, device=device), values=old.to(device),
                 returns=target.to(device), loss_mask=mask.to(device),
                 cu_seqlens=torch.tensor([0, 2 * n], dtype=torch.int32, device=device))
    v = value.to(device).unsqueeze(-1).requires_grad_(True)
    loss, cstat = critic_loss_fn(v, cdata, 0.3)
    loss.backward()
    x = value.clone().requires_grad_(True)
    w_loss, w_stat = S.critic_loss(x, old, target, 0.3, mask)
    w_loss.backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=1e-5)
    assert torch.allclose(v.grad.squeeze(-1).cpu(), x.grad, rtol=1e-4, atol=1e-9)
    red = cstat["reduced"]
    assert red["n_tokens"] == 2 * n and float(red["new_value"]["count"]) == float(mask.sum())
    assert float(red["clipped_new_value"]["count"]) == float(w_stat["clip_mask"].sum())
    assert float(red["critic_loss"]["sum"]) == pytest.approx(float(w_stat["loss"][mask].sum()), rel=1e-4)


def _check_moments(got: dict, tensors: dict, mask, tag=""):
    assert sorted(got) == sorted(tensors), (tag, sorted(got), sorted(tensors))
    for name, t in tensors.items():
        sel = t.double()[mask]
        g = {k: float(v) for k, v in got[name].items()}
        assert g["count"] == sel.numel(), (tag, name)
        scale = float(sel.abs().max()) + 1e-12
        assert abs(g["sum"] - float(sel.sum())) <= 2e-5 * scale * max(sel.numel() ** 0.5, 1.0), (tag, name, "sum")
        assert abs(g["min"] - float(sel.min())) <= 1e-5 * scale + 1e-7, (tag, name, "min")
        assert abs(g["max"] - float(sel.max())) <= 1e-5 * scale + 1e-7, (tag, name, "max")
        assert abs(g["avg"] - float(sel.mean())) <= 2e-5 * scale, (tag, name, "avg")


@pytest.mark.parametrize("method,with_gt", [("recompute", True), ("loglinear", False), ("loglinear", True),
                                            ("metrics", True), ("metrics", False)])
@pytest.mark.parametrize("n", [1, 777, 200_003])
def test_proximal_logging_stats_match_oracle(device, method, with_gt, n):
    g = torch.Generator().manual_seed(n + 17)
    lp = -torch.rand(n, generator=g) * 3
    old = lp + 0.3 * torch.randn(n, generator=g)
    gt = lp + 0.1 * torch.randn(n, generator=g) if with_gt else None
    ver = torch.randint(-1, 7, (n,), generator=g, dtype=torch.int32)
    mask = torch.rand(n, generator=g) < 0.6
    mask[0] = True
    ver[0] = 2
    tensors, stale = S.proximal_logging_tensors(old, lp, gt, ver, 6, mask, method)
    got = areal_amd.proximal_logging_stats(old.to(device), lp.to(device), None if gt is None else gt.to(device),
                                           ver.to(device), 6, mask.to(device), method)
    _check_moments(got["compute_logp"], tensors, mask, method)
    vs = got["version_stats"]
    assert vs["v_theta"] == 6 and vs["v_proximal"] == 5
    gen = mask & (ver >= 0)
    for key in ("sample_staleness_proximal", "sample_staleness_theta"):
        want = stale[key]
        assert float(vs[key]["count"]) == int(gen.sum()) == want.numel()
        assert float(vs[key]["min"]) == float(want.min()) and float(vs[key]["max"]) == float(want.max())
        assert float(vs[key]["avg"]) == pytest.approx(float(want.double().mean()), rel=1e-6)


def test_proximal_logging_stats_without_versions_or_tokens(device):
    n = 100
    lp, old, _, mask = _tok(n, 4)
    gt = lp + 0.1
    for kw in (dict(versions=None, current_version=3), dict(versions=torch.zeros(n, dtype=torch.int32), current_version=None)):
        got = areal_amd.proximal_logging_stats(old.to(device), lp.to(device), gt.to(device),
                                               None if kw["versions"] is None else kw["versions"].to(device),
                                               kw["current_version"], mask.to(device), "metrics")
        assert list(got["compute_logp"]) == ["prox_logp_gt"] and got["version_stats"] == {}
        assert float(got["compute_logp"]["prox_logp_gt"]["sum"]) == pytest.approx(float(gt[mask].sum()), rel=1e-5)
    # only prompt tokens selected: the staleness count is 0 where the reference logs nothing
    ver = torch.full((n,), -1, dtype=torch.int32)
    got = areal_amd.proximal_logging_stats(old.to(device), lp.to(device), None, ver.to(device), 3, mask.to(device))
    assert float(got["version_stats"]["sample_staleness_theta"]["count"]) == 0
    assert sorted(got["compute_logp"]) == ["kl_div_direct", "kl_div_dual", "kl_div_taylor"]
    # an empty batch (no tokens at all)
    e = torch.zeros(0, device=device)
    got = areal_amd.proximal_logging_stats(e, e, None, torch.zeros(0, dtype=torch.int32, device=device), 3,
                                           torch.zeros(0, dtype=torch.bool, device=device), "loglinear")
    assert float(got["compute_logp"]["loglinear/approx_logp"]["count"]) == 0
    # nothing selected at all
    got = areal_amd.proximal_logging_stats(old.to(device), lp.to(device), None, ver.to(device), 3,
                                           torch.zeros(n, dtype=torch.bool, device=device))
    assert float(got["compute_logp"]["kl_div_dual"]["count"]) == 0
    assert float(got["compute_logp"]["kl_div_dual"]["min"]) == float("inf")


def test_grpo_loss_fn_reports_the_logging_scopes(device):
    """Which names appear in which mode follows tests/test_prox_approx.py:795-935."""
    from areal_amd import engine_glue as G

    n = 512
    lp, old, adv, mask = _tok(n, 6)
    g = torch.Generator().manual_seed(1)
    data = dict(logprobs=old.to(device), advantages=adv.to(device), loss_mask=mask.to(device),
                prox_logp=(lp + 0.05 * torch.randn(n, generator=g)).to(device),
                versions=torch.randint(-1, 3, (n,), generator=g, dtype=torch.int32).to(device))
    ent = torch.rand(n, device=device)
    kw = dict(eps_clip=0.2, eps_clip_higher=None, c_clip=None, current_version=3, use_decoupled_loss=True)
    _, st = G.grpo_loss_fn(lp.to(device).requires_grad_(True), ent, data, prox_logp_method="recompute", **kw)
    names = st["reduced"]["compute_logp"]
    assert "prox_logp_gt" in names and "kl_div_dual" in names and not any("/" in k for k in names)
    assert float(st["reduced"]["version_stats"]["sample_staleness_theta"]["min"]) >= 1.0
    _, st = G.grpo_loss_fn(lp.to(device).requires_grad_(True), ent, data, prox_logp_method="loglinear", **kw)
    names = st["reduced"]["compute_logp"]
    assert "loglinear/approx_logp" in names and "loglinear/abs_error" not in names and "linear/approx_logp" not in names
    _, st = G.grpo_loss_fn(lp.to(device).requires_grad_(True), ent, data, prox_logp_method="metrics", **kw)
    names = st["reduced"]["compute_logp"]
    for method in ("loglinear", "linear", "rollout"):
        assert f"{method}/abs_error" in names and f"{method}/importance_weight_rel_error" in names
    tensors, _ = S.proximal_logging_tensors(old, lp, data["prox_logp"].cpu(), data["versions"].cpu(), 3, mask, "metrics")
    _check_moments(names, tensors, mask, "glue")
    data.pop("versions")
    _, st = G.grpo_loss_fn(lp.to(device).requires_grad_(True), ent, data, prox_logp_method="recompute", **kw)
    assert list(st["reduced"]["compute_logp"]) == ["prox_logp_gt"] and st["reduced"]["version_stats"] == {}


# ---------------------------------------------------------------------------------------------------------------
# SAPO fused with the log-prob op (one pass over the logits) and with the lm_head (no logits in memory)
# ---------------------------------------------------------------------------------------------------------------
_SAPO_STATS = ("loss", "importance_weight", "approx_kl", "sapo_soft_gate", "sapo_scaled_gate_pos", "sapo_scaled_gate_neg")


def _sapo_case(T_pad, T, V, seed):
    import oracle

    g = torch.Generator().manual_seed(seed)
    logits = (2.0 * torch.randn(T_pad, V, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T_pad,), generator=g)
    ref = oracle.logprobs(logits, labels)[:T]
    old = ref + 0.3 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    adv[::9] = 0.0                                   # adv == 0 takes the negative gate, as torch.where(adv > 0) does
    mask = torch.rand(T, generator=g) < 0.7
    return logits, labels, old, adv, mask


@pytest.mark.parametrize("T_pad,T,V,temperature,scale,inplace", [
    (40, 40, 9000, 1.0, None, False),       # two-pass rows
    (300, 280, 32768, 0.8, 0.37, False),    # register-resident rows, batch padding, loss scale
    (70, 64, 50257, 1.0, None, True),       # rows at every even address (V % 8 != 0), gradient written over the logits
])
def test_fused_logits_sapo_matches_oracle(device, T_pad, T, V, temperature, scale, inplace):
    import oracle
    from helpers import assert_same_magnitude, assert_within

    logits, labels, old, adv, mask = _sapo_case(T_pad, T, V, seed=T + V)
    x = logits.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_logprobs_sapo_loss(
        x, labels.to(device), old.to(device), adv.to(device), 1.0, 1.05, mask.to(device), temperature=temperature,
        loss_scale=scale, inplace_backward=inplace)
    loss.backward()
    z = logits.float().requires_grad_(True)
    o_lp, o_ent = oracle.logprobs_entropy(z, labels, temperature)
    w_loss, w_stat = S.sapo_loss(o_lp[:T], old, adv, 1.0, 1.05, mask)
    (w_loss * (1.0 if scale is None else scale)).backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()) * (1.0 if scale is None else scale), rel=1e-3)
    assert_within(stat["logprobs"], o_lp[:T].detach(), 2e-3, "log-prob")
    assert_within(stat["entropy"], o_ent[:T].detach(), 2e-3, "entropy")
    for k in _SAPO_STATS:                                        # at every token, masked ones included
        assert_within(stat[k], w_stat[k], 2e-3, k)
    assert not stat["clip_mask"].any() and not stat["dual_clip_mask"].any()
    assert cosine(x.grad.float().cpu(), z.grad) > 0.9999
    assert_same_magnitude(x.grad, z.grad, what="d(logits)")
    assert float(x.grad[T:].float().abs().sum()) == 0.0 and float(x.grad[:T][~mask.to(device)].float().abs().sum()) == 0.0
    if inplace:
        assert torch.equal(x.detach(), x.grad)
    # without a gradient to produce: the forward kernel and the loss on its log-probs
    with torch.no_grad():
        l2, s2 = areal_amd.fused_logprobs_sapo_loss(logits.to(device), labels.to(device), old.to(device), adv.to(device),
                                                    1.0, 1.05, mask.to(device), temperature=temperature, loss_scale=scale)
    assert float(l2) == pytest.approx(float(loss.detach()), rel=1e-5) and set(s2) == set(stat)
    with pytest.raises(ValueError, match="must be positive"):
        areal_amd.fused_logprobs_sapo_loss(x, labels.to(device), old.to(device), adv.to(device), 1.0, 0.0, mask.to(device))


@pytest.mark.parametrize("backward", ["carry", "recompute"])
def test_fused_lm_head_sapo_matches_oracle(device, backward):
    import oracle
    from areal_amd import _native
    from helpers import assert_same_magnitude, assert_within

    chunk = int(_native.load().aa_lmhead_chunk_tokens())
    T_pad, T, H, V = chunk + 200, chunk + 130, 64, 641           # two token chunks, a vocabulary that is no multiple of 8
    g = torch.Generator().manual_seed(4)
    hidden = torch.randn(T_pad, H, generator=g).bfloat16()
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T_pad,), generator=g)
    ref = oracle.logprobs(oracle.lmhead_logits(hidden, weight), labels)[:T]
    old = ref + 0.3 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < 0.7
    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_sapo_loss(h, w, labels.to(device), old.to(device), adv.to(device), 1.0, 1.05,
                                                   mask.to(device), temperature=0.9, loss_scale=0.5, backward=backward)
    loss.backward()
    h_o = hidden.float().requires_grad_(True)
    w_o = weight.float().requires_grad_(True)
    o_lp, o_ent = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), labels, 0.9)
    w_loss, w_stat = S.sapo_loss(o_lp[:T], old, adv, 1.0, 1.05, mask)
    (w_loss * 0.5).backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()) * 0.5, rel=1e-3)
    assert_within(stat["logprobs"], o_lp[:T].detach(), 2e-3, "log-prob")
    for k in _SAPO_STATS:
        assert_within(stat[k], w_stat[k], 2e-3, k)
    assert cosine(h.grad.float().cpu(), h_o.grad) > 0.9999 and cosine(w.grad.float().cpu(), w_o.grad) > 0.9999
    assert_same_magnitude(h.grad, h_o.grad, what="d(hidden)")
    assert_same_magnitude(w.grad, w_o.grad, what="d(W)")
    assert float(h.grad[T:].float().abs().sum()) == 0.0


def test_engine_glue_takes_the_fused_sapo_step(device):
    """``compute_logprobs_and_loss(use_sapo_loss=True)``: label roll, pad rows, loss scale around the fused SAPO pass."""
    import oracle
    from areal_amd import engine_glue

    pad, V = 8, 9000
    logits, labels, old, adv, mask = _sapo_case(64 + pad, 64, V, seed=2)
    input_ids = torch.cat([labels[-1:], labels[:-1]]).unsqueeze(0)          # rolled by one gives `labels`
    mb = dict(loss_mask=mask.to(device), logprobs=old.to(device), advantages=adv.to(device), prox_logp=None)
    x = logits.to(device).requires_grad_(True)
    loss, stat = engine_glue.compute_logprobs_and_loss(x, {"input_ids": input_ids.to(device)}, mb, pad, 100.0,
                                                       eps_clip=0.2, use_sapo_loss=True)
    loss.backward()
    z = logits.float().requires_grad_(True)
    w_loss, _ = S.sapo_loss(oracle.logprobs(z, labels)[:64], old, adv, 1.0, 1.05, mask)
    (w_loss * float(mask.sum()) / 100.0).backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()) * float(mask.sum()) / 100.0, rel=1e-3)
    assert cosine(x.grad.float().cpu(), z.grad) > 0.9999 and float(x.grad[64:].float().abs().sum()) == 0.0
    assert "sapo_soft_gate" in stat and stat["logprobs"].shape == (64,)
