"""GPU parity of the fused lm_head path.  The reference has no fused path, so the oracle is its equivalent:
logits = hidden @ weight.T in fp32, then the log-prob / entropy oracle, with autograd for the gradients."""
import math

import pytest
import torch

import areal_amd
import oracle
from helpers import cosine

pytestmark = pytest.mark.gpu


def _case(T, H, V, seed, w_std=0.02):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (w_std * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    return hidden, weight, labels


@pytest.mark.parametrize(
    "T,H,V,temperature",
    [
        (256, 128, 1024, 1.0),    # exactly one tile column, four tile rows
        (300, 192, 1088, 1.0),    # ragged in tokens and in vocabulary
        (37, 64, 576, 0.7),       # smaller than a tile
        (700, 256, 4160, 1.3),
    ],
)
def test_forward_matches_oracle(device, T, H, V, temperature):
    hidden, weight, labels = _case(T, H, V, seed=T + V, w_std=0.3)
    lp, ent = areal_amd.lm_head_logprobs_entropy(hidden.to(device), weight.to(device), labels.to(device), temperature)
    logits = oracle.lmhead_logits(hidden, weight)
    r_lp, r_ent = oracle.logprobs_entropy_f64(logits, labels, temperature)
    assert lp.dtype == torch.float32 and lp.shape == (T,)
    assert float((lp.cpu().double() - r_lp).abs().max()) < 2e-3     # stated tolerance
    assert float((lp.cpu().double() - r_lp).abs().max()) < 2e-4
    assert float((ent.cpu().double() - r_ent).abs().max()) < 2e-4
    # deterministic
    lp2, ent2 = areal_amd.lm_head_logprobs_entropy(hidden.to(device), weight.to(device), labels.to(device), temperature)
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2)


def test_closed_form_and_bad_label(device):
    # zero weights: uniform distribution over V
    T, H, V = 64, 64, 640
    hidden = torch.randn(T, H).bfloat16().to(device)
    weight = torch.zeros(V, H, dtype=torch.bfloat16, device=device)
    labels = torch.randint(0, V, (T,), device=device)
    labels[3] = V + 5
    lp, ent = areal_amd.lm_head_logprobs_entropy(hidden, weight, labels)
    ok = torch.ones(T, dtype=torch.bool, device=device)
    ok[3] = False
    assert float((lp[ok] + math.log(V)).abs().max()) < 1e-5 and float((ent - math.log(V)).abs().max()) < 1e-4
    assert torch.isnan(lp[3])
    with pytest.raises(areal_amd.NativeLibraryError):
        areal_amd.lm_head_logprobs_entropy(hidden[:, :40].contiguous(), weight[:, :40].contiguous(), labels)  # H % 64


@pytest.mark.parametrize("T,H,V,temperature,with_entropy", [(300, 128, 1088, 1.0, False), (520, 192, 832, 0.8, True)])
def test_backward_matches_autograd_of_oracle(device, T, H, V, temperature, with_entropy):
    hidden, weight, labels = _case(T, H, V, seed=7 * T + V, w_std=0.3)
    g = torch.Generator().manual_seed(3)
    gl = torch.randn(T, generator=g)
    gl[::5] = 0.0
    gh = 0.3 * torch.randn(T, generator=g) if with_entropy else None
    h_d = hidden.to(device).requires_grad_(True)
    w_d = weight.to(device).requires_grad_(True)
    lp, ent = areal_amd.lm_head_logprobs_entropy(h_d, w_d, labels.to(device), temperature)
    obj = (lp * gl.to(device)).sum()
    if with_entropy:
        obj = obj + (ent * gh.to(device)).sum()
    obj.backward()
    h_o = hidden.float().requires_grad_(True)
    w_o = weight.float().requires_grad_(True)
    o_lp, o_ent = oracle.logprobs_entropy(h_o @ w_o.t(), labels, temperature)
    ref = (o_lp * gl).sum() + ((o_ent * gh).sum() if with_entropy else 0.0)
    ref.backward()
    assert h_d.grad.dtype == torch.bfloat16 and w_d.grad.dtype == torch.bfloat16
    assert cosine(h_d.grad.cpu(), h_o.grad) > 0.9999
    assert cosine(w_d.grad.cpu(), w_o.grad) > 0.9999
    assert float((h_d.grad.cpu().float() - h_o.grad).abs().max()) < 0.02 * float(h_o.grad.abs().max()) + 1e-6
    assert float((w_d.grad.cpu().float() - w_o.grad).abs().max()) < 0.02 * float(w_o.grad.abs().max()) + 1e-6


def test_lm_head_into_ppo_loss_end_to_end(device):
    """hidden -> fused lm_head -> PPO loss -> backward, against the oracle pipeline on materialised logits."""
    T, H, V = 384, 128, 1600
    hidden, weight, labels = _case(T, H, V, seed=11, w_std=0.3)
    g = torch.Generator().manual_seed(5)
    logits = oracle.lmhead_logits(hidden, weight)
    ref_lp = oracle.logprobs(logits, labels)
    prox, old = ref_lp + 0.05 * torch.randn(T, generator=g), ref_lp + 0.05 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < 0.7
    h_d = hidden.to(device).requires_grad_(True)
    w_d = weight.to(device).requires_grad_(True)
    lp, ent = areal_amd.lm_head_logprobs_entropy(h_d, w_d, labels.to(device))
    loss, stat = areal_amd.ppo_actor_loss_fn(lp, prox.to(device), old.to(device), adv.to(device), 0.2, mask.to(device),
                                             eps_clip_higher=0.28, c_clip=3.0)
    loss.backward()
    h_o = hidden.float().requires_grad_(True)
    w_o = weight.float().requires_grad_(True)
    o_lp, _ = oracle.logprobs_entropy(h_o @ w_o.t(), labels)
    o_loss, _ = oracle.ppo_actor_loss(o_lp, prox, old, adv, 0.2, mask, 0.28, 3.0)
    o_loss.backward()
    assert float(loss.detach()) == pytest.approx(float(o_loss), rel=1e-3, abs=1e-7)
    assert cosine(h_d.grad.cpu(), h_o.grad) > 0.9999 and cosine(w_d.grad.cpu(), w_o.grad) > 0.9999
