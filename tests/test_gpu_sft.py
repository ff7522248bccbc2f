"""GPU parity of the supervised loss: given log-probs, fused with the log-prob op over the logits, and fused with
the lm_head, against the CPU oracle."""
import pytest
import torch

import areal_amd
import oracle
from areal_amd import engine_glue as G
from helpers import assert_same_magnitude, assert_within, cosine
from oracle.sft import packed_sft_loss

pytestmark = pytest.mark.gpu


def _packed(lens, seed, p=0.6):
    g = torch.Generator().manual_seed(seed)
    cu = torch.tensor([0] + lens, dtype=torch.int64).cumsum(0).to(torch.int32)
    T = int(cu[-1])
    mask = torch.rand(T, generator=g) < p
    return g, cu, T, mask


def _check_stat(stat, w_stat, n_seqs):
    assert torch.equal(stat["n_seqs"].cpu(), w_stat["n_seqs"])
    assert stat["seqlogp"].dtype == torch.float64 and stat["seqlogp"].shape == (n_seqs,)
    assert torch.allclose(stat["seqlogp"].cpu(), w_stat["seqlogp"], rtol=1e-6, atol=1e-6)
    assert torch.allclose(stat["ppl"].cpu(), w_stat["ppl"], rtol=1e-5)


@pytest.mark.parametrize("lens", [[5, 1, 0, 9, 3], [3000, 17, 0, 0, 4096, 1], [40000]])
def test_sft_loss_fn_matches_oracle(device, lens):
    g, cu, T, mask = _packed(lens, 3)
    if len(lens) > 3:
        mask[cu[3]:cu[4]] = False          # a sequence without a selected token
    lp = -torch.rand(T, generator=g) * 4
    x = lp.clone().requires_grad_(True)
    w_loss, w_stat = packed_sft_loss(x, mask, cu.long())
    (2.5 * w_loss).backward()
    y = lp.to(device).requires_grad_(True)
    loss, stat = areal_amd.sft_loss_fn(y, mask.to(device), cu.to(device))
    (2.5 * loss).backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=2e-6)
    assert torch.allclose(y.grad.cpu(), x.grad, rtol=1e-6, atol=0)
    assert torch.equal(stat["loss"].cpu(), w_stat["loss"])
    _check_stat(stat, w_stat, len(lens))
    # the loss function of the trainer
    inp = dict(loss_mask=mask.to(device), cu_seqlens=cu.to(device))
    loss2, st2 = G.compute_packed_sft_loss(lp.to(device), None, inp)
    assert float(loss2) == float(loss.detach())
    assert float(st2["reduced"]["loss"]["sum"]) == pytest.approx(float(w_stat["loss"][mask].sum()), rel=1e-5)
    assert st2["reduced"]["n_tokens"] == T


def test_sft_loss_fn_edge_cases(device):
    lp = -torch.rand(10)
    none = torch.zeros(10, dtype=torch.bool)
    loss, stat = areal_amd.sft_loss_fn(lp.to(device), none.to(device), torch.tensor([0, 4, 10], device=device))
    assert float(loss) == 0.0 and not stat["n_seqs"].any() and stat["ppl"].tolist() == [1.0, 1.0]
    # no cu_seqlens: the loss alone; a loss scale multiplies loss and gradient
    x = lp.to(device).requires_grad_(True)
    loss, stat = areal_amd.sft_loss_fn(x, torch.ones(10, dtype=torch.bool, device=device), None, loss_scale=0.5)
    loss.backward()
    assert float(loss.detach()) == pytest.approx(-0.5 * float(lp.sum()) / (10 + 1e-5), rel=1e-6)
    assert torch.allclose(x.grad.cpu(), torch.full((10,), -0.5 / (10 + 1e-5)))
    assert stat["ppl"].numel() == 0
    with pytest.raises(ValueError):
        areal_amd.sft_loss_fn(lp.to(device), none[:5].to(device))


@pytest.mark.parametrize("V,dtype,temperature", [(151936, torch.bfloat16, 1.0), (32000, torch.float16, 0.7),
                                                 (1000, torch.float32, 1.0), (262144, torch.bfloat16, 1.0)])
def test_fused_logits_sft_matches_oracle(device, V, dtype, temperature):
    lens = [37, 5, 0, 64, 22]
    g, cu, T, mask = _packed(lens, 7)
    T_pad = T + 6                                               # batch padding rows after the tokens
    logits = (3 * torch.randn(T_pad, V, generator=g)).to(dtype)
    labels = torch.randint(0, V, (T_pad,), generator=g)
    xx = logits.clone().requires_grad_(True)
    w_logp = oracle.logprobs(xx, labels, temperature)[:T]
    w_loss, w_stat = packed_sft_loss(w_logp, mask, cu.long())
    (0.3 * w_loss).backward()
    y = logits.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_logprobs_sft_loss(y, labels.to(device), mask.to(device), cu.to(device), temperature,
                                                   loss_scale=0.3)
    loss.backward()
    assert float(loss.detach()) == pytest.approx(0.3 * float(w_loss.detach()), rel=1e-3)
    assert float((stat["logprobs"].cpu() - w_logp.detach()).abs().max()) < 2e-3
    assert float((stat["loss"].cpu() + torch.where(mask, stat["logprobs"].cpu(), torch.tensor(0.0))).abs().max()) == 0.0
    _check_stat(stat, w_stat, len(lens))
    assert cosine(y.grad.float().cpu(), xx.grad.float()) > 0.9999
    assert not y.grad[T:].any() and not y.grad[:T][~mask.to(device)].any()
    # forward only: same loss, no gradient buffer
    with torch.no_grad():
        loss_f, stat_f = areal_amd.fused_logprobs_sft_loss(logits.to(device), labels.to(device), mask.to(device),
                                                           cu.to(device), temperature, loss_scale=0.3)
    assert float(loss_f) == pytest.approx(float(loss.detach()), rel=1e-6)
    assert torch.equal(stat_f["n_seqs"], stat["n_seqs"])


@pytest.mark.parametrize("skip", [True, False])
def test_fused_lm_head_sft_matches_oracle(device, skip):
    T, H, V = 700, 256, 4096
    lens = [300, 0, 250, 150]
    g, cu, _, mask = _packed(lens, 11, p=0.5)
    mask[:120] = False                                          # a prompt
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (0.05 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    h = hidden.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    w_logp = oracle.logprobs(oracle.lmhead_logits(h, w), labels, 1.0)
    w_loss, w_stat = packed_sft_loss(w_logp, mask, cu.long())
    w_loss.backward()
    hd = hidden.to(device).requires_grad_(True)
    wd = weight.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_sft_loss(hd, wd, labels.to(device), mask.to(device), cu.to(device),
                                                  skip_masked_tokens=skip)
    loss.backward()
    assert float(loss.detach()) == pytest.approx(float(w_loss.detach()), rel=1e-3)
    assert_within(stat["logprobs"].cpu(), w_logp.detach(), 2e-3, "log-prob")
    _check_stat(stat, w_stat, len(lens))
    assert cosine(hd.grad.float().cpu(), h.grad.float()) > 0.9999
    assert cosine(wd.grad.float().cpu(), w.grad.float()) > 0.9999
    assert_same_magnitude(hd.grad.float(), h.grad.float(), what="d(hidden)")
    assert_same_magnitude(wd.grad.float(), w.grad.float(), what="d(W)")
    assert not hd.grad[~mask.to(device)].any()
    with torch.no_grad():
        loss_f, _ = areal_amd.fused_lm_head_sft_loss(hidden.to(device), weight.to(device), labels.to(device),
                                                     mask.to(device), cu.to(device))
    assert float(loss_f) == pytest.approx(float(loss.detach()), rel=1e-4)


def test_engine_glue_generic_and_fused_sft_agree(device):
    """fsdp_engine.py:1977-2046 with the supervised loss function: the generic glue (log-prob op, trim, loss function,
    scale) and the fused step give the same loss and the same gradient of the logits."""
    lens = [30, 11, 0, 25]
    g, cu, T, mask = _packed(lens, 21)
    pad = 8
    V = 8200
    ids = torch.randint(0, V, (T + pad,), generator=g)
    logits = (2 * torch.randn(T + pad, V, generator=g)).bfloat16()
    model_inputs = dict(input_ids=ids.to(device)[None])
    mb = dict(loss_mask=mask.to(device), cu_seqlens=cu.to(device))
    total = 3.0 * int(mask.sum())
    x = logits.to(device).requires_grad_(True)
    loss, stat = G.compute_loss_with(x, model_inputs, mb, pad, G.compute_packed_sft_loss,
                                     lambda d: d["loss_mask"].count_nonzero(), total, loss_multiplier=2.0)
    loss.backward()
    y = logits.to(device).requires_grad_(True)
    loss_f, stat_f = G.compute_logprobs_and_sft_loss(y, model_inputs, mb, total, loss_multiplier=2.0)
    loss_f.backward()
    assert float(loss_f.detach()) == pytest.approx(float(loss.detach()), rel=1e-5)
    assert torch.equal(stat_f["n_seqs"], stat["n_seqs"]) and torch.allclose(stat_f["ppl"], stat["ppl"], rtol=1e-5)
    assert cosine(x.grad.float().cpu(), y.grad.float().cpu()) > 0.99999 and not y.grad[T:].any()
    # against the oracle: labels rolled over the whole padded tensor, loss scaled by local / total * multiplier
    labels = torch.roll(ids, -1)
    w_logp = oracle.logprobs(logits, labels, 1.0)[:T]
    w_loss, _ = packed_sft_loss(w_logp, mask, cu.long())
    assert float(loss.detach()) == pytest.approx(float(w_loss) * int(mask.sum()) / total * 2.0, rel=1e-3)
    # a loss function that returns the loss alone, and a micro-batch without weight
    only = G.compute_loss_with(logits.to(device), model_inputs, mb, pad, lambda lp, ent, d, **kw: lp.sum(),
                               lambda d: d["loss_mask"].count_nonzero(), total)
    assert only.ndim == 0
    none = dict(mb, loss_mask=torch.zeros_like(mb["loss_mask"]))
    assert float(G.compute_loss_with(logits.to(device), model_inputs, none, pad, G.compute_packed_sft_loss,
                                     lambda d: d["loss_mask"].count_nonzero(), total)) == 0.0


def test_second_backward_of_the_small_losses_is_not_rescaled(device):
    """The per-token gradients of the losses on log-probs / scores are copied before the upstream factor is applied,
    so a second backward through a retained graph gives the same gradient."""
    lp = (-torch.rand(50)).to(device).requires_grad_(True)
    mask = torch.rand(50, device=device) < 0.7
    loss, _ = areal_amd.sft_loss_fn(lp, mask, torch.tensor([0, 20, 50], device=device))
    (g1,) = torch.autograd.grad(3.0 * loss, lp, retain_graph=True)
    (g2,) = torch.autograd.grad(3.0 * loss, lp)
    assert torch.equal(g1, g2)
    s = torch.randn(50, device=device, requires_grad=True)
    loss, _ = areal_amd.rw_pair_loss(s, torch.tensor([0, 20, 50], device=device))
    (g1,) = torch.autograd.grad(0.5 * loss, s, retain_graph=True)
    (g2,) = torch.autograd.grad(0.5 * loss, s)
    assert torch.equal(g1, g2) and int((g1 != 0).sum()) == 2


def test_full_size_supervised_lm_head_step(device):
    """configs[2] shape (hidden [16384, 4096], W [151936, 4096]): the chunked supervised step against the stand-alone
    lm_head op followed by the loss on log-probs and autograd; bit-identical when repeated; prompt tokens (the masked
    30 % of every sequence) get no gradient."""
    from areal_amd import synth

    case = synth.config2(device, seed=0)

    def fused():
        h = case.hidden.detach().requires_grad_(True)
        w = case.weight.detach().requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_sft_loss(h, w, case.labels, case.loss_mask, case.cu_seqlens, loss_scale=0.5)
        loss.backward()
        return loss.detach(), stat, h.grad, w.grad

    l1, s1, dh1, dw1 = fused()
    l2, _, dh2, dw2 = fused()
    assert torch.equal(l1, l2) and torch.equal(dh1, dh2) and torch.equal(dw1, dw2)
    h = case.hidden.detach().requires_grad_(True)
    w = case.weight.detach().requires_grad_(True)
    lp, _ = areal_amd.lm_head_logprobs_entropy(h, w, case.labels)
    loss, stat = areal_amd.sft_loss_fn(lp, case.loss_mask, case.cu_seqlens, loss_scale=0.5)
    loss.backward()
    assert float(l1) == pytest.approx(float(loss.detach()), rel=1e-3)
    assert torch.equal(s1["n_seqs"], stat["n_seqs"]) and torch.allclose(s1["ppl"], stat["ppl"], rtol=2e-3)
    assert cosine(dh1.float().cpu(), h.grad.float().cpu()) > 0.9999
    assert cosine(dw1.float().cpu(), w.grad.float().cpu()) > 0.9999
    assert not dh1[~case.loss_mask.bool()].any()
