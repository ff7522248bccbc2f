"""GPU parity of the whole lm_head + PPO-loss training step (``fused_lm_head_ppo_loss``).

Oracle: the reference pipeline on materialised fp32 logits -- lm_head matmul, log-softmax / gather / entropy,
``ppo_actor_loss_fn`` with rejection sampling, autograd back to the hidden states and the lm_head weight.  Both ways
of obtaining the d(logits) rows of the backward (``backward="recompute"`` and ``"carry"``) are held to it."""
import pytest
import torch

import areal_amd
import oracle
from areal_amd import _native, engine_glue
from areal_amd import RejectionSamplingConfig
from helpers import assert_same_magnitude, assert_within, cosine

pytestmark = pytest.mark.gpu

CHUNK = int(_native.load().aa_lmhead_chunk_tokens())  # tokens per chunk of the lm_head entry points


def _inputs(T_pad, T, H, V, seed, w_std=0.3):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T_pad, H, generator=g).bfloat16()
    weight = (w_std * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T_pad,), generator=g)
    logits = oracle.lmhead_logits(hidden, weight)
    ref_lp = oracle.logprobs(logits, labels)[:T]
    prox = ref_lp + 0.05 * torch.randn(T, generator=g)
    old = ref_lp + 0.3 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < 0.7
    return hidden, weight, labels, prox, old, adv, mask


def _oracle_step(hidden, weight, labels, prox, old, adv, mask, temperature, loss_scale, **kw):
    h = hidden.float().requires_grad_(True)
    w = weight.float().requires_grad_(True)
    logits = oracle.lmhead_logits(h, w)
    lp, ent = oracle.logprobs_entropy(logits, labels, temperature)
    n = mask.shape[0]
    loss, stat = oracle.ppo_actor_loss(lp[:n], prox, old, adv, loss_mask=mask, **kw)
    (loss * loss_scale).backward()
    return float(loss.detach()) * loss_scale, stat, lp.detach(), ent.detach(), h.grad, w.grad


CASES = [
    # T_pad, T, H, V, temperature, loss_scale, options
    (300, 300, 128, 1088, 1.0, 1.0, dict(eps_clip=0.2)),                                    # ragged last tiles
    (520, 500, 64, 8256, 0.8, 0.37, dict(eps_clip=0.2, eps_clip_higher=0.28, c_clip=3.0)),  # batch padding, dual clip
    (CHUNK + 200, CHUNK + 130, 64, 640, 1.0, 1.0, dict(eps_clip=0.2, rs=True)),             # two token chunks
    (203, 203, 200, 1096, 1.3, 1.0, dict(eps_clip=0.2)),                                    # H, V multiples of 8 only
    (203, 190, 72, 1097, 0.7, 1.0, dict(eps_clip=0.2, c_clip=3.0)),                         # any vocabulary size
    (96, 90, 64, 50257, 1.0, 1.0, dict(eps_clip=0.2)),
    (64, 60, 64, 151643, 1.0, 0.5, dict(eps_clip=0.2, rs=True)),
]


@pytest.mark.parametrize("backward", ["carry", "recompute"])
@pytest.mark.parametrize("T_pad,T,H,V,temperature,loss_scale,opts", CASES)
def test_step_matches_reference_pipeline(device, T_pad, T, H, V, temperature, loss_scale, opts, backward):
    opts = dict(opts)
    rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", upper=1.3) if opts.pop("rs", False) else None
    hidden, weight, labels, prox, old, adv, mask = _inputs(T_pad, T, H, V, seed=T + V)
    cu = torch.tensor([0, T], dtype=torch.int32)
    h_d = hidden.to(device).requires_grad_(True)
    w_d = weight.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_ppo_loss(
        h_d, w_d, labels.to(device), prox.to(device), old.to(device), adv.to(device), loss_mask=mask.to(device),
        rejection_sampling=rs, cu_seqlens=cu.to(device), temperature=temperature, loss_scale=loss_scale,
        backward=backward, **opts)
    loss.backward()
    o_loss, o_stat, o_lp, o_ent, o_dh, o_dw = _oracle_step(
        hidden, weight, labels, prox, old, adv, mask, temperature, loss_scale, rejection_sampling_cfg=rs,
        cu_seqlens=cu, **opts)
    assert float(loss.detach()) == pytest.approx(o_loss, rel=1e-3)  # stated tolerances
    assert_within(stat["logprobs"], o_lp[:T], 2e-3, "log-prob")
    assert_within(stat["entropy"], o_ent[:T], 2e-3, "entropy")
    logits = oracle.lmhead_logits(hidden, weight)[:T]  # what the engine would take the extrema of (fsdp_engine.py:1893-1906)
    assert float((stat["vocab_max_logits"].cpu() - logits.max(-1).values).abs().max()) <= 1e-5 * float(logits.abs().max())
    assert float((stat["vocab_min_logits"].cpu() - logits.min(-1).values).abs().max()) <= 1e-5 * float(logits.abs().max())
    for k in ("clip_mask", "dual_clip_mask"):   # a flag can only differ where the ratio sits on a clip boundary
        assert int((stat[k].cpu() != o_stat[k]).sum()) <= 1, k
    assert cosine(h_d.grad.cpu().float(), o_dh) > 0.9999
    assert cosine(w_d.grad.cpu().float(), o_dw) > 0.9999
    assert_same_magnitude(h_d.grad, o_dh, what="d(hidden)")  # a wrong 1/n, loss scale or temperature shows here
    assert_same_magnitude(w_d.grad, o_dw, what="d(W)")
    assert float(h_d.grad[T:].abs().sum()) == 0.0  # batch padding gets no gradient
    if rs is not None:
        assert float(stat["filtered_fraction"]) == pytest.approx(float(o_stat["filtered_fraction"]), abs=1e-6)


def test_carry_and_recompute_give_the_same_step(device):
    """The two ways of filling the d(logits) rows: identical forward results, gradients equal up to the extra bf16
    rounding of the carried probabilities; with and without the rows of masked tokens left out."""
    hidden, weight, labels, prox, old, adv, mask = _inputs(900, 840, 128, 4160, seed=17)
    args = [t.to(device) for t in (labels, prox, old, adv)]

    def run(backward, skip):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device), c_clip=3.0,
                                                      temperature=0.9, backward=backward, skip_masked_tokens=skip)
        loss.backward()
        return loss.detach(), stat, h.grad.float(), w.grad.float()

    ref = run("recompute", False)
    for backward, skip in (("carry", False), ("carry", True), ("recompute", True)):
        got = run(backward, skip)
        assert torch.equal(got[0], ref[0])
        for k in ("logprobs", "entropy", "loss", "importance_weight", "clip_mask", "dual_clip_mask"):
            assert torch.equal(got[1][k], ref[1][k]), k
        for a, b in ((got[2], ref[2]), (got[3], ref[3])):
            assert cosine(a.cpu(), b.cpu()) > 0.99999
            assert_same_magnitude(a, b, rel=2e-3)


def test_carry_redoes_a_chunk_whose_labels_are_too_unlikely_to_store(device):
    """Carry mode stores p_v / p_label in bf16; a token with a gradient whose label has a log-prob below -80 does not
    fit that range, and its chunk is redone by the recompute tiles, decided on the device.  Logits with a spread of
    about 48 put many labels there; the second chunk of the batch has ordinary logits and stays on the carried rows.
    Both must match the oracle and the recompute mode."""
    T, H, V = CHUNK + 300, 64, 1088
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(T, H, generator=g)
    hidden[:CHUNK] *= 12.0                     # first chunk: logits ~ N(0, 48^2)
    hidden = hidden.bfloat16()
    weight = (0.5 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    ref_lp = oracle.logprobs(oracle.lmhead_logits(hidden, weight), labels)
    assert int((ref_lp[:CHUNK] < -80).sum()) > 100 and float(ref_lp[CHUNK:].min()) > -60
    prox = ref_lp + 0.05 * torch.randn(T, generator=g)
    old = ref_lp + 0.3 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < 0.7
    args = [t.to(device) for t in (labels, prox, old, adv)]

    def run(backward):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device), backward=backward)
        loss.backward()
        return loss.detach(), stat, h.grad.float(), w.grad.float()

    o_loss, _, o_lp, _, o_dh, o_dw = _oracle_step(hidden, weight, labels, prox, old, adv, mask, 1.0, 1.0, eps_clip=0.2)
    ref = run("recompute")
    got = run("carry")
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1]["logprobs"], ref[1]["logprobs"])
    assert_within(got[1]["logprobs"], o_lp, 2e-3, "log-prob")
    assert float(got[0]) == pytest.approx(o_loss, rel=1e-3)
    for name, a, b, o in (("d(hidden)", got[2], ref[2], o_dh), ("d(W)", got[3], ref[3], o_dw)):
        assert torch.isfinite(a).all(), name
        assert cosine(a.cpu(), o) > 0.9999, name
        assert_same_magnitude(a, o, what=name)
        assert cosine(a.cpu(), b.cpu()) > 0.99999, name
    # the flagged chunk came out of the recompute tiles: its d(hidden) rows are those of the recompute mode, bit for bit
    assert torch.equal(got[2][:CHUNK], ref[2][:CHUNK])


@pytest.mark.parametrize("backward", ["carry", "recompute"])
def test_gradient_products_with_more_tiles_than_compute_units(device, backward):
    """9 x 30 = 270 tiles of d(hidden) and 5 x 9 tiles of d(W) with 7600 rows to contract: a grid larger than the chip,
    with a partly filled last round and ragged edges in both products.  Against the oracle row by row, and bit-equal
    from call to call."""
    T, H, V = 7600, 2304, 1088
    hidden, weight, labels, prox, old, adv, mask = _inputs(T, T, H, V, seed=23, w_std=0.05)
    mask[:] = True
    args = [t.to(device) for t in (labels, prox, old, adv)]

    def run():
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device), backward=backward)
        loss.backward()
        return loss.detach(), h.grad, w.grad

    o_loss, _, _, _, o_dh, o_dw = _oracle_step(hidden, weight, labels, prox, old, adv, mask, 1.0, 1.0, eps_clip=0.2)
    loss, dh, dw = run()
    assert float(loss) == pytest.approx(o_loss, rel=1e-3)
    assert cosine(dh.cpu().float(), o_dh) > 0.9999 and cosine(dw.cpu().float(), o_dw) > 0.9999
    assert_same_magnitude(dh, o_dh, what="d(hidden)")
    assert_same_magnitude(dw, o_dw, what="d(W)")
    # row by row: one wrong tile would spoil 256 tokens x 256 columns and leave the norms nearly intact
    err = (dh.cpu().float() - o_dh).abs().amax(dim=1)
    assert float(err.max()) <= float(o_dh.abs().max()) * 2.0 ** -7
    loss2, dh2, dw2 = run()
    assert torch.equal(dh, dh2) and torch.equal(dw, dw2) and torch.equal(loss, loss2)


@pytest.mark.parametrize("backward", ["carry", "recompute"])
@pytest.mark.parametrize("T,H,V", [(300, 128, 16640), (700, 320, 20488)])
def test_hidden_gradient_cut_along_the_vocabulary(device, backward, T, H, V):
    """Few tiles of d(hidden) and a long vocabulary to contract (260 and 321 slices of 64): the product is cut into
    parts along the vocabulary, every part sums into its own fp32 plane and the planes are added in a fixed order
    (the last part is short and ragged).  Against the oracle row by row, bit-equal from call to call, masked tokens
    with a zero row."""
    hidden, weight, labels, prox, old, adv, mask = _inputs(T, T, H, V, seed=V, w_std=0.05)
    args = [t.to(device) for t in (labels, prox, old, adv)]

    def run():
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device), backward=backward)
        loss.backward()
        return loss.detach(), h.grad, w.grad

    o_loss, _, _, _, o_dh, o_dw = _oracle_step(hidden, weight, labels, prox, old, adv, mask, 1.0, 1.0, eps_clip=0.2)
    loss, dh, dw = run()
    assert float(loss) == pytest.approx(o_loss, rel=1e-3)
    assert cosine(dh.cpu().float(), o_dh) > 0.9999 and cosine(dw.cpu().float(), o_dw) > 0.9999
    assert_same_magnitude(dh, o_dh, what="d(hidden)")
    err = (dh.cpu().float() - o_dh).abs().amax(dim=1)
    assert float(err.max()) <= float(o_dh.abs().max()) * 2.0 ** -7
    assert float(dh[~mask.to(device)].float().abs().max()) == 0.0
    loss2, dh2, dw2 = run()
    assert torch.equal(dh, dh2) and torch.equal(dw, dw2) and torch.equal(loss, loss2)


def test_upstream_gradient_scales_both_gradients(device):
    hidden, weight, labels, prox, old, adv, mask = _inputs(260, 260, 64, 704, seed=3)
    args = [t.to(device) for t in (labels, prox, old, adv)]

    def grads(factor):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, _ = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device))
        (loss * factor).backward()
        return h.grad.float(), w.grad.float()

    h1, w1 = grads(1.0)
    h2, w2 = grads(-2.0)
    assert torch.allclose(h2, -2.0 * h1, rtol=1e-2, atol=1e-12) and torch.allclose(w2, -2.0 * w1, rtol=1e-2, atol=1e-12)


@pytest.mark.parametrize("carry_limit", [16 << 30, 0])   # the op keeps its rows for the backward / forms the logits again
def test_sequence_level_runs_the_unfused_kernels(device, carry_limit):
    hidden, weight, labels, prox, old, adv, mask = _inputs(320, 300, 64, 704, seed=5)
    cu = torch.tensor([0, 100, 180, 300], dtype=torch.int32)
    h_d = hidden.to(device).requires_grad_(True)
    w_d = weight.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_ppo_loss(
        h_d, w_d, labels.to(device), prox.to(device), old.to(device), adv.to(device), eps_clip=0.2,
        loss_mask=mask.to(device), importance_sampling_level="sequence", cu_seqlens=cu.to(device),
        carry_rows_limit_bytes=carry_limit)
    loss.backward()
    hidden, labels = hidden[:300], labels[:300]            # the oracle sees the tokens without the batch padding
    assert float(h_d.grad[300:].float().abs().sum()) == 0.0
    dh = h_d.grad[:300]
    h = hidden.float().requires_grad_(True)
    w = weight.float().requires_grad_(True)
    lp, _ = oracle.logprobs_entropy(h @ w.t(), labels)
    o_loss, _ = oracle.ppo_actor_loss(lp, prox, old, adv, 0.2, mask, importance_sampling_level="sequence", cu_seqlens=cu)
    o_loss.backward()
    assert float(loss.detach()) == pytest.approx(float(o_loss.detach()), rel=1e-3)
    assert cosine(dh.cpu().float(), h.grad) > 0.9999 and cosine(w_d.grad.cpu().float(), w.grad) > 0.9999
    assert_same_magnitude(dh, h.grad, what="d(hidden)")
    assert_same_magnitude(w_d.grad, w.grad, what="d(W)")
    with pytest.raises(ValueError, match="backward must be one of"):
        areal_amd.fused_lm_head_ppo_loss(h_d, w_d, labels.to(device), prox.to(device), old.to(device), adv.to(device),
                                         eps_clip=0.2, loss_mask=mask.to(device), backward="panel")
    with pytest.raises(ValueError, match="Invalid importance_sampling_level"):
        areal_amd.fused_lm_head_ppo_loss(h_d, w_d, labels.to(device), prox.to(device), old.to(device), adv.to(device),
                                         eps_clip=0.2, loss_mask=mask.to(device), importance_sampling_level="bad")


@pytest.mark.parametrize("backward", ["carry", "recompute"])
def test_full_size_step_agrees_with_unfused_path(device, backward):
    """8B shape: the chunked step against lm_head_logprobs_entropy -> ppo_actor_loss_fn -> autograd (which the slice
    tests tie to the oracle); also bit-identical when repeated."""
    from areal_amd import synth

    case = synth.config2(device, seed=0)
    with torch.no_grad():
        ref, _ = areal_amd.lm_head_logprobs_entropy(case.hidden, case.weight, case.labels)
    synth.attach_old_and_prox(case, ref, 0.05, 9)

    def fused():
        h = case.hidden.detach().requires_grad_(True)
        w = case.weight.detach().requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, case.labels, case.prox_logp, case.old_logp,
                                                      case.advantages, eps_clip=0.2, loss_mask=case.loss_mask,
                                                      backward=backward)
        loss.backward()
        return loss.detach(), stat, h.grad, w.grad

    l1, s1, dh1, dw1 = fused()
    l2, s2, dh2, dw2 = fused()
    assert torch.equal(l1, l2) and torch.equal(dh1, dh2) and torch.equal(dw1, dw2)
    h = case.hidden.detach().requires_grad_(True)
    w = case.weight.detach().requires_grad_(True)
    lp, ent = areal_amd.lm_head_logprobs_entropy(h, w, case.labels)
    loss, stat = areal_amd.ppo_actor_loss_fn(lp, case.prox_logp, case.old_logp, case.advantages, 0.2, case.loss_mask)
    loss.backward()
    assert float(l1) == pytest.approx(float(loss.detach()), rel=1e-5)
    # the same forward tiles, merged by two different kernels: a few ulp of values near 11 (ulp 9.5e-7)
    assert torch.allclose(s1["logprobs"], lp.detach(), rtol=0, atol=4e-6) and torch.allclose(s1["entropy"], ent.detach(), rtol=0, atol=4e-6)
    for got, want in ((dh1, h.grad), (dw1, w.grad)):
        a, b = got.double().reshape(-1), want.double().reshape(-1)
        assert float(a @ b / (a.norm() * b.norm())) > 0.9999
        assert abs(float(a.norm() / b.norm()) - 1.0) < 1e-2
        assert float((a - b).abs().max()) <= float(b.abs().max()) * 2.0 ** -6


def _full_size_case(name, device):
    """configs[3] / configs[4] as the benchmark builds them, with old / prox log-probs spread widely enough (0.6 nats)
    that the dual clip and the importance-weight cap both bind on a few percent of the tokens."""
    from areal_amd import synth

    case = {"cfg3": synth.config3, "cfg4": synth.config4}[name](device, seed=0)
    with torch.no_grad():
        ref, _ = areal_amd.lm_head_logprobs_entropy(case.hidden, case.weight, case.labels, case.temperature)
    synth.attach_old_and_prox(case, ref, 0.6, 9)
    kw = dict(case.ppo)
    rs = kw.pop("rejection_sampling", None)
    kw.setdefault("c_clip", 3.0)                       # configs[4] names no dual clip: switch it on for the test
    cfg = RejectionSamplingConfig(**(rs or dict(level="token", action="mask", metric="ratio", upper=5.0)))
    return case, kw, cfg


@pytest.mark.parametrize("backward", ["carry", "recompute"])
@pytest.mark.parametrize("name", ["cfg4", "cfg3"])
def test_full_size_step_against_oracle_slices(device, name, backward):
    """The whole step at the size of configs[3] (T = 262144: 16 token chunks, d(W) accumulated in fp32 chunk by chunk)
    and configs[4] (V = 262144, H = 5376, temperature 0.7, two chunks).  The oracle cannot run these whole.  A token's
    log-prob, entropy, loss terms and d(hidden) row depend on that token and on the number of unmasked tokens only, so
    48 tokens (first, middle, last) are held to the oracle; d(W) is held to it with only those tokens switched on, and
    the full d(W) to the sum of that and of the step on all other tokens (the loss is additive over tokens once the
    common 1/N is kept)."""
    case, kw, cfg = _full_size_case(name, device)
    T, H = case.hidden.shape
    V = case.weight.shape[0]
    print(f"full-size step {name} {backward}: T={T} H={H} V={V}", flush=True)
    idx = torch.cat([torch.arange(0, 16), torch.arange(T // 2 - 8, T // 2 + 8), torch.arange(T - 16, T)])
    idx_d = idx.to(device)
    n_full = int(case.loss_mask.sum())
    in_slice = torch.zeros(T, dtype=torch.bool, device=device)
    in_slice[idx_d] = True
    slice_mask = case.loss_mask.bool() & in_slice
    rest_mask = case.loss_mask.bool() & ~in_slice
    n_slice = int(slice_mask.sum())
    assert 8 <= n_slice < 48            # the slice holds masked and unmasked tokens

    def step(mask, scale):
        h = case.hidden.detach().requires_grad_(True)
        w = case.weight.detach().requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(
            h, w, case.labels, case.prox_logp, case.old_logp, case.advantages, loss_mask=mask, rejection_sampling=cfg,
            cu_seqlens=case.cu_seqlens, temperature=case.temperature, loss_scale=scale, backward=backward, **kw)
        loss.backward()
        return loss.detach(), stat, h.grad, w.grad

    loss, stat, dh, dw = step(case.loss_mask, 1.0)
    assert bool(torch.isfinite(loss)) and bool(torch.isfinite(dw.float()).all())
    assert int(stat["dual_clip_mask"].sum()) > 100 and float(stat["filtered_fraction"]) > 0.005   # both bind
    # oracle on the slice, with the full batch's 1/N
    take = lambda t: t[idx_d].cpu()
    h_o = case.hidden[idx_d].cpu().float().requires_grad_(True)
    w_o = case.weight.cpu().float().requires_grad_(True)
    o_lp, o_ent = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), take(case.labels), case.temperature)
    o_loss, o_stat = oracle.ppo_actor_loss(
        o_lp, take(case.prox_logp), take(case.old_logp), take(case.advantages), loss_mask=take(case.loss_mask).bool(),
        rejection_sampling_cfg=cfg, cu_seqlens=torch.tensor([0, idx.numel()], dtype=torch.int32), **kw)
    (o_loss * n_slice / n_full).backward()
    assert_within(stat["logprobs"][idx_d], o_lp.detach(), 2e-3, "log-prob")       # stated tolerances
    assert_within(stat["entropy"][idx_d], o_ent.detach(), 2e-3, "entropy")
    on = take(case.loss_mask).bool()
    assert_within(stat["loss"][idx_d].cpu()[on], o_stat["loss"][on], 2e-3, "per-token loss")
    assert int((stat["clip_mask"][idx_d].cpu() != o_stat["clip_mask"]).sum()) <= 1
    assert cosine(dh[idx_d].cpu().float(), h_o.grad) > 0.9999
    assert_same_magnitude(dh[idx_d], h_o.grad, what="d(hidden) rows of the slice")
    # tokens without a mask, and tokens the cap dropped, get a d(hidden) row of exactly zero
    dead = ~(case.loss_mask.bool() & stat["behave_mask"].bool())
    assert float(dh[dead].float().abs().sum()) == 0.0
    # bit-equal repeat
    loss2, _, dh2, dw2 = step(case.loss_mask, 1.0)
    assert torch.equal(loss, loss2) and torch.equal(dh, dh2) and torch.equal(dw, dw2)
    del dh2, dw2
    # d(W) with only the slice's tokens switched on (every other chunk has no token with a gradient) against the oracle
    _, _, dh_s, dw_s = step(slice_mask, n_slice / n_full)
    a, b = dw_s.double().reshape(-1), w_o.grad.to(device).double().reshape(-1)
    assert float(a @ b / (a.norm() * b.norm())) > 0.9999
    assert abs(float(a.norm() / b.norm()) - 1.0) < 1e-2
    assert cosine(dh_s[idx_d].cpu().float(), dh[idx_d].cpu().float()) > 0.99999   # the rows of the full step (1/N rounds differently)
    del a, b, w_o, h_o
    # ... and the full d(W) is that plus d(W) of all other tokens
    _, _, _, dw_r = step(rest_mask, (n_full - n_slice) / n_full)
    a, b = (dw_s.float() + dw_r.float()).double().reshape(-1), dw.double().reshape(-1)
    assert float(a @ b / (a.norm() * b.norm())) > 0.99999
    assert abs(float(a.norm() / b.norm()) - 1.0) < 2e-3


def test_padding_only_chunk_and_no_active_token(device):
    g = torch.Generator().manual_seed(0)
    T_pad, T, H, V = CHUNK + 300, CHUNK, 64, 640           # the second token chunk is batch padding only
    hidden = torch.randn(T_pad, H, generator=g).bfloat16().to(device).requires_grad_(True)
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16().to(device).requires_grad_(True)
    labels = torch.randint(0, V, (T_pad,), generator=g).to(device)
    z = torch.zeros(T, device=device)
    mask = (torch.rand(T, generator=g) < 0.7).to(device)
    loss, _ = areal_amd.fused_lm_head_ppo_loss(hidden, weight, labels, z - 6.0, z - 6.0,
                                               torch.randn(T, generator=g).to(device), 0.2, mask)
    loss.backward()
    assert float(hidden.grad[T:].abs().sum()) == 0.0 and bool(torch.isfinite(weight.grad).all())
    # no active token at all: zero loss, zero gradients (both the lm_head step and the logits path)
    e = torch.zeros(0, device=device)
    none = torch.zeros(0, dtype=torch.bool, device=device)
    h2 = hidden.detach()[:50].clone().requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_ppo_loss(h2, weight, labels[:50], e, e, e, 0.2, none)
    loss.backward()
    assert float(loss.detach()) == 0.0 and float(h2.grad.abs().sum()) == 0.0 and stat["logprobs"].numel() == 0
    x = torch.randn(30, 9000, device=device).bfloat16().requires_grad_(True)
    loss, _ = areal_amd.fused_logprobs_ppo_loss(x, labels[:30] % 9000, e, e, e, 0.2, none)
    loss.backward()
    assert float(loss.detach()) == 0.0 and float(x.grad.float().abs().sum()) == 0.0


@pytest.mark.parametrize("pattern", ["random", "second_chunk_masked", "first_chunk_masked", "all_masked", "one_token",
                                     "random_long_rows"])
def test_skipping_masked_tokens_equals_the_dense_backward(device, pattern):
    """Tokens with a zero mask are left out of the gradient GEMMs: same loss and statistics, same gradients as when
    their zero rows are multiplied through (two token chunks, batch padding at the end)."""
    g = torch.Generator().manual_seed(5)
    T_pad, T, H, V = CHUNK + 300, CHUNK + 200, 64, 8200
    if pattern == "random_long_rows":
        V = 180224
    hidden = torch.randn(T_pad, H, generator=g).bfloat16().to(device)
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16().to(device)
    labels = torch.randint(0, V, (T_pad,), generator=g).to(device)
    with torch.no_grad():
        ref, _ = areal_amd.lm_head_logprobs_entropy(hidden, weight, labels)
    ref = ref[:T]
    prox = ref + 0.05 * torch.randn(T, generator=g).to(device)
    old = ref + 0.2 * torch.randn(T, generator=g).to(device)
    adv = torch.randn(T, generator=g).to(device)
    mask = (torch.rand(T, generator=g) < 0.5).to(device)
    if pattern == "second_chunk_masked":
        mask[CHUNK:] = False
    elif pattern == "first_chunk_masked":
        mask[:CHUNK] = False
    elif pattern == "all_masked":
        mask[:] = False
    elif pattern == "one_token":
        mask[:] = False
        mask[CHUNK + 7] = True
    rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", upper=1.3)

    def run(skip):
        h = hidden.clone().requires_grad_(True)
        w = weight.clone().requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, labels, prox, old, adv, 0.2, mask, eps_clip_higher=0.28,
                                                      c_clip=3.0, rejection_sampling=rs, skip_masked_tokens=skip)
        loss.backward()
        return loss.detach(), stat, h.grad.float(), w.grad.float()

    l1, s1, dh1, dw1 = run(True)
    l0, s0, dh0, dw0 = run(False)
    assert torch.equal(l1, l0)
    for k in ("logprobs", "entropy", "loss", "importance_weight", "clip_mask", "dual_clip_mask", "behave_mask"):
        assert torch.equal(s1[k], s0[k]), k
    rows_off = torch.ones(T_pad, dtype=torch.bool, device=device)
    rows_off[:T] = ~s1["behave_mask"]
    assert float(dh1[rows_off].abs().max()) == 0.0
    if pattern == "all_masked":
        assert float(dh1.abs().max()) == 0.0 and float(dw1.abs().max()) == 0.0 and float(dw0.abs().max()) == 0.0
        return
    # different GEMM shapes may sum in a different order: equal up to the bf16 rounding of the outputs
    for a, b in ((dh1, dh0), (dw1, dw0)):
        scale = float(b.abs().max())
        assert float((a - b).abs().max()) <= scale * 2.0 ** -7
        assert cosine(a.cpu(), b.cpu()) > 0.99999


@pytest.mark.parametrize("with_rs", [False, True])
def test_not_forwarding_masked_tokens_keeps_loss_and_gradients(device, with_rs):
    """forward_masked_tokens=False: tokens without a mask never reach the lm_head; loss, gradients and the statistics
    of the other tokens are those of the default call, the masked entries are zero."""
    hidden, weight, labels, prox, old, adv, mask = _inputs(700, 650, 64, 8200, seed=31)
    rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", upper=1.3) if with_rs else None
    args = [t.to(device) for t in (labels, prox, old, adv)]

    def run(forward_masked):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device), c_clip=3.0,
                                                      rejection_sampling=rs, forward_masked_tokens=forward_masked)
        loss.backward()
        return loss.detach(), stat, h.grad.float(), w.grad.float()

    l0, s0, dh0, dw0 = run(True)
    l1, s1, dh1, dw1 = run(False)
    assert float(l1) == pytest.approx(float(l0), rel=1e-5)
    on = s0["behave_mask"] if with_rs else mask.to(device)
    for k in ("logprobs", "entropy", "loss", "importance_weight", "approx_kl"):
        assert torch.allclose(s1[k][on], s0[k][on], rtol=1e-5, atol=1e-6), k
        assert float(s1[k][~on].abs().sum()) == 0.0, k
    for k in ("clip_mask", "dual_clip_mask"):
        assert torch.equal(s1[k], s0[k]), k
    for a, b in ((dh1, dh0), (dw1, dw0)):
        assert float((a - b).abs().max()) <= float(b.abs().max()) * 2.0 ** -7 and cosine(a.cpu(), b.cpu()) > 0.99999
    # nothing valid at all
    none = torch.zeros_like(mask).to(device)
    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=none, forward_masked_tokens=False)
    loss.backward()
    assert float(loss.detach()) == 0.0 and float(h.grad.abs().sum()) == 0.0 and float(w.grad.abs().sum()) == 0.0
    assert float(stat["logprobs"].abs().sum()) == 0.0


def test_counts_from_the_caller_replace_the_read_back(device):
    hidden, weight, labels, prox, old, adv, mask = _inputs(CHUNK + 256, CHUNK + 200, 64, 640, seed=41)
    args = [t.to(device) for t in (labels, prox, old, adv)]
    counts = [int(mask[:CHUNK].sum()), int(mask[CHUNK:].sum())]            # known on the host

    def run(**kw):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, _ = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device), **kw)
        loss.backward()
        return loss.detach(), h.grad, w.grad

    a, b = run(kept_per_chunk=counts), run()
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and torch.equal(a[2], b[2])
    with pytest.raises(ValueError, match="one count per chunk"):
        run(kept_per_chunk=[1])


def _poison_the_allocator_cache(device, nbytes):
    """The workspace of the step is a fresh ``torch.empty``: fill a block of that size with NaN patterns and hand it
    back to the caching allocator, so that rows which nothing writes would show."""
    junk = torch.full((nbytes // 2,), float("nan"), dtype=torch.bfloat16, device=device)
    del junk


@pytest.mark.parametrize("backward", ["carry", "recompute"])
def test_counts_larger_than_the_mask_holds_add_nothing(device, backward):
    """Counts taken from ``loss_mask`` on the host while rejection sampling shrinks the mask on the device: the surplus
    rows have no token.  They are cleared on the device and the results are those of the exact counts."""
    hidden, weight, labels, prox, old, adv, mask = _inputs(CHUNK + 256, CHUNK + 200, 64, 640, seed=43)
    args = [t.to(device) for t in (labels, prox, old, adv)]
    rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", upper=1.2)
    cu = torch.tensor([0, CHUNK + 200], dtype=torch.int32, device=device)
    host_counts = [int(mask[:CHUNK].sum()), int(mask[CHUNK:].sum())]   # before rejection sampling: too large

    def run(**kw):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        _poison_the_allocator_cache(device, int(_native.load().aa_lmhead_workspace_bytes(CHUNK + 256, 64, 640)))
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device),
                                                      rejection_sampling=rs, cu_seqlens=cu, backward=backward, **kw)
        loss.backward()
        return loss.detach(), stat, h.grad, w.grad

    exact, over = run(), run(kept_per_chunk=host_counts)
    assert float(exact[1]["filtered_fraction"]) > 0.05              # the mask did shrink
    assert torch.isfinite(over[2].float()).all() and torch.isfinite(over[3].float()).all()
    assert torch.equal(exact[0], over[0]) and torch.equal(exact[2], over[2])
    # d(W): the same rows in the same order, plus rows of zeros at the end of each chunk
    assert cosine(exact[3].float().cpu(), over[3].float().cpu()) > 0.9999999
    assert_same_magnitude(over[3].float(), exact[3].float(), rel=1e-4)


@pytest.mark.parametrize("backward", ["carry", "recompute"])
@pytest.mark.parametrize("mask_kind", ["mixed", "second_chunk_empty", "nothing", "three_tokens",
                                       "three_tokens_long_rows", "a_tile_and_a_bit_long_rows"])
def test_rows_counted_on_the_device_match_host_counts(device, backward, mask_kind):
    """The default (``count_on_device=True``: the kernels are queued for every token that could have a row and stop at
    the rows in use, which only the device knows) against counts read back by the host and against counts passed in:
    the same loss, the same d(hidden) bits, the same d(W) up to the order of the sums; chunks with no token, with a
    handful and with all but a few.  With rows of 8256 entries and few tokens the d(hidden) product is cut along the
    vocabulary; the device then makes the choice the host makes from the same count (the same bits again)."""
    T_pad, T = CHUNK + 256, CHUNK + 200
    V = 8256 if mask_kind.endswith("long_rows") else 640
    hidden, weight, labels, prox, old, adv, mask = _inputs(T_pad, T, 64, V, seed=47)
    if mask_kind == "second_chunk_empty":
        mask[CHUNK:] = False
    elif mask_kind == "nothing":
        mask[:] = False
    elif mask_kind.startswith("three_tokens"):
        mask[:] = False
        mask[[5, CHUNK - 1, CHUNK + 7]] = True
    elif mask_kind == "a_tile_and_a_bit_long_rows":
        mask[:] = False
        mask[torch.arange(0, CHUNK, 60)] = True          # 274 rows: two tiles
        mask[CHUNK + 3:CHUNK + 120] = True
    args = [t.to(device) for t in (labels, prox, old, adv)]
    counts = [int(mask[:CHUNK].sum()), int(mask[CHUNK:].sum())]

    def run(**kw):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        _poison_the_allocator_cache(device, int(_native.load().aa_lmhead_workspace_bytes(T_pad, 64, V)))
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device),
                                                      backward=backward, **kw)
        loss.backward()
        return loss.detach(), stat, h.grad, w.grad

    on_device, read_back, given = run(), run(count_on_device=False), run(kept_per_chunk=counts)
    for other in (read_back, given):
        assert torch.equal(on_device[0], other[0])
        assert torch.equal(on_device[1]["logprobs"], other[1]["logprobs"])
        assert torch.isfinite(on_device[3].float()).all()
        assert torch.equal(on_device[2], other[2])                                   # d(hidden): row by row the same
        if mask.any():
            assert cosine(on_device[3].float().cpu(), other[3].float().cpu()) > 0.9999999
            assert_same_magnitude(on_device[3].float(), other[3].float(), rel=1e-4)
        else:
            assert float(on_device[3].float().abs().max()) == 0.0 and float(other[3].float().abs().max()) == 0.0
    rows_off = torch.ones(T_pad, dtype=torch.bool, device=device)
    rows_off[:T] = ~mask.to(device)
    assert float(on_device[2][rows_off].float().abs().max()) == 0.0                  # tokens without a mask: zero rows


def test_standalone_backward_counts_its_rows_on_the_device(device):
    """``lm_head_logprobs_entropy`` (recompute backward): rows with a zero upstream gradient are left out without a
    read-back, with the results of the dense backward; through the C ABI the same call with host counts and with
    ``AA_LMHEAD_COUNT_ON_DEVICE`` entries gives the same gradients."""
    import ctypes as C

    from areal_amd import functional as F

    T, H, V = CHUNK + 300, 64, 1288
    g = torch.Generator().manual_seed(3)
    hidden = torch.randn(T, H, generator=g).bfloat16().to(device)
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16().to(device)
    labels = torch.randint(0, V, (T,), generator=g).to(device)
    g_lp = (torch.randn(T, generator=g) * (torch.rand(T, generator=g) < 0.4)).to(device)
    lib = _native.load()
    f32 = dict(dtype=torch.float32, device=device)
    logp, ent, lse, ez = (torch.empty(T, **f32) for _ in range(4))
    ws = torch.empty(int(lib.aa_lmhead_workspace_bytes(T, H, V)), dtype=torch.uint8, device=device)
    st = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    assert lib.aa_lmhead_fwd(F._ptr(hidden), F._ptr(weight), T, H, V, F._ptr(labels), 1.0, F._ptr(logp), F._ptr(ent),
                             F._ptr(lse), F._ptr(ez), None, None, F._ptr(ws), ws.numel(), st) == 0
    has = (g_lp != 0).view(torch.uint8)

    def bwd(kept):
        dh, dw = torch.full_like(hidden, float("nan")), torch.full_like(weight, float("nan"))
        arr = None if kept is None else (C.c_int64 * len(kept))(*kept)
        assert lib.aa_lmhead_bwd(F._ptr(hidden), F._ptr(weight), T, H, V, F._ptr(labels), 1.0, F._ptr(lse), F._ptr(ez),
                                 F._ptr(g_lp), None, F._ptr(has) if kept is not None else None, arr, F._ptr(dh), F._ptr(dw),
                                 _native.AA_BF16, F._ptr(ws), ws.numel(), st) == 0
        return dh, dw

    dense = bwd(None)
    host = bwd([int(has[:CHUNK].sum()), int(has[CHUNK:].sum())])
    dev = bwd([_native.AA_LMHEAD_COUNT_ON_DEVICE] * 2)
    assert torch.equal(host[0], dev[0]) and torch.equal(dense[0], dev[0])
    for other in (host, dense):
        assert cosine(dev[1].float().cpu(), other[1].float().cpu()) > 0.9999999
        assert_same_magnitude(dev[1].float(), other[1].float(), rel=1e-4)
    # and through autograd (the wrapper passes the device-count entries)
    h = hidden.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    lp, _ = areal_amd.lm_head_logprobs_entropy(h, w, labels)
    (lp * g_lp).sum().backward()
    assert torch.equal(h.grad, dev[0])
    assert cosine(w.grad.float().cpu(), dev[1].float().cpu()) > 0.9999999


def test_carry_with_unlikely_labels_at_masked_tokens_of_a_dense_backward(device):
    """``skip_masked_tokens=False`` puts every token in the panel.  A masked token (a prompt position) whose label is a
    hundred nats unlikely stores ratios p_v / p_label at the top of the bf16 range; their sum over the vocabulary may be
    infinite, and its factor is zero: the d(hidden) row has to come out as zero, not as 0 x inf."""
    T, H, V = 600, 64, 1088
    g = torch.Generator().manual_seed(9)
    hidden = torch.randn(T, H, generator=g)
    hidden[:200] *= 14.0                       # logits ~ N(0, 56^2) at the first 200 tokens
    hidden = hidden.bfloat16()
    weight = (0.5 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    ref_lp = oracle.logprobs(oracle.lmhead_logits(hidden, weight), labels)
    mask = torch.ones(T, dtype=torch.bool)
    mask[:200] = False                          # those tokens have no gradient
    assert int((ref_lp[:200] < -100).sum()) > 20 and float(ref_lp[200:].min()) > -60
    prox = ref_lp + 0.05 * torch.randn(T, generator=g)
    old = ref_lp + 0.3 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    loss, _ = areal_amd.fused_lm_head_ppo_loss(h, w, labels.to(device), prox.to(device), old.to(device), adv.to(device),
                                               eps_clip=0.2, loss_mask=mask.to(device), backward="carry",
                                               skip_masked_tokens=False)
    loss.backward()
    o_loss, _, _, _, o_dh, o_dw = _oracle_step(hidden, weight, labels, prox, old, adv, mask, 1.0, 1.0, eps_clip=0.2)
    assert torch.isfinite(h.grad.float()).all() and torch.isfinite(w.grad.float()).all()
    assert float(h.grad[:200].abs().sum()) == 0.0
    assert float(loss.detach()) == pytest.approx(o_loss, rel=1e-3)
    assert cosine(h.grad.cpu().float(), o_dh) > 0.9999 and cosine(w.grad.cpu().float(), o_dw) > 0.9999
    assert_same_magnitude(h.grad, o_dh, what="d(hidden)")
    assert_same_magnitude(w.grad, o_dw, what="d(W)")


def test_carry_with_small_factors_keeps_the_weight_gradient(device):
    """d(W) takes the row factor -(g / T) p_label inside the hidden rows, rounded to bf16.  Labels with a log-prob
    around -70 and a small loss scale push factor x hidden out of the normal range although d(logits) itself is of
    ordinary size there: such a chunk is redone by the recompute tiles.  Held to the oracle and to recompute mode."""
    T, H, V = 700, 64, 1088
    g = torch.Generator().manual_seed(21)
    hidden = (9.5 * torch.randn(T, H, generator=g)).bfloat16()     # logits ~ N(0, 38^2)
    weight = (0.5 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    ref_lp = oracle.logprobs(oracle.lmhead_logits(hidden, weight), labels)
    window = (ref_lp < -62) & (ref_lp > -79)
    assert int(window.sum()) > 30
    mask = window | (torch.rand(T, generator=g) < 0.3)
    mask &= ref_lp > -79                        # nothing below the overflow threshold: only the factor can trigger
    prox = ref_lp + 0.05 * torch.randn(T, generator=g)
    old = ref_lp + 0.3 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    scale = 1e-4
    args = [t.to(device) for t in (labels, prox, old, adv)]

    def run(backward):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, _ = areal_amd.fused_lm_head_ppo_loss(h, w, *args, eps_clip=0.2, loss_mask=mask.to(device), backward=backward,
                                                   loss_scale=scale)
        loss.backward()
        return loss.detach(), h.grad.float(), w.grad.float()

    o_loss, _, _, _, o_dh, o_dw = _oracle_step(hidden, weight, labels, prox, old, adv, mask, 1.0, scale, eps_clip=0.2)
    ref, got = run("recompute"), run("carry")
    assert float(got[0]) == pytest.approx(o_loss, rel=1e-3)
    for name, a, b, o in (("d(hidden)", got[1], ref[1], o_dh), ("d(W)", got[2], ref[2], o_dw)):
        assert torch.isfinite(a).all(), name
        assert cosine(a.cpu(), o) > 0.9999, name
        assert_same_magnitude(a, o, what=name)
        assert cosine(a.cpu(), b.cpu()) > 0.99999, name


@pytest.mark.parametrize("backward", ["carry", "recompute"])
@pytest.mark.parametrize("skip", [True, False])
def test_labels_outside_the_vocabulary_at_masked_tokens(device, backward, skip):
    """Tokens without a mask may carry any label (prompt positions, batch padding filled with -100): their log-prob is
    NaN, as on the logits path, and nothing of it reaches the loss or the gradients, with or without their rows in
    the gradient products."""
    T, H, V = 700, 64, 1088
    hidden, weight, labels, prox, old, adv, mask = _inputs(T, T, H, V, seed=77)
    bad = ~mask
    labels = labels.clone()
    labels[bad] = torch.where(torch.arange(T)[bad] % 2 == 0, torch.tensor(-100), torch.tensor(V + 3))
    prox[bad], old[bad] = 0.0, 0.0
    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, labels.to(device), prox.to(device), old.to(device), adv.to(device),
                                                  eps_clip=0.2, loss_mask=mask.to(device), backward=backward,
                                                  skip_masked_tokens=skip)
    loss.backward()
    assert torch.isnan(stat["logprobs"].cpu()[bad]).all() and torch.isfinite(stat["logprobs"].cpu()[mask]).all()
    ok_labels = torch.where(bad, torch.zeros_like(labels), labels)      # the oracle needs labels it can gather
    o_loss, _, o_lp, _, o_dh, o_dw = _oracle_step(hidden, weight, ok_labels, prox, old, adv, mask, 1.0, 1.0, eps_clip=0.2)
    assert float(loss.detach()) == pytest.approx(o_loss, rel=1e-3)
    assert torch.isfinite(h.grad).all() and torch.isfinite(w.grad).all()
    assert cosine(h.grad.cpu().float(), o_dh) > 0.9999 and cosine(w.grad.cpu().float(), o_dw) > 0.9999
    assert_same_magnitude(h.grad, o_dh, what="d(hidden)")
    assert_same_magnitude(w.grad, o_dw, what="d(W)")
    assert float(h.grad.cpu()[bad].abs().sum()) == 0.0


@pytest.mark.parametrize("skip_masked_tokens", [False, True])
@pytest.mark.parametrize("backward", ["carry", "recompute"])
def test_step_replays_from_a_hip_graph(device, backward, skip_masked_tokens):
    """aa_lmhead_ppo_fused allocates nothing, clears memory with kernels only and never waits for the device, so the
    whole step can be captured into a HIP graph: with every token's row in the gradient products, or with the tokens
    without a mask left out (the rows in use are counted on the device, so the graph holds for any mask: the replays
    below come with masks of 70 %, 10 %, none and all of the tokens; the vocabulary is long enough for the d(hidden)
    product to be cut along it when few rows are in use).  Four replays on new inputs, with eager work and
    synchronisations in between, each equal to the eager result on the same inputs."""
    T, H, V = 600, 128, 8256 if skip_masked_tokens else 1088
    g = torch.Generator().manual_seed(3)
    h = torch.zeros(T, H, dtype=torch.bfloat16, device=device, requires_grad=True)
    w = torch.zeros(V, H, dtype=torch.bfloat16, device=device, requires_grad=True)
    labels = torch.randint(0, V, (T,), generator=g).to(device)
    prox, old, adv = (torch.zeros(T, device=device) for _ in range(3))
    mask = (torch.rand(T, generator=g) < 0.7).to(device)
    kw = dict(eps_clip=0.2, loss_mask=mask, eps_clip_higher=0.28, backward=backward,
              skip_masked_tokens=skip_masked_tokens)
    density = {0: 0.7, 1: 0.7, 2: 0.1, 3: 0.0, 4: 1.0}

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            if skip_masked_tokens:
                mask.copy_((torch.rand(T, generator=gg) < density[seed]).to(device))
            h.copy_(torch.randn(T, H, generator=gg).bfloat16())
            w.copy_((0.3 * torch.randn(V, H, generator=gg)).bfloat16())
            ref, _ = areal_amd.lm_head_logprobs_entropy(h, w, labels)
            prox.copy_(ref + 0.05 * torch.randn(T, generator=gg).to(device))
            old.copy_(ref + 0.05 * torch.randn(T, generator=gg).to(device))
            adv.copy_(torch.randn(T, generator=gg).to(device))

    def step():
        loss, stat = areal_amd.fused_lm_head_ppo_loss(h, w, labels, prox, old, adv, **kw)
        loss.backward()
        return loss, stat["logprobs"]

    fill(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            h.grad, w.grad = None, None
            step()
    torch.cuda.current_stream().wait_stream(side)
    h.grad, w.grad = None, None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_loss, g_logp = step()
    g_dh, g_dw = h.grad, w.grad
    for seed in (1, 2, 3, 4):
        fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = (g_loss.detach().clone(), g_logp.clone(), g_dh.clone(), g_dw.clone())
        h2 = h.detach().clone().requires_grad_(True)                    # eager, same inputs
        w2 = w.detach().clone().requires_grad_(True)
        e_loss, e_stat = areal_amd.fused_lm_head_ppo_loss(h2, w2, labels, prox, old, adv, **kw)
        e_loss.backward()
        torch.cuda.synchronize()
        assert torch.equal(got[0], e_loss.detach()) and torch.equal(got[1], e_stat["logprobs"])
        assert torch.equal(got[2], h2.grad) and torch.equal(got[3], w2.grad)


@pytest.mark.parametrize("with_host_mask", [True, False])
@pytest.mark.parametrize("with_rs", [False, True])
def test_engine_contract_of_the_lm_head_step(device, with_host_mask, with_rs):
    """``engine_glue.compute_lm_head_and_loss`` against the reference's engine contract (fsdp_engine.py:1977-2046) on
    ``hidden @ W.T``: labels rolled over the sequence borders, the pad rows trimmed and without gradient, the loss
    scaled by local / total weight, the vocabulary extrema handed on, the zero-weight micro-batch."""
    lengths, pad = [5, 3, 4], 4
    n = sum(lengths)
    T, H, V = n + pad, 64, 1097
    g = torch.Generator().manual_seed(3)
    input_ids = torch.randint(0, V, (1, T), generator=g)
    labels = torch.cat([input_ids[0, 1:], input_ids[0, :1]])
    hidden = torch.randn(1, T, H, generator=g).bfloat16()
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16()
    logits = oracle.lmhead_logits(hidden[0], weight)
    ref = oracle.logprobs(logits, labels)[:n]
    mb = dict(
        loss_mask=(torch.rand(n, generator=g) < 0.6), logprobs=ref + 0.3 * torch.randn(n, generator=g),
        prox_logp=ref + 0.05 * torch.randn(n, generator=g), advantages=torch.randn(n, generator=g),
        cu_seqlens=torch.tensor([0, 5, 8, 12], dtype=torch.int32),
    )
    rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", upper=1.2) if with_rs else None
    mb_d = {k: v.to(device) for k, v in mb.items()}
    total_w = torch.tensor(40.0, device=device)
    scale = float(mb["loss_mask"].sum()) / 40.0 * 0.5
    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    loss, stat = engine_glue.compute_lm_head_and_loss(
        h, w, {"input_ids": input_ids.to(device)}, mb_d, pad, total_w, eps_clip=0.2, c_clip=3.0, rejection_sampling=rs,
        loss_multiplier=0.5, host_loss_mask=mb["loss_mask"] if with_host_mask else None)
    loss.backward()
    o_loss, o_stat, o_lp, o_ent, o_dh, o_dw = _oracle_step(
        hidden[0], weight, labels, mb["prox_logp"], mb["logprobs"], mb["advantages"], mb["loss_mask"], 1.0, scale,
        eps_clip=0.2, c_clip=3.0, rejection_sampling_cfg=rs, cu_seqlens=mb["cu_seqlens"])
    assert float(loss.detach()) == pytest.approx(o_loss, rel=1e-3)
    assert stat["logprobs"].shape == (n,) and stat["entropy"].shape == (n,)
    assert_within(stat["logprobs"], o_lp[:n], 2e-3, "log-prob")
    assert_within(stat["entropy"], o_ent[:n], 2e-3, "entropy")
    assert float((stat["vocab_max_logits"].cpu() - logits[:n].max(-1).values).abs().max()) <= 1e-5 * float(logits.abs().max())
    assert float((stat["vocab_min_logits"].cpu() - logits[:n].min(-1).values).abs().max()) <= 1e-5 * float(logits.abs().max())
    assert h.grad.shape == hidden.shape
    assert cosine(h.grad[0].cpu().float(), o_dh) > 0.9999 and cosine(w.grad.cpu().float(), o_dw) > 0.9999
    assert_same_magnitude(h.grad[0], o_dh, what="d(hidden)")
    assert_same_magnitude(w.grad, o_dw, what="d(W)")
    assert float(h.grad[0, n:].float().abs().max()) == 0.0            # batch padding gets no gradient
    assert torch.equal(stat["clip_mask"].cpu(), o_stat["clip_mask"])
    if with_rs:
        assert float(stat["filtered_fraction"]) == pytest.approx(float(o_stat["filtered_fraction"]), abs=1e-6)
    # a micro-batch without any unmasked token keeps the graph to both inputs alive and contributes nothing
    mb_d["loss_mask"] = torch.zeros(n, dtype=torch.bool, device=device)
    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    loss, stat = engine_glue.compute_lm_head_and_loss(
        h, w, {"input_ids": input_ids.to(device)}, mb_d, pad, total_w, eps_clip=0.2,
        host_loss_mask=torch.zeros(n, dtype=torch.bool) if with_host_mask else None)
    loss.backward()
    assert stat == {} and float(loss.detach()) == 0.0
    assert float(h.grad.float().abs().max()) == 0.0 and float(w.grad.float().abs().max()) == 0.0
    # forward-only pass of the same micro-batch
    lp = engine_glue.compute_lm_head_logprobs(hidden.to(device), weight.to(device), {"input_ids": input_ids.to(device)})
    assert_within(lp[:n], o_lp[:n], 2e-3, "log-prob of the forward-only pass")


@pytest.mark.parametrize("backward", ["carry", "recompute"])
@pytest.mark.parametrize("variant", ["sapo", "gspo", "ppo_m2po"])
def test_any_loss_function_on_the_hidden_states(device, variant, backward):
    """``engine_glue.compute_lm_head_loss_with``: the actor's loss function in its SAPO, sequence-level (GSPO) and
    M2PO forms on hidden states and lm_head weight, against ``compute_loss_with`` on fp32 logits ``hidden @ W.T`` formed
    by torch (that path is held to the oracle in its own tests): same loss, same statistics, same gradients."""
    import functools

    lengths, pad = [90, 60, 130], 40
    n = sum(lengths)
    T, H, V = n + pad, 64, 1097
    g = torch.Generator().manual_seed(13)
    input_ids = torch.randint(0, V, (1, T), generator=g)
    labels = torch.cat([input_ids[0, 1:], input_ids[0, :1]])
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16()
    ref = oracle.logprobs(oracle.lmhead_logits(hidden, weight), labels)[:n]
    mb = dict(
        input_ids=input_ids[0, :n], loss_mask=(torch.rand(n, generator=g) < 0.6),
        logprobs=ref + 0.1 * torch.randn(n, generator=g), prox_logp=ref + 0.05 * torch.randn(n, generator=g),
        advantages=torch.randn(n, generator=g), cu_seqlens=torch.tensor([0, 90, 150, 280], dtype=torch.int32),
    )
    mb_d = {k: v.to(device) for k, v in mb.items()}
    kw = dict(eps_clip=0.2, eps_clip_higher=0.28, c_clip=3.0)
    if variant == "sapo":
        kw.update(use_sapo_loss=True, sapo_tau_pos=1.0, sapo_tau_neg=1.05)
    elif variant == "gspo":
        kw.update(importance_sampling_level="sequence")
    else:
        kw.update(m2_threshold=0.04, use_decoupled_loss=True)
    loss_fn = functools.partial(engine_glue.grpo_loss_fn, **kw)
    weight_fn = lambda d: d["loss_mask"].count_nonzero()
    model_inputs = {"input_ids": input_ids.to(device)}
    total_w = torch.tensor(500.0, device=device)

    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    loss, stat = engine_glue.compute_lm_head_loss_with(h, w, model_inputs, mb_d, pad, loss_fn, weight_fn, total_w,
                                                       temperature=0.9, backward=backward)
    loss.backward()
    h2 = hidden.float().to(device).requires_grad_(True)     # fp32 leaves: the gradients to compare with are not rounded
    w2 = weight.float().to(device).requires_grad_(True)
    logits = h2 @ w2.t()
    loss2, stat2 = engine_glue.compute_loss_with(logits, model_inputs, mb_d, pad, loss_fn, weight_fn, total_w,
                                                 temperature=0.9)
    loss2.backward()
    assert float(loss.detach()) == pytest.approx(float(loss2.detach()), rel=1e-3, abs=1e-7)
    for k in ("loss", "importance_weight", "approx_kl"):
        assert_within(stat[k], stat2[k], 2e-3, k)
    assert torch.equal(stat["clip_mask"], stat2["clip_mask"])
    assert cosine(h.grad.float().cpu(), h2.grad.float().cpu()) > 0.9999
    assert cosine(w.grad.float().cpu(), w2.grad.float().cpu()) > 0.9999
    assert_same_magnitude(h.grad, h2.grad.float(), what="d(hidden)")
    assert_same_magnitude(w.grad, w2.grad.float(), what="d(W)")
    assert float(h.grad[n:].float().abs().sum()) == 0.0
    # a micro-batch of weight zero keeps the graph alive
    mb_d["loss_mask"] = torch.zeros(n, dtype=torch.bool, device=device)
    h = hidden.to(device).requires_grad_(True)
    w = weight.to(device).requires_grad_(True)
    z = engine_glue.compute_lm_head_loss_with(h, w, model_inputs, mb_d, pad, loss_fn, weight_fn, total_w)
    z.backward()
    assert float(z.detach()) == 0.0 and float(h.grad.float().abs().max()) == 0.0
