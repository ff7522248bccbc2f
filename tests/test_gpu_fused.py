"""GPU parity of the fused logits -> log-prob/entropy -> PPO loss -> d(logits) pass, and of the engine-side
contract (packed roll of the labels, trimmed padding, loss scale)."""
import math

import pytest
import torch

import areal_amd
import oracle
from areal_amd import RejectionSamplingConfig, engine_glue, synth
from helpers import assert_same_magnitude, cosine

pytestmark = pytest.mark.gpu


def _finish_case(case, seed=0):
    ref = oracle.logprobs(case.logits.cpu(), case.labels.cpu(), case.temperature)
    return synth.attach_old_and_prox(case, ref.to(case.logits.device), 0.05, seed + 9)


def _oracle_step(case, pad=0, **over):
    kw = dict(case.ppo)
    kw.update(over)
    rs = kw.pop("rejection_sampling", None)
    cfg = RejectionSamplingConfig(**rs) if isinstance(rs, dict) else rs
    n = case.n_tokens - pad
    return oracle.logits_ppo_step(
        case.logits.cpu(), case.labels.cpu(), case.prox_logp.cpu()[:n], case.old_logp.cpu()[:n],
        case.advantages.cpu()[:n], loss_mask=case.loss_mask.cpu()[:n], rejection_sampling_cfg=cfg,
        cu_seqlens=case.cu_seqlens.cpu(), temperature=case.temperature, **kw,
    )


def _fused_step(case, pad=0, **over):
    kw = dict(case.ppo)
    kw.update(over)
    rs = kw.pop("rejection_sampling", None)
    cfg = RejectionSamplingConfig(**rs) if isinstance(rs, dict) else rs
    n = case.n_tokens - pad
    x = case.logits.clone().requires_grad_(True)
    loss, stat = areal_amd.fused_logprobs_ppo_loss(
        x, case.labels, case.prox_logp[:n], case.old_logp[:n], case.advantages[:n], loss_mask=case.loss_mask[:n],
        rejection_sampling=cfg, cu_seqlens=case.cu_seqlens, temperature=case.temperature, **kw,
    )
    loss.backward()
    return loss.detach(), stat, x.grad


def _compare(case, got, want, pad=0):
    g_loss, g_stat, g_grad = got
    w_loss, w_stat, w_grad = want
    n = case.n_tokens - pad
    ref_lp, ref_ent = oracle.logprobs_entropy_f64(case.logits.cpu(), case.labels.cpu(), case.temperature)
    assert float((g_stat["logprobs"].cpu().double() - ref_lp[:n]).abs().max()) < 2e-3        # stated
    assert float((g_stat["logprobs"].cpu().double() - ref_lp[:n]).abs().max()) < 1e-4
    assert float((g_stat["entropy"].cpu().double() - ref_ent[:n]).abs().max()) < 1e-4
    assert float(g_loss) == pytest.approx(float(w_loss), rel=1e-3, abs=1e-7)                  # stated
    assert g_grad.dtype == case.logits.dtype and g_grad.shape == case.logits.shape
    assert cosine(g_grad.cpu(), w_grad) > 0.9999                                              # stated
    assert_same_magnitude(g_grad.cpu(), w_grad, what="d_logits")   # cosine is blind to a wrong scale
    for k in ("clip_mask", "dual_clip_mask"):
        assert torch.equal(g_stat[k].cpu(), w_stat[k]), k
    for k in ("loss", "importance_weight", "approx_kl"):
        assert torch.allclose(g_stat[k].cpu(), w_stat[k], rtol=1e-3, atol=2e-4), k
    m = case.loss_mask[:n]
    rows_off = torch.ones(case.n_tokens, dtype=torch.bool, device=m.device)
    eff = g_stat["behave_mask"] if "behave_mask" in g_stat else m
    rows_off[:n] = ~eff
    assert float(g_grad[rows_off].float().abs().max()) == 0.0      # masked and padded rows: exactly zero
    assert torch.equal(g_stat["vocab_max_logits"].cpu(), case.logits.cpu()[:n].max(-1).values.float())
    assert torch.equal(g_stat["vocab_min_logits"].cpu(), case.logits.cpu()[:n].min(-1).values.float())


@pytest.mark.parametrize(
    "V,dtype,lo,hi",
    [
        (151936, torch.bfloat16, 8, 40),   # register-resident rows, 19 chunks (benchmark vocabulary)
        (32768, torch.bfloat16, 8, 40),    # register-resident rows, exact multiple of the chunk size
        (8200, torch.float16, 8, 40),      # up to two chunks: the two-pass kernel
        (16392, torch.float16, 8, 40),     # 3 chunks in registers, the third almost empty
        (50257, torch.bfloat16, 4, 20),    # V % 8 != 0: rows at every even address, held in registers all the same
        (4099, torch.float32, 4, 20),      # generic rows, fp32 logits
        (8192, torch.float32, 4, 12),      # fp32 rows held on the chip: exactly one register chunk
        (81928, torch.float32, 4, 12),     # registers full, one vector in LDS
        (114688, torch.float32, 4, 12),    # registers and LDS full: the longest row that is held exactly
        (114696, torch.float32, 4, 12),    # one vector more: the row is held in 24 bits per value from here on
        (151936, torch.float32, 4, 12),    # benchmark vocabulary in fp32: 13 chunks in registers, 5.5 in LDS
        (155648, torch.float32, 4, 12),    # registers and LDS full of 24-bit values
        (155656, torch.float32, 4, 12),    # one vector read twice
        (200000, torch.float32, 4, 12),    # 5.4 chunks read twice
        (172040, torch.bfloat16, 4, 12),   # 22 chunks: 21 in registers, one (a single 16-byte piece of it) in LDS
        (245760, torch.bfloat16, 4, 12),   # 30 chunks: registers and LDS full, no tail
        (250008, torch.float16, 4, 12),    # 31 chunks: a partial streamed tail chunk
        (262144, torch.bfloat16, 4, 12),   # 32 chunks: the largest row of the register / LDS / tail kernel
        (262152, torch.bfloat16, 4, 12),   # one vector more: generic rows again
    ],
)
def test_fused_config0_shape_matches_oracle(device, V, dtype, lo, hi):
    lengths = synth.lengths_uniform(6, lo, hi, seed=V)
    case = synth.make_logits_case("t", lengths, V, V, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  dtype=dtype, ppo=dict(eps_clip=0.2))
    _finish_case(case)
    _compare(case, _fused_step(case), _oracle_step(case))


@pytest.mark.parametrize("V,dtype", [(16392, torch.bfloat16), (32000, torch.float16), (57344, torch.bfloat16)])
def test_short_rows_with_two_workgroups_per_unit(device, V, dtype):
    """Rows of 3 to 7 chunks run two workgroups per compute unit; more rows than workgroups, so the rows after
    the first 512 are handed out through the counter."""
    lengths = synth.lengths_uniform(48, 16, 48, seed=V)           # about 1500 tokens
    case = synth.make_logits_case("t", lengths, V, V, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  dtype=dtype, ppo=dict(eps_clip=0.2))
    assert case.n_tokens > 1100
    _finish_case(case)
    first = _fused_step(case)
    _compare(case, first, _oracle_step(case))
    again = _fused_step(case)                                     # another hand-out order, the same bits
    assert torch.equal(first[2], again[2]) and float(first[0]) == float(again[0])


@pytest.mark.parametrize("V", [70004, 24576, 49152, 90112, 122880, 32776, 90120, 122888, 200008])
def test_fp32_long_rows_walked_by_large_workgroups(device, V):
    """More fp32 rows than workgroups, so every workgroup handles several rows: V = 70004 (not a multiple of 8, rows
    of 280 KB) takes the two-pass kernel with 512 walking workgroups, the others the kernel that holds the row on the
    chip with one workgroup per compute unit: in registers alone (V = 24576: up to 4 chunks, V = 49152: up to 8), in
    registers and LDS (V = 90112), and in 24 bits per value (V = 122880).  The last four widths put the rows 32 bytes
    off the 128-byte lines: their requests go out on a grid shifted per row (V = 200008: with a part of the row that is
    read twice)."""
    lengths = synth.lengths_uniform(40, 8, 24, seed=5)            # about 640 tokens
    case = synth.make_logits_case("t", lengths, V, V, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  dtype=torch.float32, ppo=dict(eps_clip=0.2))
    assert case.n_tokens > 512
    _finish_case(case)
    first = _fused_step(case)
    _compare(case, first, _oracle_step(case))
    again = _fused_step(case)                                     # rows handed out in another order, the same bits
    assert torch.equal(first[2], again[2]) and float(first[0]) == float(again[0])


@pytest.mark.parametrize("V,temperature", [(151936, 1.0), (180224, 0.6)])
def test_fp32_rows_held_in_24_bits_entry_by_entry(device, V, temperature):
    """fp32 rows past 114 688 values stay on the chip rounded to 24 bits: log-probs and entropy come from the fp32
    values (as exact as for shorter rows), every entry of the gradient row is within |x| / T * 2^-16 (relative,
    beside the error of the row's logsumexp, which all entries share) of the float64 one, and labels in the
    register, LDS and re-read parts of the row get their +g / T."""
    spots = [0, 8191, 13 * 8192 - 1, 13 * 8192, 16 * 8192 + 77, V - 1, 19 * 8192 - 8 if V > 19 * 8192 else 5,
             min(19 * 8192 + 3, V - 2)]
    lengths = [len(spots)]
    case = synth.make_logits_case("t", lengths, V, 11, device, synth.per_sequence_normal_advantages(lengths, 4),
                                  dtype=torch.float32, ppo=dict(eps_clip=0.2), temperature=temperature)
    with torch.no_grad():
        for r, j in enumerate(spots):
            case.labels[r] = j
        case.loss_mask[:] = True
    _finish_case(case)
    loss, stat, grad = _fused_step(case)
    x = case.logits.double().cpu().requires_grad_(True)
    lp = torch.log_softmax(x / temperature, dim=-1).gather(-1, case.labels.cpu()[:, None])[:, 0]
    assert float((stat["logprobs"].cpu().double() - lp.detach()).abs().max()) < 3e-5
    # a gradient row is (d loss / d logp_t) / T * (onehot(label) - softmax): fit the one factor, then compare entries
    probs = torch.softmax(x.detach() / temperature, dim=-1)
    got = grad.double().cpu()
    for r, j in enumerate(spots):
        onehot = torch.zeros(V, dtype=torch.float64)
        onehot[j] = 1.0
        want_dir = onehot - probs[r]                 # d logp_label / d x, times T
        row = got[r]
        scale = float(row @ want_dir / (want_dir @ want_dir))
        if scale == 0.0:
            assert float(row.abs().max()) == 0.0
            continue
        resid = row / (scale * want_dir) - 1.0       # relative error, entry by entry
        resid[j] = 0.0
        xr = x.detach()[r]
        common = float(resid[xr.abs() < 0.25].median())   # the row's logsumexp error, shared by every entry
        assert abs(common) < 1e-4, (r, j, common)
        bound = xr.abs() / temperature * 2.0 ** -16 + 1e-5
        assert bool(((resid - common).abs() <= bound).all()), (r, j)
        assert abs(float(row[j]) - scale * float(want_dir[j])) <= 1e-4 * abs(scale), (r, j)   # the label got its + g / T


def test_long_rows_labels_and_extrema_in_every_region(device):
    """V = 262144: labels and the row maximum / minimum placed in the register, LDS and streamed parts of the row."""
    V = 262144
    spots = [0, 8191, 21 * 8192 - 1, 21 * 8192, 25 * 8192 + 77, 30 * 8192 - 1, 30 * 8192, 31 * 8192 + 5, V - 1]
    lengths = [len(spots), len(spots)]
    case = synth.make_logits_case("t", lengths, V, 11, device, synth.per_sequence_normal_advantages(lengths, 4),
                                  ppo=dict(eps_clip=0.2, eps_clip_higher=0.28, c_clip=3.0), temperature=0.9)
    n = len(spots)
    with torch.no_grad():
        for r, j in enumerate(spots):
            case.labels[r] = j                      # first sequence: the label sits at the spot
            case.logits[n + r, j] = 30.0            # second sequence: the maximum does ...
            case.logits[n + r, spots[-1 - r]] = -40.0   # ... and the minimum at the mirrored spot
    _finish_case(case)
    case.loss_mask[:] = True
    case.loss_mask[4] = False                      # one masked row: its gradient must be exactly zero
    _compare(case, _fused_step(case), _oracle_step(case))


def test_fused_config1_options_padding_and_scale(device):
    """GRPO advantages, importance-weight cap, dual clip, temperature, a trailing pad sequence, a loss scale."""
    lengths = [37, 5, 64, 22]
    pad = 256 - sum(lengths)  # the engine pads the packed batch to a multiple of 256 tokens with one fake sequence
    V = 151936
    adv = synth.grpo_advantages(lengths + [pad], 2, 0.4, seed=2)
    case = synth.make_logits_case("t", lengths + [pad], V, 5, device, adv, temperature=0.7)
    _finish_case(case)
    case.cu_seqlens = case.cu_seqlens[:-1]
    for rs in (dict(level="token", action="mask", metric="ratio", upper=1.05),
               dict(level="token", action="clamp", metric="ratio", upper=1.05)):
        over = dict(eps_clip=0.2, eps_clip_higher=0.28, c_clip=3.0, rejection_sampling=rs, loss_scale=0.37)
        got, want = _fused_step(case, pad, **over), _oracle_step(case, pad, **over)
        _compare(case, got, want, pad)
        assert 0 < got[1]["filtered_fraction"] < 1
        assert got[1]["filtered_fraction"] == pytest.approx(want[1]["filtered_fraction"], abs=1e-12)
        assert torch.equal(got[1]["behave_mask"].cpu(), want[1]["behave_mask"])


def test_fused_equals_unfused_kernels_and_sequence_level_falls_back(device):
    lengths = [19, 33, 12]
    case = synth.make_logits_case("t", lengths, 32768, 7, device, synth.per_sequence_normal_advantages(lengths, 1),
                                  ppo=dict(eps_clip=0.2))
    _finish_case(case)
    f_loss, f_stat, f_grad = _fused_step(case)
    x = case.logits.clone().requires_grad_(True)
    lp, ent = areal_amd.gather_logprobs_entropy(x, case.labels)
    loss, stat = areal_amd.ppo_actor_loss_fn(lp, case.prox_logp, case.old_logp, case.advantages, 0.2, case.loss_mask)
    loss.backward()
    assert float(f_loss) == pytest.approx(float(loss.detach()), rel=1e-6)
    assert float((f_stat["logprobs"] - lp.detach()).abs().max()) < 1e-5
    assert cosine(f_grad, x.grad) > 0.999999
    assert_same_magnitude(f_grad, x.grad, what="fused vs unfused d_logits")
    # GSPO: per-token loss depends on the whole sequence -> unfused kernels, same API
    s_got = _fused_step(case, importance_sampling_level="sequence")
    s_want = _oracle_step(case, importance_sampling_level="sequence")
    assert float(s_got[0]) == pytest.approx(float(s_want[0]), rel=1e-3, abs=1e-7)
    assert cosine(s_got[2].cpu(), s_want[2]) > 0.9999
    assert_same_magnitude(s_got[2].cpu(), s_want[2], what="sequence-level d_logits")


def test_backward_with_upstream_factor(device):
    lengths = [9, 14]
    case = synth.make_logits_case("t", lengths, 16384, 3, device, synth.per_sequence_normal_advantages(lengths, 1),
                                  ppo=dict(eps_clip=0.2))
    _finish_case(case)
    _, _, g1 = _fused_step(case)
    x = case.logits.clone().requires_grad_(True)
    loss, _ = areal_amd.fused_logprobs_ppo_loss(x, case.labels, case.prox_logp, case.old_logp, case.advantages, 0.2,
                                                case.loss_mask)
    (loss * 3.0).backward()
    assert cosine(x.grad, g1) > 0.99999
    assert float(x.grad.float().norm() / g1.float().norm()) == pytest.approx(3.0, rel=1e-2)


def test_engine_contract_roll_pad_and_scale(device):
    """Labels are the packed input_ids rolled by one over the whole tensor (integer indexing, bit-exact): the
    last token of a sequence is labelled with the first token of the next one."""
    lengths = [5, 3, 4]
    pad = 4
    T, V = sum(lengths) + pad, 9000
    g = torch.Generator().manual_seed(0)
    input_ids = torch.randint(0, V, (1, T), generator=g)
    labels = engine_glue.rolled_labels({"input_ids": input_ids.to(device)})
    assert labels.shape == (T,) and labels.dtype == torch.int64
    assert torch.equal(labels.cpu(), torch.cat([input_ids[0, 1:], input_ids[0, :1]]))
    assert int(labels[4]) == int(input_ids[0, 5])          # crosses the boundary between sequences 0 and 1
    assert torch.equal(engine_glue.rolled_labels({"input_ids": input_ids, "rolled_input_ids": input_ids}), input_ids[0])

    logits = (2 * torch.randn(T, V, generator=g)).bfloat16()
    n = T - pad
    ref = oracle.logprobs(logits, labels.cpu())[:n]
    mb = dict(
        loss_mask=(torch.rand(n, generator=g) < 0.6), logprobs=ref + 0.05 * torch.randn(n, generator=g),
        prox_logp=ref + 0.05 * torch.randn(n, generator=g), advantages=torch.randn(n, generator=g),
        cu_seqlens=torch.tensor([0, 5, 8, 12], dtype=torch.int32),
    )
    mb_d = {k: v.to(device) for k, v in mb.items()}
    total_w = torch.tensor(40.0, device=device)
    results = []
    for fused in (True, False):
        x = logits.to(device).requires_grad_(True)
        loss, stat = engine_glue.compute_logprobs_and_loss(
            x, {"input_ids": input_ids.to(device)}, mb_d, pad, total_w, eps_clip=0.2, fused=fused
        )
        loss.backward()
        results.append((float(loss.detach()), x.grad.clone(), stat))
    w_loss, _, w_grad = oracle.logits_ppo_step(
        logits, labels.cpu(), mb["prox_logp"], mb["logprobs"], mb["advantages"], 0.2, mb["loss_mask"],
        loss_scale=float(mb["loss_mask"].sum()) / 40.0,
    )
    for loss, grad, stat in results:
        assert loss == pytest.approx(float(w_loss), rel=1e-3)
        assert cosine(grad.cpu(), w_grad) > 0.9999
        assert_same_magnitude(grad.cpu(), w_grad, what="d_logits")
        assert float(grad[n:].float().abs().max()) == 0.0
        assert stat["logprobs"].shape == (n,)
    # the same call with the gradient written over the logits: the bits of the fused result
    x = logits.to(device).requires_grad_(True)
    loss, _ = engine_glue.compute_logprobs_and_loss(x, {"input_ids": input_ids.to(device)}, mb_d, pad, total_w,
                                                    eps_clip=0.2, inplace_backward=True)
    loss.backward()
    assert float(loss.detach()) == results[0][0] and torch.equal(x.grad, results[0][1]) and torch.equal(x.detach(), x.grad)
    # an all-masked micro-batch keeps the graph alive and contributes nothing
    mb_d["loss_mask"] = torch.zeros(n, dtype=torch.bool, device=device)
    x = logits.to(device).requires_grad_(True)
    loss, _ = engine_glue.compute_logprobs_and_loss(x, {"input_ids": input_ids.to(device)}, mb_d, pad, total_w, 0.2)
    loss.backward()
    assert float(loss.detach()) == 0.0 and float(x.grad.float().abs().max()) == 0.0


def test_full_size_properties_config1(device):
    """At the benchmark's own size the oracle is too slow; check what does not depend on size."""
    case = synth.config1(device, seed=1, total_tokens=8192)
    lp = areal_amd.gather_logprobs(case.logits, case.labels)
    synth.attach_old_and_prox(case, lp, 0.05, 4)
    rs = RejectionSamplingConfig(**case.ppo["rejection_sampling"])
    runs = []
    for _ in range(2):
        x = case.logits.requires_grad_(True)
        x.grad = None
        loss, stat = areal_amd.fused_logprobs_ppo_loss(
            x, case.labels, case.prox_logp, case.old_logp, case.advantages, 0.2, case.loss_mask, rejection_sampling=rs
        )
        loss.backward()
        runs.append((loss.detach().clone(), stat, x.grad))
    (l1, s1, g1), (l2, s2, g2) = runs
    assert torch.equal(l1, l2) and torch.equal(g1, g2) and torch.equal(s1["logprobs"], s2["logprobs"])  # deterministic
    V = case.logits.shape[1]
    assert float(s1["logprobs"].max()) <= 0.0
    assert float(s1["entropy"].min()) >= 0.0 and float(s1["entropy"].max()) <= math.log(V) + 1e-4
    assert float((s1["logprobs"] - lp).abs().max()) < 1e-5               # fused forward == stand-alone forward
    keep = s1["behave_mask"]
    assert float(g1[~keep].float().abs().max()) == 0.0
    # (onehot - p) sums to zero along the vocabulary: only bf16 rounding of 151936 terms is left
    row_sums = g1[keep].float().sum(-1).abs()
    scale = g1[keep].float().abs().max(-1).values
    assert float((row_sums / scale).max()) < 0.05
    # the scalar loss is the masked sum of the per-token losses over the ORIGINAL mask count
    manual = s1["loss"][keep].double().sum() / int(case.loss_mask.sum())
    assert float(l1) == pytest.approx(float(manual), rel=1e-5)
    # linearity in the loss scale
    x = case.logits.detach().requires_grad_(True)
    loss_h, _ = areal_amd.fused_logprobs_ppo_loss(
        x, case.labels, case.prox_logp, case.old_logp, case.advantages, 0.2, case.loss_mask, rejection_sampling=rs,
        loss_scale=0.5,
    )
    assert float(loss_h.detach()) == pytest.approx(0.5 * float(l1.detach()), rel=1e-6)


def test_full_size_config1_properties_and_sampled_parity(device):
    """The benchmark's own workload, all 64 sequences as drawn (about 122 000 tokens, 37 GB of logits and as much of
    gradient): what does not depend on size over every row, and the oracle on 64 rows spread over the whole token
    range (the first, the middle and the last rows)."""
    case = synth.config1(device, seed=0)
    T, V = case.logits.shape
    assert T > 100_000 and V == 151936
    lp = areal_amd.gather_logprobs(case.logits, case.labels)
    synth.attach_old_and_prox(case, lp, 0.05, 9)
    rs = RejectionSamplingConfig(**case.ppo["rejection_sampling"])
    kw = {k: v for k, v in case.ppo.items() if k != "rejection_sampling"}
    runs = []
    for _ in range(2):
        x = case.logits.detach().requires_grad_(True)
        loss, stat = areal_amd.fused_logprobs_ppo_loss(
            x, case.labels, case.prox_logp, case.old_logp, case.advantages, loss_mask=case.loss_mask,
            rejection_sampling=rs, cu_seqlens=case.cu_seqlens, **kw)
        loss.backward()
        runs.append((loss.detach().clone(), stat, x.grad))
    (l1, s1, g1), (l2, s2, g2) = runs
    assert torch.equal(l1, l2) and torch.equal(s1["logprobs"], s2["logprobs"]) and torch.equal(s1["entropy"], s2["entropy"])
    assert torch.equal(g1, g2)                                            # bit-equal from run to run
    del g2, runs
    assert float(s1["logprobs"].max()) <= 0.0
    assert float(s1["entropy"].min()) >= 0.0 and float(s1["entropy"].max()) <= math.log(V) + 1e-4
    assert float((s1["logprobs"] - lp).abs().max()) < 1e-5               # fused forward == stand-alone forward
    keep = s1["behave_mask"]
    assert bool((keep <= case.loss_mask).all()) and 0 < int(keep.sum()) < T
    worst_off, worst_sum = 0.0, 0.0
    for a in range(0, T, 4096):                                           # row blocks: no fp32 copy of 37 GB
        g = g1[a:a + 4096].float()
        k = keep[a:a + 4096]
        if bool((~k).any()):
            worst_off = max(worst_off, float(g[~k].abs().max()))
        if bool(k.any()):
            worst_sum = max(worst_sum, float((g[k].sum(-1).abs() / g[k].abs().max(-1).values).max()))
    assert worst_off == 0.0                                               # rows without a mask: exactly zero
    assert worst_sum < 0.05                                               # rows of (onehot - p) sum to zero up to bf16 rounding
    manual = s1["loss"][keep].double().sum() / int(case.loss_mask.sum())
    assert float(l1) == pytest.approx(float(manual), rel=1e-5)
    # oracle on 64 rows: 22 first, 21 middle, 21 last
    idx = torch.cat([torch.arange(0, 22), torch.arange(T // 2 - 10, T // 2 + 11), torch.arange(T - 21, T)])
    idx_d = idx.to(device)
    n_s = idx.numel()
    mask_s = case.loss_mask[idx_d].cpu()
    assert 0 < int(mask_s.sum()) < n_s                                    # the sample holds rows of both kinds
    w_loss, w_stat, w_grad = oracle.logits_ppo_step(
        case.logits[idx_d].cpu(), case.labels[idx_d].cpu(), case.prox_logp[idx_d].cpu(), case.old_logp[idx_d].cpu(),
        case.advantages[idx_d].cpu(), loss_mask=mask_s, rejection_sampling_cfg=rs,
        cu_seqlens=torch.tensor([0, n_s], dtype=torch.int32), temperature=case.temperature, **kw)
    ref_lp, ref_ent = oracle.logprobs_entropy_f64(case.logits[idx_d].cpu(), case.labels[idx_d].cpu(), case.temperature)
    assert float((s1["logprobs"][idx_d].cpu().double() - ref_lp).abs().max()) < 1e-4      # stated: 2e-3
    assert float((s1["entropy"][idx_d].cpu().double() - ref_ent).abs().max()) < 1e-4
    for k in ("clip_mask", "dual_clip_mask", "behave_mask"):
        assert torch.equal(s1[k][idx_d].cpu(), w_stat[k]), k
    # the oracle normalised by the masked tokens of its 64 rows, the full step by those of all rows
    want = w_grad.double() * (int(mask_s.sum()) / int(case.loss_mask.sum()))
    got = g1[idx_d].cpu()
    assert cosine(got, want) > 0.9999                                     # stated
    assert_same_magnitude(got, want, what="d_logits of the sampled rows")


def test_fused_step_replays_from_a_hip_graph(device):
    """The logits step (no rejection sampling, hence no host read) captured into a HIP graph: three replays on new
    inputs, with eager work and synchronisations in between, each equal to the eager result on the same inputs."""
    T, V = 96, 16384
    g = torch.Generator().manual_seed(12)
    x = torch.zeros(T, V, dtype=torch.bfloat16, device=device, requires_grad=True)
    labels = torch.randint(0, V, (T,), generator=g).to(device)
    prox, old, adv = (torch.zeros(T, device=device) for _ in range(3))
    mask = (torch.rand(T, generator=g) < 0.7).to(device)

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            x.copy_((3 * torch.randn(T, V, generator=gg)).bfloat16())
            ref = areal_amd.gather_logprobs(x, labels)
            prox.copy_(ref + 0.05 * torch.randn(T, generator=gg).to(device))
            old.copy_(ref + 0.05 * torch.randn(T, generator=gg).to(device))
            adv.copy_(torch.randn(T, generator=gg).to(device))

    def step():
        loss, stat = areal_amd.fused_logprobs_ppo_loss(x, labels, prox, old, adv, 0.2, mask, eps_clip_higher=0.28)
        loss.backward()
        return loss, stat["logprobs"]

    fill(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            x.grad = None
            step()
    torch.cuda.current_stream().wait_stream(side)
    x.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_loss, g_logp = step()
    g_grad = x.grad
    for seed in (1, 2, 3):
        fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = (g_loss.detach().clone(), g_logp.clone(), g_grad.clone())
        y = x.detach().clone().requires_grad_(True)                     # eager, same inputs
        e_loss, e_stat = areal_amd.fused_logprobs_ppo_loss(y, labels, prox, old, adv, 0.2, mask, eps_clip_higher=0.28)
        e_loss.backward()
        torch.cuda.synchronize()
        assert torch.equal(got[0], e_loss.detach()) and torch.equal(got[1], e_stat["logprobs"])
        assert torch.equal(got[2], y.grad)


def test_forward_only_calls_skip_the_gradient(device):
    """Under torch.no_grad (or with inputs that need no gradient) the fused entry points return the same loss and
    statistics without producing a gradient buffer."""
    lengths = [21, 30]
    case = synth.make_logits_case("t", lengths, 16384, 5, device, synth.per_sequence_normal_advantages(lengths, 2),
                                  ppo=dict(eps_clip=0.2))
    _finish_case(case)
    loss, stat, _ = _fused_step(case)
    with torch.no_grad():
        l2, s2 = areal_amd.fused_logprobs_ppo_loss(case.logits, case.labels, case.prox_logp, case.old_logp,
                                                   case.advantages, 0.2, case.loss_mask, cu_seqlens=case.cu_seqlens)
    assert not l2.requires_grad and float(l2) == pytest.approx(float(loss), rel=1e-6)
    for k in ("logprobs", "entropy", "loss", "importance_weight", "vocab_max_logits"):
        assert torch.allclose(s2[k], stat[k], rtol=1e-5, atol=1e-6), k
    assert torch.equal(s2["clip_mask"], stat["clip_mask"])
    # lm_head step
    g = torch.Generator().manual_seed(3)
    T, H, V = 300, 64, 1088
    hidden = torch.randn(T, H, generator=g).bfloat16().to(device)
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16().to(device)
    labels = torch.randint(0, V, (T,), generator=g).to(device)
    z = torch.zeros(T, device=device) - 6.0
    adv, mask = torch.randn(T, generator=g).to(device), (torch.rand(T, generator=g) < 0.7).to(device)
    h = hidden.clone().requires_grad_(True)
    la, sa = areal_amd.fused_lm_head_ppo_loss(h, weight, labels, z, z, adv, 0.2, mask)
    lb, sb = areal_amd.fused_lm_head_ppo_loss(hidden, weight, labels, z, z, adv, 0.2, mask)   # nothing requires grad
    assert not lb.requires_grad and float(lb) == pytest.approx(float(la.detach()), rel=1e-6)
    assert torch.allclose(sb["logprobs"], sa["logprobs"], atol=1e-6)


def test_second_backward_of_the_fused_step_is_refused(device):
    lengths = [9, 14]
    case = synth.make_logits_case("t", lengths, 8192, 8192, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  ppo=dict(eps_clip=0.2))
    _finish_case(case)
    x = case.logits.clone().requires_grad_(True)
    loss, _ = areal_amd.fused_logprobs_ppo_loss(x, case.labels, case.prox_logp, case.old_logp, case.advantages, 0.2,
                                                case.loss_mask)
    loss.backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="already handed out"):
        loss.backward()


@pytest.mark.parametrize(
    "V,dtype",
    [
        (151936, torch.bfloat16),   # register-resident rows
        (172040, torch.bfloat16),   # registers + LDS
        (250008, torch.float16),    # registers + LDS + a tail that is read twice
        (8200, torch.float16),      # two-pass kernel, 16-byte pieces
        (50257, torch.bfloat16),    # two-pass kernel, element by element
        (4099, torch.float32),      # the same in fp32
        (90112, torch.float32),     # fp32 rows held on the chip
        (151936, torch.float32),    # fp32 rows held on the chip in 24 bits per value
        (200000, torch.float32),    # the same, the rest read twice
    ],
)
def test_gradient_written_over_the_logits(device, V, dtype):
    """inplace_backward=True: the gradient takes the place of the logits, with the bits of the separate array, on every
    kernel behind the entry point; masked rows included (their gradient is zero)."""
    lengths = synth.lengths_uniform(5, 4, 12, seed=V)
    case = synth.make_logits_case("t", lengths, V, V, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  dtype=dtype, ppo=dict(eps_clip=0.2))
    _finish_case(case)
    loss, stat, grad = _fused_step(case)
    x = case.logits.clone().requires_grad_(True)
    l2, s2 = areal_amd.fused_logprobs_ppo_loss(x, case.labels, case.prox_logp, case.old_logp, case.advantages,
                                               loss_mask=case.loss_mask, cu_seqlens=case.cu_seqlens,
                                               temperature=case.temperature, inplace_backward=True, **case.ppo)
    assert torch.equal(x.detach(), grad)               # already there after the forward call
    l2.backward()
    assert torch.equal(x.grad, grad) and torch.equal(x.detach(), grad)
    assert torch.equal(l2.detach(), loss)
    for k in ("logprobs", "entropy", "loss", "importance_weight", "clip_mask", "vocab_max_logits", "vocab_min_logits"):
        assert torch.equal(s2[k], stat[k]), k


def test_gradient_written_over_logits_that_another_operation_produced(device):
    """The usual place of the call: the logits are the output of the lm_head product.  The gradient of the hidden
    states is that of the separate array; rows with a stride (a slice of a wider array) work the same way; an
    operation that kept the logits for its own backward is told that they changed."""
    g = torch.Generator().manual_seed(4)
    T, H, V = 40, 64, 16384
    hidden = torch.randn(T, H, generator=g).bfloat16().to(device)
    weight = (0.3 * torch.randn(V + 8, H, generator=g)).bfloat16().to(device)
    labels = torch.randint(0, V, (T,), generator=g).to(device)
    z = torch.zeros(T, device=device) - 9.0
    adv, mask = torch.randn(T, generator=g).to(device), (torch.rand(T, generator=g) < 0.7).to(device)

    def step(inplace, sliced, through=lambda t: t, factor=1.0):
        h = hidden.clone().requires_grad_(True)
        wide = through(h @ weight.T)
        beside = wide.detach()[:, V:].clone()            # what lies between the rows of the slice
        if sliced:
            logits = wide[:, :V]                         # row stride V + 8
        else:
            logits = wide[:, :V].contiguous()
        loss, _ = areal_amd.fused_logprobs_ppo_loss(logits, labels, z, z, adv, 0.2, mask, inplace_backward=inplace)
        (loss * factor).backward()
        assert torch.equal(wide.detach()[:, V:], beside)
        return loss.detach(), h.grad

    for sliced in (False, True):
        for factor in (1.0, 3.0):
            l0, g0 = step(False, sliced, factor=factor)
            l1, g1 = step(True, sliced, factor=factor)
            assert torch.equal(l0, l1) and torch.equal(g0, g1), (sliced, factor)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        step(True, True, through=lambda t: torch.sigmoid(t.float()).bfloat16().sigmoid())


def test_supervised_gradient_written_over_the_logits(device):
    lengths = [9, 14]
    case = synth.make_logits_case("t", lengths, 16384, 16384, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  ppo=dict(eps_clip=0.2))
    x = case.logits.clone().requires_grad_(True)
    loss, stat = areal_amd.fused_logprobs_sft_loss(x, case.labels, case.loss_mask, case.cu_seqlens)
    loss.backward()
    y = case.logits.clone().requires_grad_(True)
    l2, s2 = areal_amd.fused_logprobs_sft_loss(y, case.labels, case.loss_mask, case.cu_seqlens, inplace_backward=True)
    l2.backward()
    assert torch.equal(l2.detach(), loss.detach()) and torch.equal(y.detach(), x.grad) and torch.equal(y.grad, x.grad)
    assert torch.equal(s2["logprobs"], stat["logprobs"])


@pytest.mark.parametrize("V,dtype", [
    (81920, torch.bfloat16),     # 10 chunks: the shortest rows that take the shifted chunk grid
    (90112, torch.bfloat16),     # 11 chunks: a stride of an odd number of chunks
    (155648, torch.float16),     # 19 chunks
    (131072, torch.float16),     # 16 chunks
    (163840, torch.bfloat16),    # 20 chunks
    (180224, torch.bfloat16),    # 22 chunks: 21 in registers, one in LDS
    (262144, torch.bfloat16),    # 32 chunks: registers, LDS and the tail that is read twice
    (151936, torch.bfloat16),    # rows 296.75 KB apart: every row gets a shift of its own (0 to 2 KB)
    (50280, torch.float16),      # 7 chunks (two workgroups per compute unit), rows not a whole number of lines apart
    (100360, torch.bfloat16),    # 13 chunks, the same
    (200064, torch.bfloat16),    # 25 chunks (registers, LDS), rows 390.75 KB apart: a shift per row
    (180232, torch.float16),     # 23 chunks, rows not a whole number of lines apart
    (250888, torch.bfloat16),    # 31 chunks (registers, LDS and the tail that is read twice), the same
])
def test_rows_on_a_shifted_chunk_grid(device, V, dtype):
    """Rows of whole 8192-value chunks at a stride of whole chunks are walked on a chunk grid laid 1 KB back (the
    first 64 threads of chunk 0 hold the last 512 values of the row); rows that are not a whole number of KB (or of
    128-byte lines) apart on a grid laid back by an amount of the row's own (up to 2 KB: the first threads of chunk 0
    hold up to 1016 values from the end of the row).  Labels in every place that moves: the first and last 1024 values,
    both sides of the first chunk borders, the last value.  Against the oracle, in place, and against the same rows at
    another stride (another grid)."""
    lengths = synth.lengths_uniform(6, 8, 14, seed=V)
    case = synth.make_logits_case("t", lengths, V, V, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  dtype=dtype, ppo=dict(eps_clip=0.2))
    special = [0, 7, 8, 511, 512, 1023, 1024, 7679, 7680, 8191, 8192, 8703, 8704, 16383, 16384, V - 8193, V - 8192,
               V - 1025, V - 1024, V - 1017, V - 1016, V - 513, V - 512, V - 9, V - 8, V - 1]
    n = min(len(special), case.n_tokens)
    case.labels[:n] = torch.tensor(special[:n], device=device)
    case.loss_mask[:n] = True
    _finish_case(case)
    got = _fused_step(case)
    _compare(case, got, _oracle_step(case))
    # the gradient written over the logits: the same bits
    x = case.logits.clone().requires_grad_(True)
    l2, s2 = areal_amd.fused_logprobs_ppo_loss(x, case.labels, case.prox_logp, case.old_logp, case.advantages,
                                               loss_mask=case.loss_mask, cu_seqlens=case.cu_seqlens,
                                               temperature=case.temperature, inplace_backward=True, **case.ppo)
    assert torch.equal(x.detach(), got[2]) and torch.equal(l2.detach(), got[0])
    assert torch.equal(s2["logprobs"], got[1]["logprobs"]) and torch.equal(s2["entropy"], got[1]["entropy"])
    # the same rows inside a wider array (stride V + 8: another grid): the same results up to the order of the sums
    wide = torch.zeros(case.n_tokens, V + 8, dtype=dtype, device=device)
    wide[:, :V] = case.logits
    y = wide[:, :V].requires_grad_(True)
    l3, s3 = areal_amd.fused_logprobs_ppo_loss(y, case.labels, case.prox_logp, case.old_logp, case.advantages,
                                               loss_mask=case.loss_mask, cu_seqlens=case.cu_seqlens,
                                               temperature=case.temperature, **case.ppo)
    l3.backward()
    assert float((s3["logprobs"] - got[1]["logprobs"]).abs().max()) < 1e-5
    assert float(l3.detach()) == pytest.approx(float(got[0]), rel=1e-5)
    step = float(got[2].float().abs().max()) * (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11)
    assert float((y.grad.float() - got[2].float()).abs().max()) <= step
    assert float((y.grad == got[2]).float().mean()) > 0.999


@pytest.mark.parametrize("V,wide_V,dtype", [
    (100360, 100864, torch.bfloat16),   # 13 chunks in registers
    (180232, 180736, torch.float16),    # 23 chunks: registers and LDS
    (250888, 251392, torch.bfloat16),   # 31 chunks: registers, LDS and the tail that is read twice
])
def test_shift_changes_from_row_to_row_of_a_workgroup(device, V, wide_V, dtype):
    """More rows than workgroups: a workgroup goes from row to row, each with a shift of its own.  Against the same
    rows a whole number of KB apart (inside a wider array), which are walked on the plain grid: the same results up
    to the order of the sums.  Masked rows (zero gradient rows) among them."""
    T = 700
    lengths = [T]
    case = synth.make_logits_case("t", lengths, V, V, device, synth.per_sequence_normal_advantages(lengths, 5),
                                  dtype=dtype, ppo=dict(eps_clip=0.2))
    case.labels[:4] = torch.tensor([0, V - 1, V - 1017, 8192], device=device)
    case.labels[-4:] = torch.tensor([V - 8, 1023, V - 513, 7], device=device)
    case.loss_mask[:4] = True
    case.loss_mask[-4:] = True
    _finish_case(case)
    got = _fused_step(case)
    assert (wide_V * case.logits.element_size()) % 1024 == 0
    wide = torch.zeros(T, wide_V, dtype=dtype, device=device)
    wide[:, :V] = case.logits
    y = wide[:, :V].requires_grad_(True)
    l3, s3 = areal_amd.fused_logprobs_ppo_loss(y, case.labels, case.prox_logp, case.old_logp, case.advantages,
                                               loss_mask=case.loss_mask, cu_seqlens=case.cu_seqlens,
                                               temperature=case.temperature, **case.ppo)
    l3.backward()
    assert float((s3["logprobs"] - got[1]["logprobs"]).abs().max()) < 1e-5
    assert float((s3["entropy"] - got[1]["entropy"]).abs().max()) < 1e-5
    assert float(l3.detach()) == pytest.approx(float(got[0]), rel=1e-5)
    step = float(got[2].float().abs().max()) * (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11)
    assert float((y.grad.float() - got[2].float()).abs().max()) <= step
    assert float((y.grad == got[2]).float().mean()) > 0.999
    assert bool((wide[:, V:] == 0).all())
    masked = ~case.loss_mask
    assert bool(masked.any()) and bool((got[2][masked] == 0).all())



def _rows_in_a_flat_array(rows, stride, lead):
    """The rows copied into a flat array filled with 7, `lead` values in and `stride` values apart."""
    T, V = rows.shape
    flat = torch.full((lead + T * stride + 16,), 7.0, dtype=rows.dtype, device=rows.device)
    view = flat.as_strided((T, V), (stride, 1), lead)
    view.copy_(rows)
    return flat, view


def _untouched_outside_the_rows(flat, T, V, stride, lead):
    seen = flat.clone()
    seen.as_strided((T, V), (stride, 1), lead).fill_(7.0)
    return bool((seen == 7.0).all())


@pytest.mark.parametrize("V,stride,lead,dtype,n_seq", [
    (50257, 50257, 0, torch.bfloat16, 6),     # 7 chunks (two workgroups per compute unit), rows 2 bytes off and more
    (32001, 32001, 3, torch.float16, 6),      # 4 chunks, the array itself 6 bytes into a 16-byte piece
    (151643, 151643, 0, torch.bfloat16, 6),   # 19 chunks
    (151936, 151937, 0, torch.bfloat16, 6),   # rows of whole pieces at a stride that is not
    (151936, 151936, 1, torch.bfloat16, 6),   # an array that starts 2 bytes into a piece: every row split the same way
    (40957, 40957, 0, torch.bfloat16, 60),    # the last chunk holds a piece only in rows that start late in theirs
    (172031, 172031, 5, torch.float16, 40),   # registers + LDS: the chunk in LDS holds one piece, in some rows
    (250002, 250003, 0, torch.bfloat16, 40),  # registers, LDS and the tail that is read twice; more rows than workgroups
])
def test_rows_at_any_alignment(device, V, stride, lead, dtype, n_seq):
    """16-bit rows that do not start on 16-byte boundaries (V or the stride not a multiple of 8, or the array itself
    inside a 16-byte piece) are held in registers like the others: the first and the last 16-byte piece of the memory
    that holds a row are shared with its neighbours.  Labels at both ends of the row; against the oracle; nothing
    outside the rows is written; and the same bits when the gradient is written over the logits."""
    lengths = synth.lengths_uniform(n_seq, 8, 14, seed=V)
    case = synth.make_logits_case("t", lengths, V, V, device, synth.per_sequence_normal_advantages(lengths, 3),
                                  dtype=dtype, ppo=dict(eps_clip=0.2))
    T = case.n_tokens
    special = [0, 1, 6, 7, 8, 9, 1023, 1024, 8191, 8192, 16383, 16384, V - 8193, V - 8192, V - 1025, V - 1024, V - 17,
               V - 16, V - 9, V - 8, V - 7, V - 2, V - 1]
    n = min(len(special), T)
    case.labels[:n] = torch.tensor(special[:n], device=device)
    case.loss_mask[:n] = True
    _finish_case(case)
    flat, view = _rows_in_a_flat_array(case.logits, stride, lead)
    x = view.detach().requires_grad_(True)
    kw = dict(loss_mask=case.loss_mask, cu_seqlens=case.cu_seqlens, temperature=case.temperature, **case.ppo)
    loss, stat = areal_amd.fused_logprobs_ppo_loss(x, case.labels, case.prox_logp, case.old_logp, case.advantages, **kw)
    loss.backward()
    assert x.grad.data_ptr() % 16 == x.data_ptr() % 16
    got = (loss.detach(), stat, x.grad)
    _compare(case, got, _oracle_step(case))
    assert torch.equal(view, case.logits) and _untouched_outside_the_rows(flat, T, V, stride, lead)
    # the gradient written over the logits: the same bits, and nothing but the rows is written
    flat2, view2 = _rows_in_a_flat_array(case.logits, stride, lead)
    y = view2.detach().requires_grad_(True)
    l2, s2 = areal_amd.fused_logprobs_ppo_loss(y, case.labels, case.prox_logp, case.old_logp, case.advantages,
                                               inplace_backward=True, **kw)
    assert torch.equal(y.detach(), got[2]) and torch.equal(l2.detach(), got[0])
    assert torch.equal(s2["logprobs"], stat["logprobs"]) and torch.equal(s2["entropy"], stat["entropy"])
    assert _untouched_outside_the_rows(flat2, T, V, stride, lead)


@pytest.mark.parametrize("V,dtype", [(50257, torch.bfloat16), (151643, torch.float16), (250002, torch.bfloat16)])
def test_register_kernel_and_twice_read_kernel_agree_on_unaligned_rows(device, V, dtype):
    """Through the C ABI: the same unaligned rows with the gradient array at the same offset inside a 16-byte piece as
    the logits (rows held in registers) and at another offset (the kernel that reads a row twice).  The same results up
    to the order of the sums, and neither writes outside its rows."""
    import ctypes as C
    from areal_amd import _native as N, functional as F

    lib = N.load()
    T = 300
    g = torch.Generator(device=device).manual_seed(V)
    logits = (torch.randn(T, V, device=device, generator=g) * 3).to(dtype)
    labels = torch.randint(0, V, (T,), device=device, generator=g)
    labels[:4] = torch.tensor([0, V - 1, 7, V - 8], device=device)
    prox = torch.full((T,), -12.0, device=device)
    adv = torch.randn(T, device=device, generator=g)
    mask = (torch.rand(T, device=device, generator=g) < 0.7).to(torch.uint8)
    mask[:4] = 1
    counts = F._count_nonzero(mask)
    params = F._ppo_params(0.2, None, None, False)
    work = torch.zeros(2, dtype=torch.int32, device=device)
    stream = torch.cuda.current_stream(device)
    results = []
    for lead in (0, 3):                  # values between a 16-byte boundary and the gradient array
        flat = torch.full((lead + T * V + 16,), 7.0, dtype=dtype, device=device)
        assert flat.data_ptr() % 16 == 0 and logits.data_ptr() % 16 == 0
        dlogits = flat.as_strided((T, V), (V, 1), lead)
        f32 = dict(dtype=torch.float32, device=device)
        logp, ent, stat_loss, ratio = (torch.empty(T, **f32) for _ in range(4))
        flags = torch.empty(T, dtype=torch.uint8, device=device)
        N.check(lib.aa_logits_ppo_fused(
            F._ptr(logits), F._DTYPES[dtype], T, V, V, F._ptr(labels), 1.0, T, F._ptr(prox), F._ptr(adv), F._ptr(mask),
            None, C.byref(params), F._ptr(counts), None, F._ptr(logp), F._ptr(ent), None, None, F._ptr(stat_loss),
            F._ptr(ratio), F._ptr(flags), F._ptr(dlogits), F._ptr(work), C.c_void_p(stream.cuda_stream)),
            "aa_logits_ppo_fused")
        torch.cuda.synchronize()
        assert _untouched_outside_the_rows(flat, T, V, V, lead)
        results.append((dlogits.clone(), logp, ent, stat_loss, flags))
    (g0, lp0, e0, sl0, f0), (g1, lp1, e1, sl1, f1) = results
    assert float((lp0 - lp1).abs().max()) < 1e-5 and float((e0 - e1).abs().max()) < 1e-5
    assert torch.equal(f0, f1) and torch.allclose(sl0, sl1, rtol=1e-4, atol=1e-6)
    step = float(g1.float().abs().max()) * (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11)
    assert float((g0.float() - g1.float()).abs().max()) <= step
    assert float((g0 == g1).float().mean()) > 0.999
    assert bool((g0[mask == 0] == 0).all()) and bool((g1[mask == 0] == 0).all())

