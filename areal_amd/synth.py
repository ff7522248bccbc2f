"""Seeded synthetic micro-batches in the packed 1-D layout, shaped like the benchmark configurations.

The generators only produce inputs (logits or hidden states, labels, masks,
advantages, ``cu_seqlens``).  The behaviour / proximal log-probs are "reference
log-prob plus noise", so the caller supplies the reference log-probs (from the
CPU oracle in tests, from the forward kernel in the benchmark) and calls
``attach_old_and_prox``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch


@dataclass
class PackedCase:
    name: str
    cu_seqlens: torch.Tensor            # int32 [B+1]
    labels: torch.Tensor                # int64 [T]
    loss_mask: torch.Tensor             # bool  [T]
    advantages: torch.Tensor            # fp32  [T]
    logits: torch.Tensor | None = None  # [T, V]
    hidden: torch.Tensor | None = None  # [T, H]
    weight: torch.Tensor | None = None  # [V, H]
    old_logp: torch.Tensor | None = None
    prox_logp: torch.Tensor | None = None
    temperature: float = 1.0
    ppo: dict = field(default_factory=dict)  # eps_clip, eps_clip_higher, c_clip, rejection_sampling kwargs

    @property
    def n_tokens(self) -> int:
        return int(self.labels.shape[0])


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def lengths_uniform(n_seqs: int, lo: int, hi: int, seed: int) -> list[int]:
    """Integer lengths uniform in [lo, hi]."""
    return torch.randint(lo, hi + 1, (n_seqs,), generator=_gen(seed)).tolist()


def lengths_lognormal(n_seqs: int, mu: float, sigma: float, lo: int, hi: int, seed: int) -> list[int]:
    """round(exp(N(mu, sigma^2))) clipped to [lo, hi]."""
    z = torch.randn(n_seqs, generator=_gen(seed), dtype=torch.float64)
    return [int(min(max(round(math.exp(mu + sigma * float(v))), lo), hi)) for v in z]


def truncate_to_total(lengths: list[int], total: int) -> list[int]:
    """Leading sequences whose lengths add up to ``total`` (the last one is shortened)."""
    out, acc = [], 0
    for n in lengths:
        if acc >= total:
            break
        n = min(n, total - acc)
        out.append(n)
        acc += n
    if acc < total:
        out[-1] += total - acc
    return out


def cu_from_lengths(lengths: list[int]) -> torch.Tensor:
    cu = [0]
    for n in lengths:
        cu.append(cu[-1] + n)
    return torch.tensor(cu, dtype=torch.int32)


def prefix_mask(lengths: list[int], masked_fraction: float) -> torch.Tensor:
    """loss_mask with the first floor(fraction * len) tokens of every sequence set to 0."""
    parts = []
    for n in lengths:
        m = torch.ones(n, dtype=torch.bool)
        m[: int(masked_fraction * n)] = False
        parts.append(m)
    return torch.cat(parts)


def alternating_mask(lengths: list[int], span: int) -> torch.Tensor:
    """Multi-turn mask: spans of ``span`` tokens alternate masked / unmasked, starting masked."""
    parts = []
    for n in lengths:
        idx = torch.arange(n)
        parts.append(((idx // span) % 2) == 1)
    return torch.cat(parts)


def per_sequence_normal_advantages(lengths: list[int], seed: int) -> torch.Tensor:
    a = torch.randn(len(lengths), generator=_gen(seed))
    return torch.repeat_interleave(a, torch.tensor(lengths))


def grpo_advantages(lengths: list[int], group_size: int, p_reward: float, seed: int, eps: float = 1e-5) -> torch.Tensor:
    """Bernoulli(p) rewards, normalised by the mean / unbiased std of each group of ``group_size`` sequences."""
    n = len(lengths)
    r = (torch.rand(n, generator=_gen(seed)) < p_reward).float()
    adv = torch.zeros(n)
    for g0 in range(0, n, group_size):
        grp = r[g0 : g0 + group_size]
        std = grp.std(unbiased=True) if grp.numel() > 1 else torch.zeros(())
        adv[g0 : g0 + group_size] = (grp - grp.mean()) / (std + eps)
    return torch.repeat_interleave(adv, torch.tensor(lengths))


def random_logits(T: int, V: int, std: float, seed: int, device, dtype=torch.bfloat16, rows_per_chunk: int = 2048):
    """``std * N(0,1)`` logits generated chunk by chunk on ``device`` (bounded fp32 temporaries)."""
    out = torch.empty(T, V, dtype=dtype, device=device)
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    for a in range(0, T, rows_per_chunk):
        b = min(a + rows_per_chunk, T)
        out[a:b] = (torch.randn(b - a, V, generator=g, device=device, dtype=torch.float32) * std).to(dtype)
    return out


def attach_old_and_prox(case: PackedCase, ref_logp: torch.Tensor, noise: float, seed: int) -> PackedCase:
    """old_logp and prox_logp = reference log-prob + independent N(0, noise^2) draws."""
    g = _gen(seed)
    n = case.n_tokens
    ref = ref_logp.detach().float().cpu()[:n]
    case.old_logp = (ref + noise * torch.randn(n, generator=g)).to(ref_logp.device)
    case.prox_logp = (ref + noise * torch.randn(n, generator=g)).to(ref_logp.device)
    return case


def make_logits_case(
    name: str,
    lengths: list[int],
    V: int,
    seed: int,
    device,
    advantages: torch.Tensor,
    loss_mask: torch.Tensor | None = None,
    logits_std: float = 3.0,
    dtype=torch.bfloat16,
    temperature: float = 1.0,
    ppo: dict | None = None,
) -> PackedCase:
    T = sum(lengths)
    labels = torch.randint(0, V, (T,), generator=_gen(seed + 1), dtype=torch.int64)
    mask = prefix_mask(lengths, 0.3) if loss_mask is None else loss_mask
    return PackedCase(
        name=name,
        cu_seqlens=cu_from_lengths(lengths).to(device),
        labels=labels.to(device),
        loss_mask=mask.to(device),
        advantages=advantages.float().to(device),
        logits=random_logits(T, V, logits_std, seed + 2, device, dtype),
        temperature=temperature,
        ppo=dict(ppo or {}),
    )


V_QWEN = 151936


def config0(device, seed: int = 0, V: int = V_QWEN, n_seqs: int = 16, lo: int = 64, hi: int = 512) -> PackedCase:
    """Logits path, CPU-runnable: 16 sequences of 64..512 tokens, per-sequence N(0,1) advantages, eps_clip 0.2."""
    lengths = lengths_uniform(n_seqs, lo, hi, seed)
    return make_logits_case(
        "cfg0", lengths, V, seed, device, per_sequence_normal_advantages(lengths, seed + 3), ppo=dict(eps_clip=0.2)
    )


def config1(device, seed: int = 0, V: int = V_QWEN, n_seqs: int = 64, total_tokens: int | None = None,
            lo: int = 128, hi: int = 4096) -> PackedCase:
    """8B-shape logits path: 64 sequences, lengths lognormal(7.5, 0.6) clipped to [128, 4096], GRPO groups of
    16 with Bernoulli(0.4) rewards, decoupled loss with importance-weight cap 5.0.  ``total_tokens`` keeps the
    leading sequences that add up to that many tokens."""
    lengths = lengths_lognormal(n_seqs, 7.5, 0.6, lo, hi, seed)
    name = "cfg1"
    if total_tokens is not None:
        lengths = truncate_to_total(lengths, total_tokens)
        name = f"cfg1-{total_tokens}"
    adv = grpo_advantages(lengths, 16, 0.4, seed + 3)
    ppo = dict(eps_clip=0.2, rejection_sampling=dict(level="token", action="mask", metric="ratio", upper=5.0))
    return make_logits_case(name, lengths, V, seed, device, adv, ppo=ppo)


# ----------------------------------------------------------------------------
# fused lm_head configurations: hidden states and lm_head weights instead of logits
# ----------------------------------------------------------------------------
def random_matrix(rows: int, cols: int, std: float, seed: int, device, rows_per_chunk: int = 8192) -> torch.Tensor:
    """``std * N(0,1)`` bf16 matrix generated chunk by chunk on ``device``."""
    out = torch.empty(rows, cols, dtype=torch.bfloat16, device=device)
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    for a in range(0, rows, rows_per_chunk):
        b = min(a + rows_per_chunk, rows)
        out[a:b] = (torch.randn(b - a, cols, generator=g, device=device, dtype=torch.float32) * std).to(torch.bfloat16)
    return out


def lengths_until_total(lo: int, hi: int, total: int, seed: int) -> list[int]:
    """Uniform lengths in [lo, hi], drawn until they add up to ``total`` (the last one is shortened)."""
    out, acc, g = [], 0, _gen(seed)
    while acc < total:
        n = int(torch.randint(lo, hi + 1, (1,), generator=g))
        n = min(n, total - acc)
        out.append(n)
        acc += n
    return out


def make_hidden_case(name, lengths, H, V, seed, device, advantages, loss_mask=None, temperature=1.0, ppo=None,
                     labels=None) -> PackedCase:
    T = sum(lengths)
    if labels is None:
        labels = torch.randint(0, V, (T,), generator=_gen(seed + 1), dtype=torch.int64)
    mask = prefix_mask(lengths, 0.3) if loss_mask is None else loss_mask
    return PackedCase(
        name=name,
        cu_seqlens=cu_from_lengths(lengths).to(device),
        labels=labels.to(device),
        loss_mask=mask.to(device),
        advantages=advantages.float().to(device),
        hidden=random_matrix(T, H, 1.0, seed + 2, device),
        weight=random_matrix(V, H, 0.02, seed + 4, device),
        temperature=temperature,
        ppo=dict(ppo or {}),
    )


def config2(device, seed: int = 0, T: int = 16384, H: int = 4096, V: int = V_QWEN) -> PackedCase:
    """Fused lm_head path at the 8B shape: hidden [16384, 4096] ~ N(0,1), W [151936, 4096] ~ N(0, 0.02^2), labels
    and masks as in configuration 0 on sequences of 64..512 tokens covering T tokens."""
    lengths = lengths_until_total(64, 512, T, seed)
    return make_hidden_case("cfg2", lengths, H, V, seed, device, per_sequence_normal_advantages(lengths, seed + 3),
                            ppo=dict(eps_clip=0.2))


def config3(device, seed: int = 0, n_seqs: int = 8, seq_len: int = 32768, H: int = 4096, V: int = V_QWEN) -> PackedCase:
    """Long-context agentic rollout: 8 packed sequences of 32768 tokens, multi-turn mask (alternating 512-token
    masked / unmasked spans), dual clip c = 3, importance-weight cap 5, eps_clip 0.2 low / 0.28 high."""
    lengths = [seq_len] * n_seqs
    ppo = dict(eps_clip=0.2, eps_clip_higher=0.28, c_clip=3.0,
               rejection_sampling=dict(level="token", action="mask", metric="ratio", upper=5.0))
    return make_hidden_case("cfg3", lengths, H, V, seed, device, per_sequence_normal_advantages(lengths, seed + 3),
                            loss_mask=alternating_mask(lengths, 512), ppo=ppo)


def config4(device, seed: int = 0, T: int = 32768, H: int = 5376, V: int = 262144, argmax_fraction: float = 0.2,
            lo: int = 32, hi: int = 256) -> PackedCase:
    """Large vocabulary, wide hidden: hidden [32768, 5376], W [262144, 5376], temperature 0.7, sequences of
    32..256 tokens, 20 % of the labels are the argmax token of their row, 80 % uniform."""
    lengths = lengths_until_total(lo, hi, T, seed)
    case = make_hidden_case("cfg4", lengths, H, V, seed, device, per_sequence_normal_advantages(lengths, seed + 3),
                            temperature=0.7, ppo=dict(eps_clip=0.2))
    pick = (torch.rand(T, generator=_gen(seed + 5)) < argmax_fraction).to(device)
    labels = case.labels.clone()
    rows = 64 if torch.device(device).type == "cpu" else 1024
    on_cpu = torch.device(device).type == "cpu"
    for a in range(0, T, rows):  # tiled argmax of hidden @ W.T (input generation only)
        b = min(a + rows, T)
        h, w = case.hidden[a:b], case.weight
        scores = h.float() @ w.float().t() if on_cpu else torch.matmul(h, w.t())
        labels[a:b] = torch.where(pick[a:b], scores.argmax(-1), labels[a:b])
    case.labels = labels
    return case
