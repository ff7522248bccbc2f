#!/usr/bin/env python3
"""Benchmark of the PPO/GRPO log-prob + entropy + actor-loss path (forward and backward) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg1|cfg1-32k|cfg0|cfg2|cfg3|cfg4|adv|aux|hbm|mfma|torch-ops]

One "step" is one pass of the hot path over one synthetic packed micro-batch that is already resident in HBM.

* logits workloads (cfg0, cfg1, cfg1-32k; cfg1 is the default, the configuration the metric is quoted on):
  rejection sampling (importance-weight cap) -> fused log-prob / entropy / clipped PPO loss / d(logits) -> scalar
  loss, i.e. ``fused_logprobs_ppo_loss(...)`` followed by ``loss.backward()``.  Roofline: HBM, algorithmic bytes
  4 * V per token (the bf16 logits read once, their gradient written once); ``--logits-dtype f32`` casts the logits
  to fp32 first (8 * V per token).  The line also carries ``sft_loss_same_logits``: the supervised loss on the same
  logits, fused in one pass against the log-prob op followed by the loss and a separate backward pass, and
  ``forward_only_logprobs``: the forward-only op on the same logits (read once: 2 * V bytes per bf16 token).
* fused lm_head workloads (cfg2, cfg3, cfg4): ``fused_lm_head_ppo_loss(hidden, W, labels, ...)`` followed by
  ``loss.backward()``: lm_head, log-prob / entropy, PPO loss and the gradients d(hidden), d(W) on this library's own
  bf16 MFMA tile GEMM; the forward writes no logits.  Roofline: bf16 MFMA, from HIP events around every step of the
  same timed loop that gives ``ms_per_step``.  ``needed_flops_per_step``: 2 T V H for the logits of every token +
  4 T_grad V H for the two gradient GEMMs over the tokens that have a gradient (masked tokens have none and are left
  out; ``--dense-backward`` multiplies their zero rows through like the reference's autograd).  With
  ``--lmhead-backward recompute`` the backward forms the logits of those tokens a second time (2 T_grad V H more
  flops are executed; they are not counted as needed).  ``flops_per_step_6TVH`` is the dense figure 6 T V H.

* adv: the advantage pipeline that precedes the loss (not one of the headline configurations): GAE reverse scan plus batch
  normalisation over a padded [512, 4096] batch.  Roofline: HBM, 20 bytes per token for the scan (rewards, values,
  mask read; advantages, returns written).

* aux: the other per-token pieces around the loss at the configs[1] token count (SAPO loss, clipped value loss, DPO
  loss over 32 pairs, M2PO masking, proximal log-prob approximation, the 36 logged moments of the approximation
  metrics) and the packing helpers (pack of a [512, 4096] batch, un-padding of
  [32768 + pad, 151936] bf16 logits).  Roofline: HBM, on the logits un-padding copy (4 * V bytes per token).

Prints ONE JSON line.  Besides the whole-step throughput it carries
  roofline      of the dominant kernel(s), timed with HIP events on the launch stream;
  cpu_baseline  the CPU oracle (a PyTorch restatement of the reference path) timed on this machine's host cores on a
                bounded token sample of the same workload (three windows: first, middle and last tokens);
  parity        the GPU result checked against that oracle on the same sample;
and, in the default run only (every GPU timing is taken before the first CPU baseline starts):
  configs1_cut_to_32k_tokens  the cfg1 sequences cut at 32 768 tokens;
  logits_config0              the cfg0 workload with its own roofline, and the plain copy kernel on the same buffers;
  fp32_logits_cut_to_32k_tokens  the 32 768-token cut with the logits cast to fp32 (8 * V bytes per token);
  fused_lm_head               the same figures for the cfg2 workload, so that one run reports both paths;
  fused_lm_head_cfg3, _cfg4   the cfg3 and cfg4 workloads (GPU only: three timed steps each, their own roofline).

``--workload hbm`` runs plain HBM streams (aa_hbm_stream_probe: read only, write only, copy, either cache policy), the
measured ceilings of the logits path.  ``--workload mfma`` runs the MFMA-only loop (aa_mfma_only_loop: no LDS, no memory traffic), the measured ceiling that
the fused lm_head figures are also quoted against (``roofline.frac_of_mfma_only_loop``).  ``--workload torch-ops``
times what the reference itself executes for the two paths, restated in plain torch ops, on this GPU (cfg1-32k and
cfg2; ``--torch-compile`` adds the compiled form), beside this library's step on the same inputs.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published peak
METRIC = "tokens/sec for logprob+entropy+PPO loss fwd+bwd; % HBM / % MFMA peak"  # BASELINE.json's metric, verbatim
LOGITS_WORKLOADS = ("cfg0", "cfg1", "cfg1-32k")
FUSED_WORKLOADS = ("cfg2", "cfg3", "cfg4")
ADV_WORKLOADS = ("adv", "aux")
MFMA_WORKLOADS = ("mfma", "hbm")
TORCH_WORKLOADS = ("torch-ops",)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg1", choices=LOGITS_WORKLOADS + FUSED_WORKLOADS + ADV_WORKLOADS + MFMA_WORKLOADS + TORCH_WORKLOADS)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--cpu-tokens", type=int, default=6144,
                    help="token sample of the CPU baseline (0 = skip); fused lm_head workloads use at most 384")
    ap.add_argument("--cpu-iters", type=int, default=3)
    ap.add_argument("--no-fused-extra", action="store_true",
                    help="default workload only: do not append the cfg2 fused lm_head figures")
    ap.add_argument("--rs-action", choices=["mask", "clamp"], default=None,
                    help="override the action of the workload's importance-weight cap (cfg1 is quoted with 'mask', "
                         "the documented equivalent of behave_imp_weight_cap; 'clamp' keeps every token)")
    ap.add_argument("--dense-backward", action="store_true",
                    help="lm_head workloads: run masked tokens through the gradient GEMMs too (as the reference's "
                         "autograd does) instead of leaving their zero rows out")
    ap.add_argument("--lmhead-backward", choices=["carry", "recompute"], default="carry",
                    help="lm_head workloads: how the d(logits) rows of the backward are obtained (see "
                         "fused_lm_head_ppo_loss)")
    ap.add_argument("--no-forward-of-masked", action="store_true",
                    help="lm_head workloads, outside the reference's semantics: masked tokens skip the lm_head "
                         "altogether (fused_lm_head_ppo_loss(forward_masked_tokens=False)); only ms_per_step and value "
                         "reflect it, and the line says so in config.path")
    ap.add_argument("--logits-dtype", choices=["bf16", "f32"], default="bf16",
                    help="logits workloads: hand the kernels fp32 logits (what a Megatron-style head emits) instead of "
                         "bf16; 8 bytes per element instead of 4")
    ap.add_argument("--vocab", type=int, default=None,
                    help="cfg1-32k only: width of the logits rows instead of 151936 (other vocabulary sizes through the "
                         "same kernels; the traffic factor quoted is that of 151936)")
    ap.add_argument("--steps-only", action="store_true",
                    help="fused lm_head workloads: launch the steps of the selected backward mode only (no stand-alone "
                         "op, no other mode), so that every dispatch a profiler sees belongs to a step")
    ap.add_argument("--torch-compile", action="store_true",
                    help="torch-ops only: also time the reference's two vocabulary functions under torch.compile, as "
                         "the reference wraps them on GPUs (compilation takes a minute or two)")
    ap.add_argument("--copy-launches", type=int, default=0,
                    help="also launch the plain copy kernel this many times over the logits buffer (lm_head workloads: the weight matrix) "
                         "(the calibration point for FETCH_SIZE / WRITE_SIZE counters)")
    return ap.parse_args()


RS_ACTION = None  # set from --rs-action


def ppo_kwargs(case):
    from areal_amd import RejectionSamplingConfig

    kw = dict(case.ppo)
    rs = kw.pop("rejection_sampling", None)
    if rs and RS_ACTION:
        rs = dict(rs, action=RS_ACTION)
    cfg = RejectionSamplingConfig(**rs) if rs else None
    return kw, cfg


def cosine(a, b) -> float:
    a, b = a.double().reshape(-1), b.double().reshape(-1)
    return float(a @ b / (a.norm() * b.norm()))


def sample_windows(n_total: int, n_sample: int):
    """Token indices of the parity / CPU sample: three equal windows, the first, the middle and the last tokens of the
    workload (sorted, without repeats), and a description of them."""
    import torch

    n = min(n_sample, n_total)
    w = n // 3
    sizes = [w, w, n - 2 * w]
    starts = [0, (n_total - sizes[1]) // 2, n_total - sizes[2]]
    idx = torch.unique(torch.cat([torch.arange(a, a + k) for a, k in zip(starts, sizes)]))
    desc = ", ".join(f"{a}..{a + k - 1}" for a, k in zip(starts, sizes) if k > 0)
    return idx, desc


def time_events(launch, iters: int, stream):
    """(mean, min) milliseconds of ``launch()`` between HIP events recorded on ``stream``."""
    import torch

    for _ in range(5):
        launch()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record(stream)
        launch()
        b.record(stream)
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) for a, b in evs)
    return sum(times) / len(times), times[0]


# ----------------------------------------------------------------------------------------------------------------
# logits path
# ----------------------------------------------------------------------------------------------------------------
def build_logits_case(name: str, seed: int, device, vocab: int | None = None):
    import areal_amd
    from areal_amd import synth

    if name == "cfg0":
        case = synth.config0(device, seed)
        desc = "configs[0]: 16 packed seqs, lengths U[64,512], V=151936, eps_clip=0.2"
    elif name == "cfg1":
        case = synth.config1(device, seed)
        desc = ("configs[1]: 64 packed seqs, lengths lognormal(7.5,0.6) clipped to [128,4096], V=151936, GRPO groups "
                "of 16, decoupled loss, importance-weight cap 5.0 (token/mask/ratio)")
    elif vocab is not None:
        case = synth.config1(device, seed, V=vocab, total_tokens=32768)
        desc = f"configs[1] truncated to the leading sequences that total 32768 tokens, with a vocabulary of {vocab}"
    else:
        case = synth.config1(device, seed, total_tokens=32768)
        desc = "configs[1] truncated to the leading sequences that total 32768 tokens"
    ref = areal_amd.gather_logprobs(case.logits, case.labels, case.temperature)
    synth.attach_old_and_prox(case, ref, 0.05, seed + 9)
    return case, desc


def run_logits_steps(case, n, kw, cfg):
    import areal_amd

    x = case.logits
    loss = None
    for _ in range(n):
        x.grad = None
        loss, _ = areal_amd.fused_logprobs_ppo_loss(
            x, case.labels, case.prox_logp, case.old_logp, case.advantages, loss_mask=case.loss_mask,
            rejection_sampling=cfg, cu_seqlens=case.cu_seqlens, temperature=case.temperature, **kw,
        )
        loss.backward()
    return loss


def time_fused_logits_kernel(case, kw, cfg, iters: int, inplace: bool = False):
    """Duration of aa_logits_ppo_fused alone, HIP events on the launch stream, outputs pre-allocated.  ``inplace``:
    the gradient is written over the logits (which are lost: the caller times this variant last)."""
    import torch

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    dev = case.logits.device
    T, V = case.logits.shape
    f32 = dict(dtype=torch.float32, device=dev)
    m8 = F._mask_u8(case.loss_mask)
    prox, old, adv = (F._f32(t) for t in (case.prox_logp, case.old_logp, case.advantages))
    params = F._ppo_params(kw["eps_clip"], kw.get("eps_clip_higher"), kw.get("c_clip"), cfg is not None)
    if cfg is not None:
        mask_eff, w, counts = F._rejection_sampling_device(prox, old, m8, m8.shape, case.cu_seqlens, cfg)
        if cfg.action != "mask":
            mask_eff = m8
    else:
        mask_eff, w, counts = m8, None, F._count_nonzero(m8)
    logp, ent, sl, ratio, vmax, vmin = (torch.empty(T, **f32) for _ in range(6))
    flags = torch.empty(T, dtype=torch.uint8, device=dev)
    dlogits = case.logits if inplace else torch.empty_like(case.logits)
    stream = torch.cuda.current_stream(dev)

    def launch():
        N.check(
            lib.aa_logits_ppo_fused(
                F._ptr(case.logits), F._DTYPES[case.logits.dtype], T, V, V, F._ptr(case.labels), 1.0 / case.temperature, T,
                F._ptr(prox), F._ptr(adv), F._ptr(mask_eff), F._ptr(w), C.byref(params), F._ptr(counts), None,
                F._ptr(logp), F._ptr(ent), None, None, F._ptr(sl), F._ptr(ratio), F._ptr(flags), F._ptr(dlogits),
                F._ptr(F._work_words(dev)), C.c_void_p(stream.cuda_stream),
            ),
            "aa_logits_ppo_fused",
        )

    return time_events(launch, iters, stream)


def logits_gpu_sample(case, kw, cfg, n_tokens: int):
    """The GPU path on the sample tokens (see sample_windows), with everything the CPU phase needs copied to the host:
    the workload itself can be freed before the CPU baseline runs."""
    import torch

    import areal_amd

    idx, desc = sample_windows(case.n_tokens, n_tokens)
    n = int(idx.numel())
    idx_d = idx.to(case.logits.device)
    take = lambda t: t[idx_d]
    cu = torch.tensor([0, n], dtype=torch.int32)  # token-level options only: segments do not matter here
    x = take(case.logits).detach().clone().requires_grad_(True)
    loss, stat = areal_amd.fused_logprobs_ppo_loss(
        x, take(case.labels), take(case.prox_logp), take(case.old_logp), take(case.advantages),
        loss_mask=take(case.loss_mask), rejection_sampling=cfg, cu_seqlens=cu.to(x.device),
        temperature=case.temperature, **kw,
    )
    loss.backward()
    torch.cuda.synchronize()
    cpu = lambda t: take(t).cpu()
    return dict(
        n=n, windows=desc, cu=cu, kw=kw, cfg=cfg, temperature=case.temperature,
        args=(x.detach().cpu(), cpu(case.labels), cpu(case.prox_logp), cpu(case.old_logp), cpu(case.advantages)),
        loss_mask=cpu(case.loss_mask),
        gpu=dict(loss=float(loss.detach()), logprobs=stat["logprobs"].cpu(), clip_mask=stat["clip_mask"].cpu(),
                 grad=x.grad.cpu()),
    )


def logits_cpu_phase(sample, iters: int):
    """Oracle fwd+bwd on the sample tokens (host cores), and the GPU results of logits_gpu_sample checked against it."""
    import torch

    import oracle

    n, g = sample["n"], sample["gpu"]
    okw = dict(sample["kw"], loss_mask=sample["loss_mask"], rejection_sampling_cfg=sample["cfg"], cu_seqlens=sample["cu"],
               temperature=sample["temperature"])
    threads = torch.get_num_threads()
    oracle.logits_ppo_step(*sample["args"], **okw)  # warm-up
    t0 = time.perf_counter()
    for _ in range(iters):
        w_loss, w_stat, w_grad = oracle.logits_ppo_step(*sample["args"], **okw)
    dt = (time.perf_counter() - t0) / iters
    parity = dict(
        tokens=n, token_windows=sample["windows"],
        logp_max_abs_err=float((g["logprobs"] - w_stat["logprobs"]).abs().max()),
        loss_rel_err=abs(g["loss"] - float(w_loss)) / max(abs(float(w_loss)), 1e-12),
        grad_cosine=cosine(g["grad"], w_grad),
        grad_norm_ratio=float(g["grad"].double().norm() / w_grad.double().norm()),
        masks_equal=bool(torch.equal(g["clip_mask"], w_stat["clip_mask"])),
    )
    baseline = dict(
        value=n / dt, unit="tokens/s", cores=threads, kind="port",
        sample=f"{n} tokens of the workload (tokens {sample['windows']}), {iters} timed fwd+bwd passes of the PyTorch "
               f"CPU oracle (chunked fp32 log_softmax + gather + entropy + PPO loss + autograd to bf16 d(logits))",
    )
    return baseline, parity


def time_sft_steps(case, iters: int):
    """The supervised loss on the same logits: fused (one pass, 4 V bytes per token) against the log-prob op followed
    by the loss on log-probs (forward pass + backward pass, 6 V bytes per token)."""
    import torch

    import areal_amd

    T = case.logits.shape[0]

    def fused():
        x = case.logits.detach().requires_grad_(True)
        loss, _ = areal_amd.fused_logprobs_sft_loss(x, case.labels, case.loss_mask, case.cu_seqlens, case.temperature)
        loss.backward()

    def two_pass():
        x = case.logits.detach().requires_grad_(True)
        logp = areal_amd.gather_logprobs(x, case.labels, case.temperature)
        loss, _ = areal_amd.sft_loss_fn(logp, case.loss_mask, case.cu_seqlens)
        loss.backward()

    out = {}
    for name, fn in (("fused", fused), ("two_pass", two_pass)):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / iters * 1e3
        out[name] = dict(ms_per_step=ms, tokens_per_s=T / (ms * 1e-3))
    return out


def time_copy_kernel(src, dst, iters: int):
    """The plain copy kernel (aa_copy_bytes: 16 bytes per lane, nothing else) from ``src`` to ``dst``: what this chip
    delivers for a read-once / write-once stream over buffers of this very size."""
    import torch

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    nbytes = src.numel() * src.element_size()
    stream = torch.cuda.current_stream(src.device)
    st = C.c_void_p(stream.cuda_stream)
    ms, ms_min = time_events(lambda: N.check(lib.aa_copy_bytes(F._ptr(src), F._ptr(dst), nbytes, st), "aa_copy_bytes"),
                             iters, stream)
    gbs = 2.0 * nbytes / (ms * 1e-3) / 1e9
    return dict(kernel="k_copy16 (aa_copy_bytes)", bytes_read=nbytes, bytes_written=nbytes, avg_kernel_ms=ms,
                min_kernel_ms=ms_min, achieved=gbs, unit="GB/s", frac=gbs / HBM_PEAK_GBS)


def bench_logits(args, dev, workload: str, steps: int, warmup: int, cpu_tokens: int, with_sft: bool = True):
    """GPU part of a logits workload.  Returns the result line and the sample for the CPU phase (None: no CPU phase)."""
    import torch

    case, desc = build_logits_case(workload, args.seed, dev, getattr(args, "vocab", None) if workload == "cfg1-32k" else None)
    kw, cfg = ppo_kwargs(case)
    T, V = case.logits.shape
    f32 = args.logits_dtype == "f32"
    if f32:
        case.logits = case.logits.float()
        desc += "; logits cast to fp32"
    case.logits.requires_grad_(True)
    run_logits_steps(case, warmup, kw, cfg)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loss = run_logits_steps(case, steps, kw, cfg)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    assert bool(torch.isfinite(loss)), "loss is not finite"

    case.logits.grad = None
    case.logits.requires_grad_(False)
    k_ms, k_min_ms = time_fused_logits_kernel(case, kw, cfg, max(steps, 10))
    alg_bytes = (8.0 if f32 else 4.0) * T * V
    achieved = alg_bytes / (k_ms * 1e-3) / 1e9
    roofline = dict(
        bound="hbm", kernel=("k_fused_f32_hold" if f32 else "k_fused_regs") + " (aa_logits_ppo_fused)",
        achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS,
        # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters read
        # for the plain copy kernel: 1.002 x the algorithmic bytes (profiles/k_fused_regs_cfg1-32k_hbm_traffic.md);
        # fp32 logits: 1.001 x (profiles/k_fused_f32_hold_cfg1-32k_hbm_traffic.md)
        traffic=alg_bytes * (1.001 if f32 else 1.002), avg_kernel_ms=k_ms, min_kernel_ms=k_min_ms,
        traffic_source=("profiles/k_fused_f32_hold_cfg1-32k_hbm_traffic.md" if f32 else
                        "profiles/k_fused_regs_cfg1-32k_hbm_traffic.md") +
                       ": counter bytes / algorithmic bytes measured on the cfg1-32k workload, applied to this one's "
                       "algorithmic bytes (not a reading of this run)",
        algorithmic_bytes_per_launch=alg_bytes,
    )
    out = dict(
        metric=METRIC, value=T / (ms_per_step * 1e-3), unit="tokens/s",
        n_gpus=1, steps=steps, warmup=warmup, ms_per_step=ms_per_step, higher_is_better=True,
        scaling="weak", vs_baseline=None, dtype="f32" if f32 else "bf16", data="synthetic",
        config=dict(workload=f"{case.name}: {desc}", tokens=T, vocab=V, sequences=int(case.cu_seqlens.numel() - 1),
                    accumulate="f32", path="logits (fused fwd + PPO loss + bwd, one launch)"),
        roofline=roofline,
    )
    if cfg is not None:
        out["config"]["importance_weight_cap"] = f"{cfg.level} {cfg.metric} <= {cfg.upper}, action={cfg.action}"
    if with_sft:
        out["sft_loss_same_logits"] = time_sft_steps(case, max(steps // 2, 3))
    # the forward-only op on the same logits (compute_logp: log-probs of a reference or proximal policy): one read
    out["forward_only_logprobs"] = time_forward_only(case, max(steps, 10))
    # the measured ceiling of a read-once / write-once kernel on buffers of this size
    dst = torch.empty_like(case.logits)
    out["copy_same_buffers"] = time_copy_kernel(case.logits, dst, max(steps, 10))
    out["roofline"]["frac_of_copy_kernel"] = achieved / out["copy_same_buffers"]["achieved"]
    if args.copy_launches > 0:
        from areal_amd import _native as N
        from areal_amd import functional as F

        nbytes = case.logits.numel() * case.logits.element_size()
        for _ in range(args.copy_launches):
            N.check(N.load().aa_copy_bytes(F._ptr(case.logits), F._ptr(dst), nbytes, F._stream(dev)), "aa_copy_bytes")
        torch.cuda.synchronize()
        out["copy_calibration"] = dict(kernel="k_copy16 (aa_copy_bytes)", bytes_read=nbytes, bytes_written=nbytes,
                                       launches=args.copy_launches)
    del dst
    sample = logits_gpu_sample(case, kw, cfg, cpu_tokens) if cpu_tokens > 0 else None
    # last, because it overwrites the workload: the same kernel with the gradient written over the logits
    # (inplace_backward=True: one [T, V] array instead of two)
    i_ms, i_min_ms = time_fused_logits_kernel(case, kw, cfg, max(steps, 10), inplace=True)
    out["gradient_over_logits"] = dict(
        avg_kernel_ms=i_ms, min_kernel_ms=i_min_ms, achieved=alg_bytes / (i_ms * 1e-3) / 1e9, unit="GB/s",
        frac=alg_bytes / (i_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        bytes_of_logits_and_gradient=case.logits.numel() * case.logits.element_size(),
        note="inplace_backward=True; after the first launch the rows hold gradients, the traffic is the same")
    return out, sample


def time_forward_only(case, iters: int):
    """aa_logits_fwd (k_logits_fwd) on the workload's logits: log-probs alone (what ``gather_logprobs`` asks for), and
    with entropy and the vocabulary extrema.  Algorithmic bytes: every logit read once."""
    import torch

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    dev = case.logits.device
    T, V = case.logits.shape
    f32 = dict(dtype=torch.float32, device=dev)
    logp, ent, vmax, vmin = (torch.empty(T, **f32) for _ in range(4))
    stream = torch.cuda.current_stream(dev)
    st = C.c_void_p(stream.cuda_stream)
    nbytes = float(case.logits.numel() * case.logits.element_size())
    out = dict(kernel="k_logits_fwd (aa_logits_fwd)", algorithmic_bytes_per_launch=nbytes)
    for name, extra in (("logprobs_only", (None, None, None, None, None)),
                        ("with_entropy_and_extrema", (F._ptr(ent), None, None, F._ptr(vmax), F._ptr(vmin)))):
        def launch():
            N.check(lib.aa_logits_fwd(F._ptr(case.logits), F._DTYPES[case.logits.dtype], T, V, V, F._ptr(case.labels),
                                      1.0 / case.temperature, F._ptr(logp), *extra, st), "aa_logits_fwd")
        ms, ms_min = time_events(launch, iters, stream)
        out[name] = dict(avg_kernel_ms=ms, min_kernel_ms=ms_min, achieved=nbytes / (ms * 1e-3) / 1e9, unit="GB/s",
                         frac=nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, tokens_per_s=T / (ms * 1e-3))
    return out


def finish_with_cpu_phase(out, sample, cpu_phase, iters: int):
    if sample is not None:
        out["cpu_baseline"], out["parity"] = cpu_phase(sample, iters)
    return out


# ----------------------------------------------------------------------------------------------------------------
# fused lm_head path
# ----------------------------------------------------------------------------------------------------------------
def build_fused_case(name: str, seed: int, device):
    import torch

    import areal_amd
    from areal_amd import synth

    if name == "cfg2":
        case = synth.config2(device, seed)
        desc = "configs[2]: hidden [16384,4096], W [151936,4096], masks as configs[0], eps_clip=0.2"
    elif name == "cfg3":
        case = synth.config3(device, seed)
        desc = ("configs[3]: 8 packed seqs of 32768 tokens, hidden [262144,4096], W [151936,4096], alternating "
                "512-token mask, dual clip c=3, importance-weight cap 5, eps_clip 0.2 / 0.28")
    else:
        case = synth.config4(device, seed)
        desc = "configs[4]: hidden [32768,5376], W [262144,5376], temperature 0.7, 20% argmax labels"
    with torch.no_grad():
        ref, _ = areal_amd.lm_head_logprobs_entropy(case.hidden, case.weight, case.labels, case.temperature)
    synth.attach_old_and_prox(case, ref, 0.05, seed + 9)
    return case, desc


DENSE_BACKWARD = False  # set from --dense-backward
BACKWARD_MODE = 1  # aa_lmhead_backward_mode: 1 carry, 0 recompute (set from --lmhead-backward)
NO_FORWARD_OF_MASKED = False  # set from --no-forward-of-masked
MODE_NAMES = {1: "carry", 0: "recompute"}

# HBM bytes per step of aa_lmhead_ppo_fused, all its kernels together: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (one
# run each) summed over the kernels of one step, each scaled by what the same counter reads for the plain copy kernel of
# known size.  The counters sit behind the L2 of each XCD: what the memory-side cache serves is in these figures too.
# Transcribed from the profile summaries named beside them, not read in this run; other workloads: not measured.
LMHEAD_MEASURED_HBM_BYTES = {
    ("cfg2", "carry"): (81.7e9, "profiles/lmhead_step_cfg2_hbm_traffic.md"),
    ("cfg2", "recompute"): (111.1e9, "profiles/lmhead_step_cfg2_hbm_traffic.md"),
    ("cfg4", "carry"): (515.3e9, "profiles/lmhead_step_cfg4_hbm_traffic.md"),
}


def lmhead_measured_bytes(workload: str, mode: str):
    return LMHEAD_MEASURED_HBM_BYTES.get((workload, mode), (None, None))


def time_mfma_only_loop(dev, reps: int = 4, target_ms: float = 40.0):
    """The MFMA-only loop (aa_mfma_only_loop) in both instruction forms, on random and on zero operands: TFLOP/s of
    launches of about ``target_ms`` each, HIP events on the launch stream, one workgroup per compute unit."""
    import torch

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    wgs = torch.cuda.get_device_properties(dev).multi_processor_count
    out = torch.empty(wgs * 256, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev)
    st = C.c_void_p(stream.cuda_stream)
    res = {}
    for form, name, flops_per_iter in ((0, "v_mfma_f32_32x32x16_bf16", 2097152.0), (1, "v_mfma_f32_16x16x32_bf16", 4194304.0)):
        for random_operands in (1, 0):
            # iterations for the target duration at 2 PFLOP/s
            iters = int(target_ms * 1e-3 * 2.0e15 / (wgs * flops_per_iter))

            def launch():
                N.check(lib.aa_mfma_only_loop(form, random_operands, wgs, iters, F._ptr(out), st), "aa_mfma_only_loop")

            avg_ms, min_ms = time_events(launch, reps, stream)
            res[f"{name}, {'random' if random_operands else 'zero'} operands"] = dict(
                avg_ms=avg_ms, min_ms=min_ms, workgroups=wgs, iterations=iters,
                tflops=wgs * flops_per_iter * iters / (avg_ms * 1e-3) / 1e12)
    res["best_on_random_operands_tflops"] = max(v["tflops"] for k, v in res.items() if k.endswith("random operands"))
    return res


def lmhead_compulsory_bytes(T: int, kept: int, H: int, V: int, mode: str, chunk: int) -> dict:
    """HBM bytes a step cannot avoid, kernel by kernel: every operand of a kernel read once, every result written
    once (bf16 = 2 bytes).  ``kept`` = tokens with a gradient.  What the counters read above this is re-fetching."""
    n_chunks = -(-T // chunk)
    blocks = 2 * -(-V // 256)
    w_bytes = 2.0 * V * H
    partials = 12.0 * blocks * T
    panel = 2.0 * kept * V
    out = dict(
        forward_tiles=n_chunks * w_bytes + 2.0 * T * H + partials + (panel if mode == "carry" else 0.0),
        merge_partials=partials,
        recompute_tiles=(n_chunks * w_bytes + 2.0 * kept * H + panel) if mode == "recompute" else 0.0,
        d_hidden_gemm=panel + n_chunks * w_bytes + 2.0 * kept * H,
        # d_weight: written once in bf16 when one chunk holds every token, else accumulated in fp32 chunk by chunk
        d_weight_gemm=panel + 2.0 * kept * H + (w_bytes if n_chunks == 1 else (2 * n_chunks - 1) * 2.0 * w_bytes + 3.0 * w_bytes),
    )
    out["total"] = sum(out.values())
    out["logits_panel_written"] = panel
    return out


def run_fused_steps(case, n, kw, cfg, events=None):
    """``n`` steps; with ``events`` (a list) a pair of HIP events on the launch stream brackets every step."""
    import torch

    import areal_amd

    h, w = case.hidden, case.weight
    stream = torch.cuda.current_stream(h.device)
    loss = None
    for _ in range(n):
        h.grad = None
        w.grad = None
        if events is not None:
            ev = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            ev[0].record(stream)
        loss, _ = areal_amd.fused_lm_head_ppo_loss(
            h, w, case.labels, case.prox_logp, case.old_logp, case.advantages, loss_mask=case.loss_mask,
            rejection_sampling=cfg, cu_seqlens=case.cu_seqlens, temperature=case.temperature,
            skip_masked_tokens=not DENSE_BACKWARD, forward_masked_tokens=not NO_FORWARD_OF_MASKED,
            backward=MODE_NAMES[BACKWARD_MODE], **kw,
        )
        loss.backward()
        if events is not None:
            ev[1].record(stream)
            events.append(ev)
    return loss


def time_lmhead_step(case, kw, cfg, iters: int, skip_masked: bool, mode: int):
    """Duration of aa_lmhead_ppo_fused (every kernel it enqueues) called through the C ABI with pre-allocated outputs,
    HIP events on the launch stream, and the number of tokens that go through the gradient GEMMs."""
    import torch

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    dev = case.hidden.device
    T, H = case.hidden.shape
    V = case.weight.shape[0]
    f32 = dict(dtype=torch.float32, device=dev)
    m8 = F._mask_u8(case.loss_mask)
    prox, old, adv = (F._f32(t) for t in (case.prox_logp, case.old_logp, case.advantages))
    params = F._ppo_params(kw["eps_clip"], kw.get("eps_clip_higher"), kw.get("c_clip"), cfg is not None)
    if cfg is not None:
        mask_eff, w, counts = F._rejection_sampling_device(prox, old, m8, m8.shape, case.cu_seqlens, cfg)
        if cfg.action != "mask":
            mask_eff = m8
    else:
        mask_eff, w, counts = m8, None, F._count_nonzero(m8)
    logp, ent, sl, ratio, vmax, vmin = (torch.empty(T, **f32) for _ in range(6))
    flags = torch.empty(T, dtype=torch.uint8, device=dev)
    dh = torch.empty_like(case.hidden)
    dw = torch.empty_like(case.weight)  # bf16, as the Python wrapper asks for
    ws = F._lmhead_workspace(T, H, V, dev)
    stream = torch.cuda.current_stream(dev)
    kept, kept_tokens = None, T
    if skip_masked:  # per-chunk counts of tokens with a mask, read once here (the Python wrapper reads them per step)
        chunk = int(lib.aa_lmhead_chunk_tokens())
        per_chunk = [int(mask_eff[i:i + chunk].ne(0).sum()) for i in range(0, T, chunk)]
        kept, kept_tokens = (C.c_int64 * len(per_chunk))(*per_chunk), sum(per_chunk)

    def launch():
        N.check(
            lib.aa_lmhead_ppo_fused(
                F._ptr(case.hidden), F._ptr(case.weight), T, H, V, F._ptr(case.labels), 1.0 / case.temperature, T,
                F._ptr(prox), F._ptr(adv), F._ptr(mask_eff), F._ptr(w), C.byref(params), F._ptr(counts), None, kept,
                mode, F._ptr(logp), F._ptr(ent), F._ptr(sl), F._ptr(ratio), F._ptr(flags), F._ptr(vmax), F._ptr(vmin),
                F._ptr(dh), F._ptr(dw), N.AA_BF16, F._ptr(ws), ws.numel(), C.c_void_p(stream.cuda_stream),
            ),
            "aa_lmhead_ppo_fused",
        )

    return time_events(launch, iters, stream) + (kept_tokens,)


def time_lmhead_op(case, iters: int):
    """Durations of aa_lmhead_fwd and aa_lmhead_bwd, the stand-alone differentiable op (its backward forms the
    logits of the tokens with a gradient again), HIP events on the launch stream."""
    import torch

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    dev = case.hidden.device
    T, H = case.hidden.shape
    V = case.weight.shape[0]
    f32 = dict(dtype=torch.float32, device=dev)
    logp, ent, lse, ez = (torch.empty(T, **f32) for _ in range(4))
    ws = F._lmhead_workspace(T, H, V, dev)
    g = torch.randn(T, **f32) * case.loss_mask.float() / T
    dh = torch.empty_like(case.hidden)
    dw = torch.empty_like(case.weight)  # bf16, as the Python wrapper asks for
    stream = torch.cuda.current_stream(dev)
    st = C.c_void_p(stream.cuda_stream)
    inv_t = 1.0 / case.temperature

    def fwd():
        N.check(lib.aa_lmhead_fwd(F._ptr(case.hidden), F._ptr(case.weight), T, H, V, F._ptr(case.labels), inv_t,
                                  F._ptr(logp), F._ptr(ent), F._ptr(lse), F._ptr(ez), None, None, F._ptr(ws), ws.numel(), st),
                "aa_lmhead_fwd")

    has_grad, kept, kept_tokens = None, None, T
    if not DENSE_BACKWARD:  # rows with a zero upstream gradient stay out of the gradient GEMMs
        has_grad = (g != 0).view(torch.uint8)
        chunk = int(lib.aa_lmhead_chunk_tokens())
        per_chunk = [int(has_grad[i:i + chunk].ne(0).sum()) for i in range(0, T, chunk)]
        kept, kept_tokens = (C.c_int64 * len(per_chunk))(*per_chunk), sum(per_chunk)

    def bwd():
        N.check(lib.aa_lmhead_bwd(F._ptr(case.hidden), F._ptr(case.weight), T, H, V, F._ptr(case.labels), inv_t,
                                  F._ptr(lse), F._ptr(ez), F._ptr(g), None, F._ptr(has_grad), kept, F._ptr(dh), F._ptr(dw),
                                  N.AA_BF16, F._ptr(ws), ws.numel(), st), "aa_lmhead_bwd")

    f_ms, _ = time_events(fwd, iters, stream)
    b_ms, _ = time_events(bwd, iters, stream)
    # the same op in carry form: the forward keeps p_v / p_label of the tokens with a gradient, the backward is two GEMMs
    rows = kept_tokens if has_grad is not None else T
    panel = torch.empty(rows, int(lib.aa_lmhead_panel_pitch(V)), dtype=torch.bfloat16, device=dev)
    ws_c = torch.empty(lib.aa_lmhead_carry_workspace_bytes(T, H, V), dtype=torch.uint8, device=dev)

    def fwd_carry():
        N.check(lib.aa_lmhead_fwd_carry(F._ptr(case.hidden), F._ptr(case.weight), T, H, V, F._ptr(case.labels), inv_t,
                                        F._ptr(has_grad), kept, F._ptr(logp), F._ptr(ent), F._ptr(lse), F._ptr(ez), None, None,
                                        F._ptr(panel), rows, F._ptr(ws_c), ws_c.numel(), st), "aa_lmhead_fwd_carry")

    def bwd_carry():
        N.check(lib.aa_lmhead_bwd_carry(F._ptr(case.hidden), F._ptr(case.weight), T, H, V, F._ptr(case.labels), inv_t,
                                        F._ptr(logp), F._ptr(lse), F._ptr(g), F._ptr(has_grad), kept, F._ptr(panel), rows,
                                        F._ptr(dh), F._ptr(dw), N.AA_BF16, F._ptr(ws_c), ws_c.numel(), st), "aa_lmhead_bwd_carry")

    def both_carry():  # the backward patches the stored rows: every timed backward follows a forward of its own
        fwd_carry()
        bwd_carry()

    fc_ms, _ = time_events(fwd_carry, iters, stream)
    pair_ms, _ = time_events(both_carry, iters, stream)
    return f_ms, b_ms, kept_tokens, fc_ms, pair_ms - fc_ms


def fused_gpu_sample(case, kw, cfg, n_tokens: int):
    """The GPU step on the sample tokens (see sample_windows) against the full weight matrix, with everything the CPU
    phase needs copied to the host."""
    import torch

    import areal_amd

    idx, desc = sample_windows(case.n_tokens, n_tokens)
    n = int(idx.numel())
    idx_d = idx.to(case.hidden.device)
    take = lambda t: t[idx_d]
    cu = torch.tensor([0, n], dtype=torch.int32)
    h = take(case.hidden).detach().clone().requires_grad_(True)
    w = case.weight.detach().clone().requires_grad_(True)
    loss, stat = areal_amd.fused_lm_head_ppo_loss(
        h, w, take(case.labels), take(case.prox_logp), take(case.old_logp), take(case.advantages),
        loss_mask=take(case.loss_mask), rejection_sampling=cfg, cu_seqlens=cu.to(h.device),
        temperature=case.temperature, backward=MODE_NAMES[BACKWARD_MODE], **kw)
    loss.backward()
    torch.cuda.synchronize()
    cpu = lambda t: take(t).cpu()
    return dict(
        n=n, windows=desc, cu=cu, kw=kw, cfg=cfg, temperature=case.temperature,
        hidden=h.detach().cpu().float(), weight=case.weight.cpu().float(), labels=cpu(case.labels),
        prox=cpu(case.prox_logp), old=cpu(case.old_logp), adv=cpu(case.advantages), mask=cpu(case.loss_mask),
        gpu=dict(loss=float(loss.detach()), logprobs=stat["logprobs"].detach().cpu(), d_hidden=h.grad.cpu(),
                 d_weight=w.grad.cpu()),
    )


def fused_cpu_phase(sample, iters: int):
    """Oracle (fp32 matmul + logits path + PPO loss + autograd) on the sample tokens against the full weight matrix
    (host cores), and the GPU results of fused_gpu_sample checked against it."""
    import torch

    import oracle

    n, g = sample["n"], sample["gpu"]
    threads = torch.get_num_threads()

    def oracle_step():
        h = sample["hidden"].clone().requires_grad_(True)
        w = sample["weight"].clone().requires_grad_(True)
        logits = oracle.lmhead_logits(h, w)
        lp, _ent = oracle.logprobs_entropy(logits, sample["labels"], sample["temperature"])
        loss, _stat = oracle.ppo_actor_loss(lp, sample["prox"], sample["old"], sample["adv"], loss_mask=sample["mask"].bool(),
                                            rejection_sampling_cfg=sample["cfg"], cu_seqlens=sample["cu"], **sample["kw"])
        loss.backward()
        return loss.detach(), lp.detach(), h.grad, w.grad

    oracle_step()
    t0 = time.perf_counter()
    for _ in range(iters):
        w_loss, w_lp, w_dh, w_dw = oracle_step()
    dt = (time.perf_counter() - t0) / iters
    parity = dict(
        tokens=n, token_windows=sample["windows"], tokens_with_mask=int(sample["mask"].sum()),
        logp_max_abs_err=float((g["logprobs"] - w_lp).abs().max()),
        loss_rel_err=abs(g["loss"] - float(w_loss)) / max(abs(float(w_loss)), 1e-12),
        d_hidden_cosine=cosine(g["d_hidden"], w_dh), d_weight_cosine=cosine(g["d_weight"], w_dw),
        d_hidden_norm_ratio=float(g["d_hidden"].double().norm() / w_dh.double().norm()),
        d_weight_norm_ratio=float(g["d_weight"].double().norm() / w_dw.double().norm()),
    )
    baseline = dict(
        value=n / dt, unit="tokens/s", cores=threads, kind="port",
        sample=f"{n} tokens of the workload (tokens {sample['windows']}) against the full weight matrix, {iters} timed "
               f"fwd+bwd passes of the PyTorch CPU oracle (fp32 hidden @ W.T, log_softmax + gather + entropy, PPO loss, "
               f"autograd to d(hidden) and d(W))",
    )
    return baseline, parity


def bench_fused(args, dev, workload: str, steps: int, warmup: int, cpu_tokens: int):
    """GPU part of a fused lm_head workload.  Returns the result line and the sample for the CPU phase."""
    import torch

    from areal_amd import _native as N

    case, desc = build_fused_case(workload, args.seed, dev)
    kw, cfg = ppo_kwargs(case)
    T, H = case.hidden.shape
    V = case.weight.shape[0]
    case.hidden.requires_grad_(True)
    case.weight.requires_grad_(True)
    run_fused_steps(case, warmup, kw, cfg)
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    loss = run_fused_steps(case, steps, kw, cfg, events)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    assert bool(torch.isfinite(loss)), "loss is not finite"
    ev_ms = sorted(a.elapsed_time(b) for a, b in events)
    ev_avg = sum(ev_ms) / len(ev_ms)
    case.hidden.grad = None
    case.weight.grad = None
    case.hidden.requires_grad_(False)
    case.weight.requires_grad_(False)

    # the same step through the C ABI alone (outputs pre-allocated, no autograd), in both backward modes
    mode_name = MODE_NAMES[BACKWARD_MODE]
    chunk = int(N.load().aa_lmhead_chunk_tokens())
    modes = {}
    kept_tokens = T
    for mode, name in ((1, "carry"), (0, "recompute")):
        if args.steps_only and mode != BACKWARD_MODE:
            continue
        c_ms, c_min, kept_tokens = time_lmhead_step(case, kw, cfg, 2 if args.steps_only else 10, not args.dense_backward,
                                                    mode)
        modes[name] = dict(avg_call_ms=c_ms, min_call_ms=c_min,
                           executed_flops=(2.0 * T + (4.0 if mode == 1 else 6.0) * kept_tokens) * V * H,
                           compulsory_hbm_bytes=lmhead_compulsory_bytes(T, kept_tokens, H, V, name, chunk),
                           measured_hbm_bytes=lmhead_measured_bytes(workload, name)[0],
                           measured_hbm_bytes_source=lmhead_measured_bytes(workload, name)[1])
    standalone = None
    if not args.steps_only:
        # the stand-alone differentiable op lm_head_logprobs_entropy: its forward writes softmax partials only, its
        # backward forms the logits of the tokens with a gradient again (6 T_grad V H flops executed)
        f_ms, b_ms, op_kept, fc_ms, bc_ms = time_lmhead_op(case, 5)
        standalone = dict(fwd_ms=f_ms, bwd_ms=b_ms, fwd_tflops=2.0 * T * V * H / (f_ms * 1e-3) / 1e12,
                          bwd_executed_tflops=6.0 * op_kept * V * H / (b_ms * 1e-3) / 1e12,
                          # lm_head_logprobs_entropy(backward="carry"): the forward also keeps the bf16 rows of the
                          # tokens with a gradient, the backward is the two gradient GEMMs (4 T_grad V H flops)
                          carry_fwd_ms=fc_ms, carry_bwd_ms=bc_ms,
                          carry_bwd_tflops=4.0 * op_kept * V * H / (bc_ms * 1e-3) / 1e12)
    # Flops the step needs: logits of every token (2 T V H) and the two gradient GEMMs over the tokens that have a
    # gradient (4 T_kept V H).  The reference's autograd runs them over all T tokens: 6 T V H.
    needed_flops = 2.0 * T * V * H + 4.0 * kept_tokens * V * H
    achieved = needed_flops / (ev_avg * 1e-3) / 1e12
    roofline = dict(
        bound="mfma",
        kernel="every kernel of one fused_lm_head_ppo_loss(...) + backward() step: k_lmhead_tiles (logits tiles on the "
               "library's bf16 MFMA tile GEMM, softmax partials per tile, " +
               ("p_v / p_label of the tokens with a gradient kept in bf16" if mode_name == "carry"
                else "nothing else written") +
               "), k_label_logit, k_token_loss, " +
               ("" if mode_name == "carry" else "k_lmhead_tiles again for the tokens with a gradient, ") +
               "k_gemm_store twice (d_hidden, d_weight; in carry mode they apply the per-token gradient factor)",
        achieved=achieved, peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s", frac=achieved / MFMA_BF16_PEAK_TFLOPS,
        traffic=lmhead_measured_bytes(workload, mode_name)[0],
        traffic_source=lmhead_measured_bytes(workload, mode_name)[1],
        timed="HIP events on the launch stream around each of the steps that ms_per_step is the wall-clock mean of",
        avg_step_ms=ev_avg, min_step_ms=ev_ms[0], max_step_ms=ev_ms[-1],
        needed_flops_per_step=needed_flops, flops_per_step_6TVH=6.0 * T * V * H, tokens_with_gradient=kept_tokens,
        backward_mode=mode_name, backward_modes_through_c_abi=modes,
        standalone_op=standalone,
    )
    # the measured ceiling of the matrix cores in this process: a loop of MFMAs only (no LDS, no memory traffic)
    mfma_only = time_mfma_only_loop(dev)
    roofline["mfma_only_loop"] = mfma_only
    roofline["frac_of_mfma_only_loop"] = achieved / mfma_only["best_on_random_operands_tflops"]
    out = dict(
        metric=METRIC, value=T / (ms_per_step * 1e-3), unit="tokens/s",
        n_gpus=1, steps=steps, warmup=warmup, ms_per_step=ms_per_step, higher_is_better=True,
        scaling="weak", vs_baseline=None, dtype="bf16", data="synthetic",
        config=dict(workload=f"{case.name}: {desc}", tokens=T, hidden=H, vocab=V,
                    sequences=int(case.cu_seqlens.numel() - 1), accumulate="f32",
                    path=f"lm_head + PPO loss step, fwd + bwd (backward={mode_name}); the forward writes no logits"),
        roofline=roofline,
    )
    if NO_FORWARD_OF_MASKED:
        out["config"]["path"] += "; NOT the reference's semantics: masked tokens skip the lm_head"
    if args.copy_launches > 0:  # calibration point of the FETCH_SIZE / WRITE_SIZE counters: a copy of the weight matrix
        from areal_amd import functional as F

        dst = torch.empty_like(case.weight)
        nbytes = case.weight.numel() * case.weight.element_size()
        for _ in range(args.copy_launches):
            N.check(N.load().aa_copy_bytes(F._ptr(case.weight), F._ptr(dst), nbytes, F._stream(dev)), "aa_copy_bytes")
        torch.cuda.synchronize()
        out["copy_calibration"] = dict(kernel="k_copy16 (aa_copy_bytes)", bytes_read=nbytes, bytes_written=nbytes,
                                       launches=args.copy_launches)
    sample = fused_gpu_sample(case, kw, cfg, cpu_tokens) if cpu_tokens > 0 else None
    return out, sample

def bench_fused_leg(args, dev, workload: str, steps: int, warmup: int):
    """A fused lm_head workload, GPU only: ``warmup`` + ``steps`` steps of fused_lm_head_ppo_loss + backward through the
    Python API, HIP events on the launch stream around every timed step, roofline on the flops the step needs."""
    import torch

    case, desc = build_fused_case(workload, args.seed, dev)
    kw, cfg = ppo_kwargs(case)
    T, H = case.hidden.shape
    V = case.weight.shape[0]
    case.hidden.requires_grad_(True)
    case.weight.requires_grad_(True)
    run_fused_steps(case, warmup, kw, cfg)
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    loss = run_fused_steps(case, steps, kw, cfg, events)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    assert bool(torch.isfinite(loss)), "loss is not finite"
    assert bool(torch.isfinite(case.hidden.grad.float()).all()) and bool(torch.isfinite(case.weight.grad.float()).all())
    ev_ms = sorted(a.elapsed_time(b) for a, b in events)
    ev_avg = sum(ev_ms) / len(ev_ms)
    with torch.no_grad():
        from areal_amd import functional as F

        m8 = F._mask_u8(case.loss_mask)
        if cfg is not None and cfg.action == "mask":
            prox, old = F._f32(case.prox_logp), F._f32(case.old_logp)
            m8, _, _ = F._rejection_sampling_device(prox, old, m8, m8.shape, case.cu_seqlens, cfg)
        kept_tokens = int(m8.ne(0).sum()) if not DENSE_BACKWARD else T
    needed_flops = 2.0 * T * V * H + 4.0 * kept_tokens * V * H
    achieved = needed_flops / (ev_avg * 1e-3) / 1e12
    mode_name = MODE_NAMES[BACKWARD_MODE]
    return dict(
        value=T / (ms_per_step * 1e-3), unit="tokens/s", steps=steps, warmup=warmup, ms_per_step=ms_per_step,
        config=dict(workload=f"{case.name}: {desc}", tokens=T, hidden=H, vocab=V,
                    sequences=int(case.cu_seqlens.numel() - 1), accumulate="f32",
                    path=f"lm_head + PPO loss step, fwd + bwd (backward={mode_name}); the forward writes no logits"),
        roofline=dict(
            bound="mfma", kernel="every kernel of one fused_lm_head_ppo_loss(...) + backward() step",
            achieved=achieved, peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s", frac=achieved / MFMA_BF16_PEAK_TFLOPS,
            traffic=lmhead_measured_bytes(workload, mode_name)[0],
            traffic_source=lmhead_measured_bytes(workload, mode_name)[1],
            timed="HIP events on the launch stream around each of the timed steps",
            avg_step_ms=ev_avg, min_step_ms=ev_ms[0], max_step_ms=ev_ms[-1], needed_flops_per_step=needed_flops,
            flops_per_step_6TVH=6.0 * T * V * H, tokens_with_gradient=kept_tokens, backward_mode=mode_name),
    )


def bench_mfma(args, dev):
    res = time_mfma_only_loop(dev, reps=max(args.steps, 6), target_ms=50.0)
    best = res["best_on_random_operands_tflops"]
    return dict(
        metric="TFLOP/s of a loop of bf16 MFMAs only (no LDS, no memory traffic): the measured matrix-core ceiling",
        value=best, unit="TFLOP/s", n_gpus=1, steps=max(args.steps, 6), warmup=2, higher_is_better=True, dtype="bf16",
        data="synthetic", vs_baseline=None, scaling="weak",
        config=dict(workload="aa_mfma_only_loop: 4 waves per workgroup, one workgroup per compute unit, operands in "
                             "registers"),
        roofline=dict(bound="mfma", kernel="k_mfma_16x16x32 / k_mfma_32x32x16", achieved=best,
                      peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s", frac=best / MFMA_BF16_PEAK_TFLOPS, traffic=0.0),
        forms=res,
    )


def bench_hbm(args, dev):
    """Plain streams over 20 GB (aa_hbm_stream_probe): read only, write only and copy, with the default and with the
    streaming cache policy.  The measured ceilings beside the HBM-bound kernels of the logits path."""
    import torch

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    nbytes = 20 << 30
    src = torch.full((nbytes,), 1, dtype=torch.uint8, device=dev)
    dst = torch.full((nbytes,), 2, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev)
    st = C.c_void_p(stream.cuda_stream)
    wgs = 8 * torch.cuda.get_device_properties(dev).multi_processor_count
    res = {}
    for kind, name, moved in ((0, "read", nbytes), (1, "write", nbytes), (2, "copy", 2 * nbytes)):
        for nt in (0, 1):
            def launch():
                N.check(lib.aa_hbm_stream_probe(kind, nt, F._ptr(src), F._ptr(dst), nbytes, wgs, st), "aa_hbm_stream_probe")
            ms, ms_min = time_events(launch, max(args.steps, 10), stream)
            res[f"{name}, {'nt' if nt else 'default'} policy"] = dict(avg_ms=ms, min_ms=ms_min, gb_per_s=moved / (ms * 1e-3) / 1e9,
                                                                      frac_of_peak=moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS)
    rd = max(res["read, nt policy"]["gb_per_s"], res["read, default policy"]["gb_per_s"])
    wr = max(res["write, nt policy"]["gb_per_s"], res["write, default policy"]["gb_per_s"])
    both = 2.0 / (1.0 / rd + 1.0 / wr)
    return dict(
        metric="GB/s of plain HBM streams (read only, write only, copy): the measured ceilings of the logits path",
        value=both, unit="GB/s", n_gpus=1, steps=max(args.steps, 10), warmup=5, higher_is_better=True, dtype="u8",
        data="synthetic", vs_baseline=None, scaling="weak",
        config=dict(workload="aa_hbm_stream_probe over 20 GiB buffers, 8 workgroups of 256 threads per compute unit, "
                             "32 KB pieces"),
        roofline=dict(bound="hbm", kernel="k_stream_read / k_stream_write", achieved=both, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=both / HBM_PEAK_GBS, traffic=None,
                      note="value = rate of a kernel that reads as many bytes as it writes if its reads ran at the read-only "
                           "rate and its writes at the write-only rate (harmonic mean of the two)"),
        streams=res,
    )


# ----------------------------------------------------------------------------------------------------------------
# advantage pipeline
# ----------------------------------------------------------------------------------------------------------------
def bench_adv(args, dev):
    import torch

    import areal_amd
    from areal_amd import NormConfig, Normalization
    from oracle import advantages as O

    bs, L = 512, 4096
    g = torch.Generator().manual_seed(args.seed)
    lens = torch.randint(L // 4, L + 1, (bs,), generator=g)
    pos = torch.arange(L)[None, :]
    mask = ((pos >= (lens[:, None] * 0.3).long()) & (pos < lens[:, None] - 1)).float()
    rewards = torch.zeros(bs, L)
    rewards[torch.arange(bs), (lens - 2).clamp(min=0)] = torch.randn(bs, generator=g)
    rewards = rewards - 0.01 * torch.rand(bs, L, generator=g) * mask
    values = torch.randn(bs, L, generator=g) * 0.1
    no_eos = lens == L
    d = [t.to(dev) for t in (rewards, values, mask, no_eos)]
    norm = Normalization(NormConfig(mean_level="batch", std_level="batch"))

    def step():
        adv, ret = areal_amd.gae_advantages(d[0], d[1], d[2], d[3], 1.0, 0.95)
        return norm(adv, d[2]), ret

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out, ret = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    adv = torch.empty_like(d[0])
    ret = torch.empty_like(d[0])
    ne8 = F._mask_u8(d[3])
    stream = torch.cuda.current_stream(dev)

    def launch():
        N.check(lib.aa_gae(F._ptr(d[0]), F._ptr(d[1]), F._ptr(d[2]), F._ptr(ne8), bs, L, 1.0, 0.95, F._ptr(adv),
                           F._ptr(ret), C.c_void_p(stream.cuda_stream)), "aa_gae")

    k_ms, k_min = time_events(launch, max(args.steps, 10), stream)
    alg_bytes = 20.0 * bs * L
    achieved = alg_bytes / (k_ms * 1e-3) / 1e9
    t0 = time.perf_counter()
    w_adv, _ = O.gae(rewards, values, mask, no_eos.float(), 1.0, 0.95)
    w_out = O.normalization(w_adv, mask)
    cpu_s = time.perf_counter() - t0
    # masked_normalization of the same batch over all axes: 12 bytes per value read twice + 4 written
    mn_ms, _ = time_events(lambda: areal_amd.masked_normalization(d[0], d[2]), max(args.steps, 10), stream)
    mn_err = float((areal_amd.masked_normalization(d[0], d[2]).cpu() - O.masked_normalization(rewards, mask)).abs().max())
    return dict(
        metric="tokens/sec for GAE + advantage normalisation", value=bs * L / (ms_per_step * 1e-3), unit="tokens/s",
        n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms_per_step, higher_is_better=True,
        scaling="weak", vs_baseline=None, dtype="f32", data="synthetic",
        config=dict(workload="adv: padded batch [512, 4096], one terminal reward per sequence plus KL penalties, "
                             "critic values, gamma 1, lambda 0.95, batch-level mean / std normalisation",
                    sequences=bs, max_seqlen=L),
        roofline=dict(bound="hbm", kernel="k_gae (aa_gae)", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=achieved / HBM_PEAK_GBS, traffic=None, avg_kernel_ms=k_ms, min_kernel_ms=k_min,
                      algorithmic_bytes_per_launch=alg_bytes),
        cpu_baseline=dict(value=bs * L / cpu_s, unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                          sample="the whole workload once: the reference's Python loop over max_seqlen (4095 steps "
                                 "of [512]-wide tensor ops) and Normalization, restated in the CPU oracle"),
        masked_normalization_ms=mn_ms,
        parity=dict(adv_max_abs_err=float((out.cpu() - w_out).abs().max()),
                    returns_max_abs_err=float((ret.cpu() - (w_adv + values)).abs().max()),
                    masked_normalization_max_abs_err=mn_err),
    )

def bench_aux(args, dev):
    import torch

    import areal_amd
    from oracle import packing as OP
    from oracle import siblings as OS

    g = torch.Generator().manual_seed(args.seed)
    T = 122433
    lp = -torch.rand(T, generator=g) * 3
    old = lp + 0.05 * torch.randn(T, generator=g)
    prox = lp + 0.05 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < 0.7
    ver = torch.randint(-1, 6, (T,), generator=g)
    val, tgt = torch.randn(T, generator=g), torch.randn(T, generator=g)
    d = {k: v.to(dev) for k, v in dict(lp=lp, old=old, prox=prox, adv=adv, mask=mask, ver=ver, val=val, tgt=tgt).items()}
    stream = torch.cuda.current_stream(dev)

    def sapo():
        x = d["lp"].detach().requires_grad_(True)
        loss, _ = areal_amd.sapo_loss_fn(x, d["old"], d["adv"], 1.0, 1.05, d["mask"])
        loss.backward()

    def critic():
        x = d["val"].detach().requires_grad_(True)
        loss, _ = areal_amd.ppo_critic_loss_fn(x, d["val"] * 0.9, d["tgt"], 0.2, d["mask"])
        loss.backward()

    # DPO: the same tokens as 32 interleaved (chosen, rejected) pairs of random lengths
    cuts = torch.sort(torch.randperm(T - 1, generator=g)[:63] + 1).values
    dpo_cu = torch.cat([torch.zeros(1, dtype=torch.long), cuts, torch.tensor([T])]).to(torch.int32)
    dpo_cu_d = dpo_cu.to(dev)

    def dpo():
        x = d["lp"].detach().requires_grad_(True)
        loss, _ = areal_amd.dpo_loss(x, d["old"], dpo_cu_d, d["mask"], beta=0.1)
        loss.backward()
        return x, loss

    pieces = dict(
        sapo_loss_fwd_bwd=sapo, critic_loss_fwd_bwd=critic, dpo_loss_fwd_bwd=dpo,
        m2po_masking=lambda: areal_amd.apply_m2po_masking(d["old"], d["prox"], d["mask"], 0.002),
        prox_logp_loglinear=lambda: areal_amd.compute_prox_logp_approximations(d["old"], d["lp"], d["ver"], 6, "loglinear"),
        logging_stats_metrics_mode=lambda: areal_amd.proximal_logging_stats(d["old"], d["lp"], d["prox"], d["ver"], 6,
                                                                            d["mask"], "metrics"),
    )
    out_pieces = {}
    for name, fn in pieces.items():
        ms, _ = time_events(fn, max(args.steps, 10), stream)
        out_pieces[name] = dict(ms=ms, tokens_per_s=T / (ms * 1e-3))
    t0 = time.perf_counter()
    x = lp.clone().requires_grad_(True)
    w_loss, _ = OS.sapo_loss(x, old, adv, 1.0, 1.05, mask)
    w_loss.backward()
    OS.m2po_mask(old, prox, mask, 0.002)
    cpu_sib_s = time.perf_counter() - t0
    y = d["lp"].detach().requires_grad_(True)
    g_loss, _ = areal_amd.sapo_loss_fn(y, d["old"], d["adv"], 1.0, 1.05, d["mask"])
    g_loss.backward()
    m2_gpu = areal_amd.apply_m2po_masking(d["old"], d["prox"], d["mask"], 0.002).cpu()
    m2_cpu = OS.m2po_mask(old, prox, mask, 0.002)
    from oracle import dpo as OD

    xd = lp.clone().requires_grad_(True)
    t0 = time.perf_counter()
    wd_loss, _ = OD.compute_dpo_loss(xd, old, dpo_cu, mask, 0.1)
    wd_loss.backward()
    cpu_dpo_s = time.perf_counter() - t0
    yd, gd_loss = dpo()

    # packing: a padded batch, and the logits of an aligned + page-padded micro-batch
    bs, S, V = 512, 4096, 151936
    lens = torch.randint(S // 8, S + 1, (bs,), generator=g)
    am = (torch.arange(S)[None, :] < lens[:, None])
    batch = dict(attention_mask=am.to(dev), input_ids=torch.randint(0, V, (bs, S), generator=g).to(dev),
                 logprobs=torch.randn(bs, S, generator=g).to(dev), loss_mask=(torch.rand(bs, S, generator=g) < 0.5).to(dev))
    pack_ms, _ = time_events(lambda: areal_amd.pack_tensor_dict(batch), max(args.steps, 10), stream)
    mb_lens = synth_lengths(32768, args.seed)
    cu = torch.tensor([0] + list(torch.tensor(mb_lens).cumsum(0)), dtype=torch.int32)
    mb = dict(cu_seqlens=cu, max_seqlen=max(mb_lens), rows=torch.arange(int(cu[-1])))
    padded, pad_len, old_cu, _ = OP.pad_packed_tensor_dict(mb, int(cu[-1]), seq_align_to=64)
    T_pad = padded["rows"].shape[0]
    logits = torch.randn(T_pad, V, device=dev, dtype=torch.bfloat16)
    new_cu_d, old_cu_d = padded["cu_seqlens"].to(dev), old_cu.to(dev)
    un_ms, un_min = time_events(lambda: areal_amd.unpad_logits(logits, pad_len, new_cu_d, old_cu_d),
                                max(args.steps, 10), stream)
    n_tok = int(old_cu[-1])
    alg_bytes = 4.0 * n_tok * V
    achieved = alg_bytes / (un_ms * 1e-3) / 1e9
    sample = 2048
    t0 = time.perf_counter()
    cpu_rows = OP.unpad_logits(logits[: int(padded["cu_seqlens"][8])].cpu(), 0, padded["cu_seqlens"][:9], old_cu[:9])
    cpu_un_s = time.perf_counter() - t0
    got_rows = areal_amd.unpad_logits(logits, pad_len, new_cu_d, old_cu_d)[: cpu_rows.shape[0]].cpu()
    return dict(
        metric="tokens/sec for logits un-padding (packed, sequence-aligned micro-batch)",
        value=n_tok / (un_ms * 1e-3), unit="tokens/s", n_gpus=1, steps=args.steps, warmup=args.warmup,
        ms_per_step=un_ms, higher_is_better=True, scaling="weak", vs_baseline=None, dtype="bytes", data="synthetic",
        config=dict(workload=f"aux: per-token pieces at T={T}; pack of a [{bs}, {S}] batch; un-padding of bf16 logits "
                             f"[{T_pad}, {V}] (sequences aligned to 64 tokens, page padding {pad_len}) to [{n_tok}, {V}]"),
        roofline=dict(bound="hbm", kernel="k_copy_rows (aa_segment_copy)", achieved=achieved, peak=HBM_PEAK_GBS,
                      unit="GB/s", frac=achieved / HBM_PEAK_GBS, traffic=None, avg_kernel_ms=un_ms,
                      min_kernel_ms=un_min, algorithmic_bytes_per_launch=alg_bytes),
        cpu_baseline=dict(value=cpu_rows.shape[0] / cpu_un_s, unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                          sample=f"un-padding of the first 8 sequences ({cpu_rows.shape[0]} tokens) with the per-sequence "
                                 f"slice loop of the CPU oracle"),
        per_token_pieces=out_pieces, pack_tensor_dict_ms=pack_ms,
        cpu_sapo_plus_m2po_s=cpu_sib_s, cpu_dpo_loss_fwd_bwd_s=cpu_dpo_s,
        parity=dict(unpad_rows_equal=bool(torch.equal(got_rows, cpu_rows)),
                    sapo_loss_rel_err=abs(float(g_loss.detach()) - float(w_loss.detach())) / abs(float(w_loss.detach())),
                    sapo_grad_cosine=cosine(y.grad.cpu(), x.grad),
                    m2po_mask_mismatches=int((m2_gpu != m2_cpu).sum()),
                    dpo_loss_rel_err=abs(float(gd_loss.detach()) - float(wd_loss.detach())) / abs(float(wd_loss.detach())),
                    dpo_grad_cosine=cosine(yd.grad.cpu(), xd.grad)),
    )


def synth_lengths(total, seed):
    from areal_amd import synth

    return synth.truncate_to_total(synth.lengths_lognormal(64, 7.5, 0.6, 128, 4096, seed), total)


def bench_torch_ops(args, dev):
    """What the reference itself would execute on this GPU for the two paths, restated in plain torch ops (no kernel
    of this library runs in the timed regions): the vocabulary-sized functions exactly as
    areal/utils/functional/vocab_parallel.py:15-81 has them (log_softmax of the fp32 cast, gather, entropy, applied in
    chunks of 1024 rows; optionally under torch.compile, as the reference wraps them on GPUs), a token-level clipped
    surrogate on the [T] vectors after areal/utils/functional/functional.py:429-559 (a dozen elementwise ops, well under
    1 % of the time), autograd for the backward, and for the lm_head path the logits as torch.nn.functional.linear of
    hidden and weight (the library GEMM) with its two backward GEMMs over all tokens.  A reported baseline beside the
    figures of this library's paths on the same workloads; not a parity check."""
    import torch

    import areal_amd

    def logp_entropy(logits, labels, temperature):
        log_probs = torch.nn.functional.log_softmax(logits.float() / temperature, dim=-1)
        entropy = -torch.sum(log_probs.exp() * log_probs, dim=-1)
        return log_probs.gather(dim=-1, index=labels.unsqueeze(-1)).squeeze(-1), entropy

    def chunked(fn, logits, labels, temperature, chunk=1024):
        parts = [fn(logits[i:i + chunk], labels[i:i + chunk], temperature) for i in range(0, logits.shape[0], chunk)]
        return torch.cat([p[0] for p in parts]), torch.cat([p[1] for p in parts])

    def surrogate(logp, case, kw, cfg):
        mask = case.loss_mask.bool()
        behave = torch.exp(case.prox_logp - case.old_logp)
        if cfg is not None:
            mask = mask & (behave <= cfg.upper)
        ratio = torch.exp(logp - case.prox_logp)
        hi = kw.get("eps_clip_higher") or kw["eps_clip"]
        pg = torch.max(-case.advantages * ratio, -case.advantages * ratio.clamp(1.0 - kw["eps_clip"], 1.0 + hi))
        if kw.get("c_clip"):
            pg = torch.where(case.advantages < 0, torch.min(pg, -case.advantages * kw["c_clip"]), pg)
        return torch.where(mask, pg * behave, 0.0).sum() / mask.count_nonzero().clamp(min=1)

    def timed(step, iters):
        step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / iters * 1e3

    variants = [("eager", logp_entropy)]
    if args.torch_compile:
        variants.append(("torch.compile", torch.compile(logp_entropy)))
    out = dict(metric=METRIC, unit="tokens/s", n_gpus=1, data="synthetic", higher_is_better=True,
               config=dict(workload="the reference's torch ops on this GPU, beside this library's paths on the same inputs"))
    iters = max(args.steps // 4, 3)

    # logits path: configs[1] cut to 32 768 tokens
    case, desc = build_logits_case("cfg1-32k", args.seed, dev)
    kw, cfg = ppo_kwargs(case)
    T = case.logits.shape[0]
    leg = dict(workload=f"{case.name}: {desc}", tokens=T)
    for name, fn in variants:
        def step():
            x = case.logits.detach().requires_grad_(True)
            logp, _ = chunked(fn, x, case.labels, case.temperature)
            surrogate(logp, case, kw, cfg).backward()
        try:
            ms = timed(step, iters)
            leg[name] = dict(ms_per_step=ms, tokens_per_s=T / (ms * 1e-3))
        except Exception as e:  # a compiler that is not there or fails is reported, not fatal
            leg[name] = dict(error=f"{type(e).__name__}: {str(e)[:200]}")
    def ours():
        x = case.logits.detach().requires_grad_(True)
        loss, _ = areal_amd.fused_logprobs_ppo_loss(x, case.labels, case.prox_logp, case.old_logp, case.advantages,
                                                    loss_mask=case.loss_mask, rejection_sampling=cfg,
                                                    cu_seqlens=case.cu_seqlens, temperature=case.temperature, **kw)
        loss.backward()
    ms = timed(ours, max(args.steps, 10))
    leg["this_library"] = dict(ms_per_step=ms, tokens_per_s=T / (ms * 1e-3))
    out["logits_path"] = leg
    del case
    torch.cuda.empty_cache()

    # lm_head path: configs[2]
    case, desc = build_fused_case("cfg2", args.seed, dev)
    kw, cfg = ppo_kwargs(case)
    T = case.hidden.shape[0]
    leg = dict(workload=f"{case.name}: {desc}", tokens=T)
    for name, fn in variants:
        def step():
            h = case.hidden.detach().requires_grad_(True)
            w = case.weight.detach().requires_grad_(True)
            logp, _ = chunked(fn, torch.nn.functional.linear(h, w), case.labels, case.temperature)
            surrogate(logp, case, kw, cfg).backward()
        try:
            ms = timed(step, iters)
            leg[name] = dict(ms_per_step=ms, tokens_per_s=T / (ms * 1e-3))
        except Exception as e:
            leg[name] = dict(error=f"{type(e).__name__}: {str(e)[:200]}")
    def gemm():
        return torch.nn.functional.linear(case.hidden, case.weight)
    ms = timed(gemm, max(args.steps, 10))
    leg["library_gemm_logits_only"] = dict(ms=ms, tflops=2.0 * T * case.weight.shape[0] * case.hidden.shape[1] / (ms * 1e-3) / 1e12,
                                           note="torch.nn.functional.linear(hidden, weight) alone: the forward product, "
                                                "5 GB of bf16 logits written")
    # the two backward products at the step's shapes (rows of the tokens that have a gradient), library GEMM alone
    n_grad = int(case.loss_mask.count_nonzero())
    V_, H_ = case.weight.shape
    panel = (1e-3 * torch.randn(n_grad, V_, device=dev)).to(torch.bfloat16)
    rows = case.hidden[:n_grad].contiguous()
    for key, fn in (("library_gemm_d_hidden_only", lambda: panel @ case.weight),
                    ("library_gemm_d_weight_only", lambda: panel.t() @ rows)):
        ms = timed(fn, max(args.steps, 10))
        leg[key] = dict(ms=ms, tflops=2.0 * n_grad * V_ * H_ / (ms * 1e-3) / 1e12, rows=n_grad)
    del panel, rows

    def ours2():
        h = case.hidden.detach().requires_grad_(True)
        w = case.weight.detach().requires_grad_(True)
        loss, _ = areal_amd.fused_lm_head_ppo_loss(h, w, case.labels, case.prox_logp, case.old_logp, case.advantages,
                                                   loss_mask=case.loss_mask, rejection_sampling=cfg,
                                                   cu_seqlens=case.cu_seqlens, temperature=case.temperature, **kw)
        loss.backward()
    ms = timed(ours2, max(args.steps, 10))
    leg["this_library"] = dict(ms_per_step=ms, tokens_per_s=T / (ms * 1e-3))
    out["lm_head_path"] = leg
    best = min(v["ms_per_step"] for k, v in out["logits_path"].items() if isinstance(v, dict) and "ms_per_step" in v and k != "this_library")
    out["value"] = out["logits_path"]["tokens"] / (best * 1e-3)
    out["ms_per_step"] = best
    out["dtype"] = "bf16"
    return out


def main():
    global RS_ACTION, DENSE_BACKWARD, NO_FORWARD_OF_MASKED, BACKWARD_MODE
    args = parse_args()
    BACKWARD_MODE = 1 if args.lmhead_backward == "carry" else 0
    RS_ACTION = args.rs_action
    DENSE_BACKWARD = args.dense_backward
    NO_FORWARD_OF_MASKED = args.no_forward_of_masked
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; run it with --gpus 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "hbm":
        out = bench_hbm(args, dev)
    elif args.workload in MFMA_WORKLOADS:
        out = bench_mfma(args, dev)
    elif args.workload in TORCH_WORKLOADS:
        out = bench_torch_ops(args, dev)
        print(json.dumps(out))
        return
    elif args.workload == "aux":
        out = bench_aux(args, dev)
    elif args.workload in ADV_WORKLOADS:
        out = bench_adv(args, dev)
    elif args.workload in LOGITS_WORKLOADS:
        out, sample = bench_logits(args, dev, args.workload, args.steps, args.warmup, args.cpu_tokens)
        extra, fused_sample = None, None
        if args.workload == "cfg1" and not args.no_fused_extra and args.copy_launches == 0:
            # Every GPU timing of the run comes first, the CPU baselines last.
            # configs[1] says "T = 32k" of a length distribution that draws about 130k tokens: the headline figures
            # are on the distribution as stated; the same sequences cut at 32 768 tokens are quoted beside them
            torch.cuda.empty_cache()
            keys = ("value", "unit", "ms_per_step", "steps", "warmup", "config", "roofline", "copy_same_buffers",
                    "forward_only_logprobs")
            cut, _ = bench_logits(args, dev, "cfg1-32k", args.steps, args.warmup, 0, with_sft=False)
            out["configs1_cut_to_32k_tokens"] = {k: cut[k] for k in keys}
            torch.cuda.empty_cache()
            small, _ = bench_logits(args, dev, "cfg0", max(args.steps, 50), args.warmup, 0, with_sft=False)
            out["logits_config0"] = {k: small[k] for k in keys}
            torch.cuda.empty_cache()
            # the same 32 768 tokens handed over as fp32 logits (what a head that computes in fp32 emits): 8 bytes
            # per element, its own kernel
            import copy

            args32 = copy.copy(args)
            args32.logits_dtype = "f32"
            wide, _ = bench_logits(args32, dev, "cfg1-32k", args.steps, args.warmup, 0, with_sft=False)
            out["fp32_logits_cut_to_32k_tokens"] = {k: wide[k] for k in keys}
            torch.cuda.empty_cache()
            extra, fused_sample = bench_fused(args, dev, "cfg2", args.steps, args.warmup, min(args.cpu_tokens, 384))
            torch.cuda.empty_cache()
            # the two larger fused configurations, GPU only
            for wl in ("cfg3", "cfg4"):
                out[f"fused_lm_head_{wl}"] = bench_fused_leg(args, dev, wl, 3, 1)
                torch.cuda.empty_cache()
        finish_with_cpu_phase(out, sample, logits_cpu_phase, args.cpu_iters)
        if extra is not None:
            finish_with_cpu_phase(extra, fused_sample, fused_cpu_phase, args.cpu_iters)
            keys = ("value", "unit", "ms_per_step", "steps", "warmup", "config", "roofline", "cpu_baseline", "parity")
            out["fused_lm_head"] = {k: extra[k] for k in keys if k in extra}
    else:
        out, sample = bench_fused(args, dev, args.workload, args.steps, args.warmup, min(args.cpu_tokens, 384))
        torch.cuda.empty_cache()
        finish_with_cpu_phase(out, sample, fused_cpu_phase, args.cpu_iters)
    # the two fractions the metric names, beside the throughput: of the HBM peak on the logits path, of the bf16 MFMA
    # peak on the fused lm_head path (whichever of the two this run measured)
    fractions = {}
    for part in (out, out.get("fused_lm_head", {})):
        roof = part.get("roofline")
        if roof:
            fractions["pct_hbm_peak" if roof["bound"] == "hbm" else "pct_mfma_peak"] = 100.0 * roof["frac"]
    if "fp32_logits_cut_to_32k_tokens" in out:
        fractions["pct_hbm_peak_fp32_logits"] = 100.0 * out["fp32_logits_cut_to_32k_tokens"]["roofline"]["frac"]
    for wl in ("cfg3", "cfg4"):
        if f"fused_lm_head_{wl}" in out:
            fractions[f"pct_mfma_peak_{wl}"] = 100.0 * out[f"fused_lm_head_{wl}"]["roofline"]["frac"]
    out["pct_of_peak"] = fractions
    print(json.dumps(out))


if __name__ == "__main__":
    main()
