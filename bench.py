#!/usr/bin/env python3
"""Benchmark of the PPO/GRPO log-prob + entropy + actor-loss path (forward and backward) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg1|cfg1-32k|cfg0]

One "step" is one pass of the hot path over one synthetic packed micro-batch that is already resident in HBM:
rejection sampling (importance-weight cap) -> fused log-prob / entropy / clipped PPO loss / d(logits) -> scalar
loss, i.e. ``fused_logprobs_ppo_loss(...)`` followed by ``loss.backward()``.  Prints ONE JSON line.

Besides the whole-step throughput the line carries
  roofline      achieved HBM bandwidth of the dominant kernel (algorithmic bytes = 4 * V per token: the bf16
                logits read once, their gradient written once) from HIP events around each launch;
  cpu_baseline  the CPU oracle (a PyTorch restatement of the reference path) timed on this machine's host
                cores on a bounded token sample of the same workload;
  parity        the GPU result checked against that oracle on the same sample.
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

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg1", choices=["cfg0", "cfg1", "cfg1-32k"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--cpu-tokens", type=int, default=1024, help="token sample of the CPU baseline (0 = skip)")
    ap.add_argument("--cpu-iters", type=int, default=3)
    ap.add_argument("--copy-launches", type=int, default=0,
                    help="also launch the plain copy kernel this many times over the logits buffer "
                         "(the calibration point for FETCH_SIZE / WRITE_SIZE counters)")
    return ap.parse_args()


def build_case(name: str, seed: int, device):
    import areal_amd
    from areal_amd import synth

    if name == "cfg0":
        case = synth.config0(device, seed)
        desc = "configs[0]: 16 packed seqs, lengths U[64,512], V=151936, eps_clip=0.2"
    elif name == "cfg1":
        case = synth.config1(device, seed)
        desc = ("configs[1]: 64 packed seqs, lengths lognormal(7.5,0.6) clipped to [128,4096], V=151936, GRPO groups "
                "of 16, decoupled loss, importance-weight cap 5.0 (token/mask/ratio)")
    else:
        case = synth.config1(device, seed, total_tokens=32768)
        desc = "configs[1] truncated to the leading sequences that total 32768 tokens"
    ref = areal_amd.gather_logprobs(case.logits, case.labels, case.temperature)
    synth.attach_old_and_prox(case, ref, 0.05, seed + 9)
    return case, desc


def ppo_kwargs(case):
    from areal_amd import RejectionSamplingConfig

    kw = dict(case.ppo)
    rs = kw.pop("rejection_sampling", None)
    cfg = RejectionSamplingConfig(**rs) if rs else None
    return kw, cfg


def run_steps(case, n, kw, cfg):
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


def time_dominant_kernel(case, kw, cfg, iters: int):
    """Average duration of aa_logits_ppo_fused alone, HIP events on the launch stream, outputs pre-allocated."""
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
    logp, ent, sl, ratio = (torch.empty(T, **f32) for _ in range(4))
    flags = torch.empty(T, dtype=torch.uint8, device=dev)
    dlogits = torch.empty_like(case.logits)
    stream = torch.cuda.current_stream(dev)

    def launch():
        N.check(
            lib.aa_logits_ppo_fused(
                F._ptr(case.logits), N.AA_BF16, T, V, V, F._ptr(case.labels), 1.0 / case.temperature, T,
                F._ptr(prox), F._ptr(adv), F._ptr(mask_eff), F._ptr(w), C.byref(params), F._ptr(counts), None,
                F._ptr(logp), F._ptr(ent), None, None, F._ptr(sl), F._ptr(ratio), F._ptr(flags), F._ptr(dlogits),
                F._ptr(F._work_words(dev)), C.c_void_p(stream.cuda_stream),
            ),
            "aa_logits_ppo_fused",
        )

    for _ in range(3):
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


def cpu_baseline_and_parity(case, kw, cfg, n_tokens: int, iters: int):
    """Oracle fwd+bwd on the first ``n_tokens`` tokens (host cores), and the GPU path checked on the same slice."""
    import torch

    import areal_amd
    import oracle

    n = min(n_tokens, case.n_tokens)
    sl = slice(0, n)
    cpu = lambda t: t[sl].cpu()
    args = (cpu(case.logits), cpu(case.labels), cpu(case.prox_logp), cpu(case.old_logp), cpu(case.advantages))
    cu = torch.tensor([0, n], dtype=torch.int32)  # token-level options only: segments do not matter here
    okw = dict(kw, loss_mask=cpu(case.loss_mask), rejection_sampling_cfg=cfg, cu_seqlens=cu,
               temperature=case.temperature)
    threads = torch.get_num_threads()
    oracle.logits_ppo_step(*args, **okw)  # warm-up
    t0 = time.perf_counter()
    for _ in range(iters):
        w_loss, w_stat, w_grad = oracle.logits_ppo_step(*args, **okw)
    dt = (time.perf_counter() - t0) / iters

    x = case.logits[sl].detach().clone().requires_grad_(True)
    loss, stat = areal_amd.fused_logprobs_ppo_loss(
        x, case.labels[sl], case.prox_logp[sl], case.old_logp[sl], case.advantages[sl], loss_mask=case.loss_mask[sl],
        rejection_sampling=cfg, cu_seqlens=cu.to(x.device), temperature=case.temperature, **kw,
    )
    loss.backward()
    torch.cuda.synchronize()
    a, b = x.grad.cpu().double().reshape(-1), w_grad.double().reshape(-1)
    parity = dict(
        tokens=n,
        logp_max_abs_err=float((stat["logprobs"].cpu() - w_stat["logprobs"]).abs().max()),
        loss_rel_err=abs(float(loss.detach()) - float(w_loss)) / max(abs(float(w_loss)), 1e-12),
        grad_cosine=float(a @ b / (a.norm() * b.norm())),
        masks_equal=bool(torch.equal(stat["clip_mask"].cpu(), w_stat["clip_mask"])),
    )
    baseline = dict(
        value=n / dt, unit="tokens/s", cores=threads, kind="port",
        sample=f"first {n} tokens of the workload, {iters} timed fwd+bwd passes of the PyTorch CPU oracle "
               f"(chunked fp32 log_softmax + gather + entropy + PPO loss + autograd to bf16 d(logits))",
    )
    return baseline, parity


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; run it with --gpus 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    case, desc = build_case(args.workload, args.seed, dev)
    kw, cfg = ppo_kwargs(case)
    T, V = case.logits.shape
    case.logits.requires_grad_(True)

    run_steps(case, args.warmup, kw, cfg)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loss = run_steps(case, args.steps, kw, cfg)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    assert bool(torch.isfinite(loss)), "loss is not finite"

    case.logits.grad = None
    case.logits.requires_grad_(False)
    k_ms, k_min_ms = time_dominant_kernel(case, kw, cfg, max(args.steps, 10))
    alg_bytes = 4.0 * T * V
    achieved = alg_bytes / (k_ms * 1e-3) / 1e9
    roofline = dict(
        bound="hbm", kernel="k_fused_regs (aa_logits_ppo_fused)", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s",
        frac=achieved / HBM_PEAK_GBS,
        # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters read
        # for the plain copy kernel: 1.001 x the algorithmic bytes (profiles/k_fused_regs_cfg1-32k_hbm_traffic.md)
        traffic=alg_bytes * 1.001, avg_kernel_ms=k_ms, min_kernel_ms=k_min_ms,
        algorithmic_bytes_per_launch=alg_bytes,
    )
    out = dict(
        metric="tokens/sec for logprob+entropy+PPO loss fwd+bwd", value=T / (ms_per_step * 1e-3), unit="tokens/s",
        n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms_per_step, higher_is_better=True,
        scaling="weak", vs_baseline=None, dtype="bf16", data="synthetic",
        config=dict(workload=f"{case.name}: {desc}", tokens=T, vocab=V, sequences=int(case.cu_seqlens.numel() - 1),
                    accumulate="f32", path="logits (fused fwd + PPO loss + bwd, one launch)"),
        roofline=roofline,
    )
    if args.copy_launches > 0:
        from areal_amd import _native as N
        from areal_amd import functional as F

        dst = torch.empty_like(case.logits)
        nbytes = case.logits.numel() * case.logits.element_size()
        for _ in range(args.copy_launches):
            N.check(N.load().aa_copy_bytes(F._ptr(case.logits), F._ptr(dst), nbytes, F._stream(dev)), "aa_copy_bytes")
        torch.cuda.synchronize()
        out["copy_calibration"] = dict(kernel="k_copy16 (aa_copy_bytes)", bytes_read=nbytes, bytes_written=nbytes,
                                       launches=args.copy_launches)
    if args.cpu_tokens > 0:
        baseline, parity = cpu_baseline_and_parity(case, kw, cfg, args.cpu_tokens, args.cpu_iters)
        out["cpu_baseline"] = baseline
        out["parity"] = parity
    print(json.dumps(out))


if __name__ == "__main__":
    main()
