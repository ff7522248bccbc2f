"""GPU parity of gather_logprobs / gather_logprobs_entropy (forward and backward) against the CPU oracle.

Tolerances are the ones the task states: log-probs within 2e-3 absolute of an fp32/fp64 reference, gradient
cosine similarity above 0.9999; integer indexing (labels) bit-exact, which shows as exact agreement of the
gathered element."""
import math

import pytest
import torch

import areal_amd
import oracle
from helpers import assert_same_magnitude, cosine

pytestmark = pytest.mark.gpu

LOGP_ATOL = 2e-3   # stated tolerance
TIGHT = 2e-5       # what fp32 accumulation actually delivers


def _case(T, V, dtype, seed, std=3.0):
    g = torch.Generator().manual_seed(seed)
    x = (std * torch.randn(T, V, generator=g)).to(dtype)
    y = torch.randint(0, V, (T,), generator=g)
    return x, y


@pytest.mark.parametrize(
    "T,V,dtype",
    [
        (37, 128, torch.float32),       # the reference's determinism-test shape class
        (33, 1000, torch.bfloat16),
        (5, 50257, torch.bfloat16),     # odd V: rows are not 16-byte aligned
        (19, 32003, torch.float16),
        (3, 151936, torch.bfloat16),    # the benchmark vocabulary
        (2, 262144, torch.float32),
        (1, 7, torch.bfloat16),         # shorter than one vector
    ],
)
@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_forward_matches_oracle(device, T, V, dtype, temperature):
    x, y = _case(T, V, dtype, seed=T + V)
    lp, ent = areal_amd.gather_logprobs_entropy(x.to(device), y.to(device), temperature)
    lp_only = areal_amd.gather_logprobs(x.to(device), y.to(device), temperature)
    ref_lp, ref_ent = oracle.logprobs_entropy_f64(x, y, temperature)
    assert lp.dtype == torch.float32 and lp.shape == y.shape
    assert float((lp.cpu().double() - ref_lp).abs().max()) < min(LOGP_ATOL, TIGHT * max(1.0, math.log(V)))
    assert float((ent.cpu().double() - ref_ent).abs().max()) < 1e-4
    assert torch.equal(lp_only, lp)
    # fp32 restatement of the reference path agrees as well
    o_lp, o_ent = oracle.logprobs_entropy(x, y, temperature)
    assert float((lp.cpu() - o_lp).abs().max()) < 1e-4


def test_vocab_min_max_by_products_are_exact(device):
    x, y = _case(9, 4099, torch.bfloat16, seed=3)
    lp, ent, vmin, vmax = areal_amd.gather_logprobs_entropy_stats(x.to(device), y.to(device))
    assert torch.equal(vmin.cpu(), x.min(-1).values.float())
    assert torch.equal(vmax.cpu(), x.max(-1).values.float())


def test_leading_dims_strides_and_label_dtypes(device):
    x, y = _case(24, 515, torch.bfloat16, seed=5)
    ref, _ = oracle.logprobs_entropy_f64(x, y)
    # [B, S, V] input, int32 labels
    lp3 = areal_amd.gather_logprobs(x.view(4, 6, 515).to(device), y.view(4, 6).int().to(device))
    assert lp3.shape == (4, 6)
    assert float((lp3.cpu().double().view(-1) - ref).abs().max()) < TIGHT * 10
    # rows of a wider buffer (row stride > V)
    wide = torch.zeros(24, 640, dtype=torch.bfloat16, device=device)
    wide[:, :515] = x.to(device)
    lp_s = areal_amd.gather_logprobs(wide[:, :515], y.to(device))
    assert float((lp_s - lp3.view(-1)).abs().max()) < 1e-5  # other alignment, other summation order
    # offset view: base pointer not 16-byte aligned
    flat = torch.zeros(24 * 515 + 3, dtype=torch.bfloat16, device=device)
    flat[3:] = x.to(device).reshape(-1)
    lp_o = areal_amd.gather_logprobs(flat[3:].view(24, 515), y.to(device))
    assert float((lp_o - lp_s).abs().max()) < 1e-5


def test_closed_forms_and_stability(device):
    V = 4096
    x = torch.full((2, V), 0.75, dtype=torch.bfloat16, device=device)
    y = torch.tensor([0, V - 1], device=device)
    lp, ent = areal_amd.gather_logprobs_entropy(x, y)
    assert float((lp + math.log(V)).abs().max()) < 1e-5 and float((ent - math.log(V)).abs().max()) < 1e-4
    x = torch.zeros(1, V, device=device)
    x[0, 9] = 80.0
    lp, ent = areal_amd.gather_logprobs_entropy(x, torch.tensor([9], device=device))
    assert abs(float(lp)) < 1e-6 and abs(float(ent)) < 1e-6
    # logits scaled by 100 stay finite and match (run_vocab_parallel.py:169-215 of the reference)
    g = torch.Generator().manual_seed(7)
    big = torch.randn(6, 333, generator=g) * 100
    yy = torch.randint(0, 333, (6,), generator=g)
    lp, ent = areal_amd.gather_logprobs_entropy(big.to(device), yy.to(device))
    r_lp, r_ent = oracle.logprobs_entropy_f64(big, yy)
    assert torch.isfinite(lp).all() and float((lp.cpu().double() - r_lp).abs().max()) < 1e-3
    assert float((ent.cpu().double() - r_ent).abs().max()) < 1e-3
    # shift invariance
    a = areal_amd.gather_logprobs(big.to(device) / 100, yy.to(device))
    b = areal_amd.gather_logprobs(big.to(device) / 100 + 5.0, yy.to(device))
    assert float((a - b).abs().max()) < 1e-5


def test_two_calls_are_bit_identical(device):
    # tests/test_cuda_deterministic.py:199-225 of the reference asks rtol=0, atol=0 of its compiled op
    torch.manual_seed(42)
    x = torch.randn(32, 128, device=device)
    y = torch.randint(0, 128, (32,), device=device)
    a = areal_amd.gather_logprobs_entropy(x, y)
    b = areal_amd.gather_logprobs_entropy(x, y)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    xb = (3 * torch.randn(16, 151936, device=device)).bfloat16()
    yb = torch.randint(0, 151936, (16,), device=device)
    a = areal_amd.gather_logprobs_entropy(xb, yb)
    b = areal_amd.gather_logprobs_entropy(xb, yb)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_errors_and_out_of_range_labels(device):
    with pytest.raises(AssertionError):
        areal_amd.gather_logprobs(torch.zeros(0, 8, device=device), torch.zeros(0, dtype=torch.long, device=device))
    with pytest.raises(ValueError, match="shape"):
        areal_amd.gather_logprobs(torch.zeros(2, 8, device=device), torch.zeros(3, dtype=torch.long, device=device))
    x = torch.randn(3, 64, device=device)
    y = torch.tensor([5, 64, -1], device=device)  # only the first is valid
    lp = areal_amd.gather_logprobs(x, y)
    assert torch.isfinite(lp[0]) and torch.isnan(lp[1]) and torch.isnan(lp[2])


@pytest.mark.parametrize(
    "T,V,dtype,temperature,with_entropy",
    [
        (11, 257, torch.float32, 1.0, True),
        (11, 257, torch.float32, 0.6, True),
        (7, 4104, torch.bfloat16, 1.0, False),
        (7, 4104, torch.bfloat16, 0.7, True),
        (4, 50257, torch.bfloat16, 1.0, True),
        (5, 1031, torch.float16, 1.3, True),
        (2, 151936, torch.bfloat16, 1.0, False),
    ],
)
def test_backward_matches_autograd_of_oracle(device, T, V, dtype, temperature, with_entropy):
    x, y = _case(T, V, dtype, seed=11 * T + V, std=2.0)
    g = torch.Generator().manual_seed(1)
    gl = torch.randn(T, generator=g)
    gh = torch.randn(T, generator=g) if with_entropy else None
    gl[0] = 0.0  # a row without log-prob gradient
    xd = x.to(device).requires_grad_(True)
    if with_entropy:
        lp, ent = areal_amd.gather_logprobs_entropy(xd, y.to(device), temperature)
        ((lp * gl.to(device)).sum() + (ent * gh.to(device)).sum()).backward()
    else:
        lp = areal_amd.gather_logprobs(xd, y.to(device), temperature)
        (lp * gl.to(device)).sum().backward()
    got = xd.grad
    assert got.dtype == dtype and got.shape == x.shape
    want64 = oracle.logprobs_entropy_grad_closed_form(x, y, gl, gh, temperature)
    # autograd of the fp32 restatement (what the reference itself would return in this dtype)
    xo = x.clone().requires_grad_(True)
    o_lp, o_ent = oracle.logprobs_entropy(xo, y, temperature)
    ((o_lp * gl).sum() + ((o_ent * gh).sum() if with_entropy else 0.0)).backward()
    assert cosine(got.cpu(), want64) > 0.9999
    assert cosine(got.cpu(), xo.grad) > 0.9999
    if dtype == torch.float32:
        assert float((got.cpu().double() - want64).abs().max()) < 1e-5  # atol of run_vocab_parallel.py:257-317
    else:
        # no worse than one rounding of the exact value to the storage type
        err = (got.cpu().double() - want64).abs()
        assert bool((err <= want64.abs() * 2 ** -7 + 1e-6).all())
    if not with_entropy:
        assert float(got[0].float().abs().max()) == 0.0
        assert float(got.float().sum(-1).abs().max()) < 5e-2  # each row of (onehot - p) sums to zero


@pytest.mark.parametrize(
    "T,V,dtype",
    [
        (6, 4104, torch.bfloat16),     # rows that stay in registers
        (5, 1031, torch.float32),      # unaligned rows: the generic walk
        (3, 151936, torch.bfloat16),   # the benchmark vocabulary
        (2, 300000, torch.float32),    # rows longer than the register file
    ],
)
def test_masked_vocabulary_entries_of_minus_infinity(device, T, V, dtype):
    """Logits of -inf (vocabulary entries a sampler has masked) take probability 0: the log-probs stay finite and the
    gradient of the log-probs is exactly 0 there, as autograd of log_softmax gives it (not 0 * inf)."""
    x, y = _case(T, V, dtype, seed=V + T, std=2.0)
    g = torch.Generator().manual_seed(2)
    masked = torch.rand(T, V, generator=g) < 0.3
    masked[torch.arange(T), y] = False
    masked[:, -1] = True       # the scalar tail of an unaligned row
    masked[:, 0] = y != 0      # and its head
    x[masked] = float("-inf")
    gl = torch.randn(T, generator=g)
    xd = x.to(device).requires_grad_(True)
    lp = areal_amd.gather_logprobs(xd, y.to(device), 0.8)
    (lp * gl.to(device)).sum().backward()
    xo = x.double().requires_grad_(True)
    o_lp = torch.log_softmax(xo / 0.8, dim=-1).gather(-1, y[:, None]).squeeze(-1)
    (o_lp * gl.double()).sum().backward()
    assert torch.isfinite(lp).all()
    assert float((lp.detach().cpu().double() - o_lp.detach()).abs().max()) < LOGP_ATOL
    got = xd.grad.cpu()
    assert torch.isfinite(got).all()
    assert float(got[masked].float().abs().max()) == 0.0
    assert cosine(got, xo.grad) > 0.9999
    assert_same_magnitude(got, xo.grad, what="d_logits")
    # the fused PPO step walks the same rows with its own gradient code.  Importance ratio 1 on every token:
    # loss = -mean(adv), so d loss / d logits = -(adv / T) d logp / d logits
    xf = x.to(device).requires_grad_(True)
    loss, stat = areal_amd.fused_logprobs_ppo_loss(xf, y.to(device), lp.detach(), lp.detach(), gl.to(device), 0.2,
                                                   torch.ones(T, dtype=torch.bool, device=device), temperature=0.8)
    loss.backward()
    assert torch.isfinite(stat["logprobs"]).all() and torch.isfinite(xf.grad).all()
    assert float(xf.grad.cpu()[masked].float().abs().max()) == 0.0
    assert_same_magnitude(xf.grad.cpu(), -xo.grad / T, what="fused d_logits")


def test_plain_c_consumer_of_the_abi(device):
    """tests/c_abi/consumer.c drives the library from C99 with hipMalloc'ed buffers and checks log-probs, entropy, the
    supervised loss, its gradient and the per-sequence statistics against values it computes itself in double."""
    import subprocess
    from pathlib import Path

    exe = Path(__file__).resolve().parent / "c_abi" / "consumer"
    if not exe.exists():      # normally built beforehand by __graft_entry__.build(); built here only if it is missing
        import sys

        sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
        import __graft_entry__

        __graft_entry__.build_c_abi_consumer()
    assert exe.exists()
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "c_abi consumer ok" in run.stdout


@pytest.mark.parametrize("cuts,dtype,temperature", [([0.5], torch.bfloat16, 1.0), ([0.1, 0.35, 0.8], torch.float32, 0.7),
                                                    ([0.125 * i for i in range(1, 8)], torch.bfloat16, 1.3)])
def test_vocab_shards_equal_the_unsharded_op(device, cuts, dtype, temperature):
    """The vocabulary axis cut into 2 / 4 / 8 slices (uneven ones too): statistics per slice, one combine, backward
    per slice from the combined statistics (vocab_parallel.py:84-372 without its collectives) against the oracle and
    against the unsharded kernels."""
    import oracle
    from areal_amd import vocab_parallel as VP

    T, V = 300, 24000
    g = torch.Generator().manual_seed(3)
    logits = (torch.randn(T, V, generator=g) * 3).to(dtype)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[:4] = torch.tensor([0, V - 1, int(cuts[0] * V) // 8 * 8 - 1, int(cuts[0] * V) // 8 * 8])   # slice borders
    bounds = [0] + [int(c * V) // 8 * 8 for c in cuts] + [V]
    x = logits.clone().requires_grad_(True)
    w_lp, w_ent = oracle.logprobs_entropy(x, labels, temperature)
    gl, gh = torch.randn(T, generator=g), torch.randn(T, generator=g)
    (w_lp * gl + w_ent * gh).sum().backward()
    shards = [logits[:, a:b].contiguous().to(device).requires_grad_(True) for a, b in zip(bounds[:-1], bounds[1:])]
    lp, ent = VP.gather_logprobs_entropy_vocab_shards(shards, labels.to(device), temperature)
    (lp * gl.to(device) + ent * gh.to(device)).sum().backward()
    assert float((lp.detach().cpu() - w_lp.detach()).abs().max()) < 2e-3
    assert float((ent.detach().cpu() - w_ent.detach()).abs().max()) < 2e-3
    grad = torch.cat([sh.grad for sh in shards], dim=1).float().cpu()
    assert cosine(grad, x.grad.float()) > 0.9999
    assert_same_magnitude(grad, x.grad.float(), what="sharded d_logits")
    # against the unsharded kernels: the same numbers up to the order of the sums
    y = logits.to(device).requires_grad_(True)
    lp1, ent1 = areal_amd.gather_logprobs_entropy(y, labels.to(device), temperature)
    (lp1 * gl.to(device) + ent1 * gh.to(device)).sum().backward()
    assert torch.allclose(lp, lp1, atol=2e-5) and torch.allclose(ent, ent1, atol=2e-5)
    tol = (1e-4 if dtype == torch.float32 else 2e-2) * float(y.grad.float().abs().max())   # bf16: one rounding step
    assert float((grad - y.grad.float().cpu()).abs().max()) <= tol
    # a label that lies in no slice gives NaN, as the unsharded op does for a label out of range
    lse, ez, lpl, _ = VP.shard_statistics(shards[0], torch.full((T,), V + 5), 0, temperature)
    out = VP.combine_shard_statistics(lse[None], ez[None], lpl[None])
    assert bool(torch.isnan(out[0]).all()) and bool(torch.isfinite(out[1]).all())


@pytest.mark.parametrize("V,dtype", [(16384, torch.bfloat16), (50257, torch.bfloat16), (4099, torch.float32)])
def test_backward_written_over_the_logits(device, V, dtype):
    """inplace_backward=True: the backward pass of the log-prob op writes the gradient over the logits, with the bits
    of the separate array; through a producer of the logits, and through the sequence-level PPO loss."""
    g = torch.Generator().manual_seed(V)
    T = 37
    logits = (2 * torch.randn(T, V, generator=g)).to(dtype).to(device)
    labels = torch.randint(0, V, (T,), generator=g).to(device)
    g_lp, g_ent = torch.randn(T, generator=g).to(device), torch.randn(T, generator=g).to(device)

    def run(inplace):
        base = logits.clone().requires_grad_(True)
        x = base * 1.0                                   # a producer: the logits are not a leaf
        lp, ent = areal_amd.gather_logprobs_entropy(x, labels, 0.8, inplace_backward=inplace)
        (lp * g_lp + ent * g_ent).sum().backward()
        return lp.detach(), ent.detach(), base.grad, x.detach()

    lp0, ent0, grad0, x0 = run(False)
    lp1, ent1, grad1, x1 = run(True)
    assert torch.equal(lp0, lp1) and torch.equal(ent0, ent1) and torch.equal(grad0, grad1)
    assert torch.equal(x0, logits) and torch.equal(x1, grad1)   # untouched / holds its own gradient

    # sequence-level importance ratios: the unfused kernels behind fused_logprobs_ppo_loss
    cu = torch.tensor([0, 20, T], dtype=torch.int32, device=device)
    ref = areal_amd.gather_logprobs(logits, labels).detach()
    adv, mask = torch.randn(T, generator=g).to(device), (torch.rand(T, generator=g) < 0.7).to(device)

    def step(inplace):
        base = logits.clone().requires_grad_(True)
        x = base * 1.0
        loss, _ = areal_amd.fused_logprobs_ppo_loss(x, labels, ref - 0.05, ref + 0.03, adv, 0.2, mask,
                                                    importance_sampling_level="sequence", cu_seqlens=cu,
                                                    inplace_backward=inplace)
        loss.backward()
        return loss.detach(), base.grad

    l0, s0 = step(False)
    l1, s1 = step(True)
    assert torch.equal(l0, l1) and torch.equal(s0, s1)


def test_hbm_stream_probe_moves_what_it_says(device):
    """The measurement kernels behind `bench.py --workload hbm`: the copy copies every byte (ragged last piece
    included), the write fills exactly the buffer, the read writes nothing, with either cache policy."""
    import ctypes as C

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    st = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    n = 16 * (256 * 8 * 5 + 77)                              # five whole 32 KB pieces and a ragged one
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device=device)
    for nt in (0, 1):
        dst = torch.full((n + 64,), 7, dtype=torch.uint8, device=device)
        assert lib.aa_hbm_stream_probe(2, nt, F._ptr(src), F._ptr(dst), n, 3, st) == 0
        assert torch.equal(dst[:n], src) and bool((dst[n:] == 7).all())
        dst.fill_(7)
        assert lib.aa_hbm_stream_probe(1, nt, None, F._ptr(dst), n, 3, st) == 0
        assert bool((dst[n:] == 7).all())
        words = dst[:n].view(torch.int32).view(-1, 4)
        assert bool((words[:, 2] == 2).all()) and bool((words[:, 3] == 3).all())
        before = src.clone()
        assert lib.aa_hbm_stream_probe(0, nt, F._ptr(src), None, n, 3, st) == 0
        assert torch.equal(src, before)
    assert lib.aa_hbm_stream_probe(3, 0, F._ptr(src), None, n, 3, st) == 1      # unknown kind
    assert lib.aa_hbm_stream_probe(2, 0, F._ptr(src), None, n, 3, st) == 1      # a copy needs a destination
    assert lib.aa_hbm_stream_probe(0, 0, F._ptr(src), None, n + 8, 3, st) == 1  # not a multiple of 16
