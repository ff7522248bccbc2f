"""GPU parity of the lm_head path.  The reference has no such path, so the oracle is its equivalent in fp32:
logits = hidden @ weight.T, then the log-prob / entropy oracle, with autograd for the gradients.  Stated tolerance:
log-probs within 2e-3 of that fp32 reference, for every token.  The reference's own pipeline rounds the lm_head output
to bf16 first; one test ties the two together."""
import math

import pytest
import torch

import areal_amd
import oracle
from areal_amd import _native
from helpers import assert_same_magnitude, assert_within, assert_within_one_bf16_logit_step, cosine

pytestmark = pytest.mark.gpu

CHUNK = int(_native.load().aa_lmhead_chunk_tokens())  # tokens per chunk of the lm_head entry points


def _case(T, H, V, seed, w_std=0.02):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (w_std * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    return hidden, weight, labels


@pytest.mark.parametrize(
    "T,H,V,temperature",
    [
        (256, 128, 1024, 1.0),
        (300, 192, 1088, 1.0),    # token count not a multiple of 8
        (37, 64, 576, 0.7),
        (700, 256, 4160, 1.3),
        (203, 200, 1096, 1.0),    # H and V multiples of 8 only
        (37, 64, 577, 0.7),       # vocabularies that are no multiple of 8 (the reference takes any, vocab_parallel.py:15-29)
        (300, 128, 1001, 1.0),
        (70, 64, 50257, 1.0),
        (40, 64, 151643, 1.0),
    ],
)
def test_forward_matches_oracle(device, T, H, V, temperature):
    hidden, weight, labels = _case(T, H, V, seed=T + V, w_std=0.3)
    lp, ent = areal_amd.lm_head_logprobs_entropy(hidden.to(device), weight.to(device), labels.to(device), temperature)
    logits = oracle.lmhead_logits(hidden, weight)
    r_lp, r_ent = oracle.logprobs_entropy_f64(logits, labels, temperature)
    assert lp.dtype == torch.float32 and lp.shape == (T,)
    assert_within(lp, r_lp, 2e-3, "log-prob")  # stated tolerance, every token
    assert_within(ent, r_ent, 2e-3, "entropy")
    assert float((lp.cpu().double() - r_lp).abs().max()) < 1e-4  # what the kernel actually achieves
    # the reference's pipeline hands bf16 logits to gather_logprobs_entropy: no token further from it than that rounding
    b_lp, b_ent = oracle.logprobs_entropy_f64(oracle.lmhead_logits(hidden, weight, round_to_bf16=True), labels, temperature)
    assert_within_one_bf16_logit_step(lp, b_lp, float(logits.abs().max()) / temperature, "log-prob vs bf16 pipeline")
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
        areal_amd.lm_head_logprobs_entropy(hidden[:, :44].contiguous(), weight[:, :44].contiguous(), labels)  # H % 8


@pytest.mark.parametrize("T,H,V,temperature,with_entropy",
                         [(300, 128, 1088, 1.0, False), (520, 192, 832, 0.8, True), (203, 200, 1096, 1.0, True),
                          (300, 128, 16640, 1.0, True),    # d(hidden) cut into parts along the vocabulary
                          (203, 72, 1097, 1.0, True), (70, 64, 50257, 0.9, False),  # any vocabulary size
                          (300, 128, 16643, 1.0, True)])   # ... with d(hidden) cut into parts
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
    o_lp, o_ent = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), labels, temperature)
    ref = (o_lp * gl).sum() + ((o_ent * gh).sum() if with_entropy else 0.0)
    ref.backward()
    assert h_d.grad.dtype == torch.bfloat16 and w_d.grad.dtype == torch.bfloat16
    assert cosine(h_d.grad.cpu(), h_o.grad) > 0.9999
    assert cosine(w_d.grad.cpu(), w_o.grad) > 0.9999
    assert_same_magnitude(h_d.grad, h_o.grad, what="d(hidden)")
    assert_same_magnitude(w_d.grad, w_o.grad, what="d(W)")


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
    o_lp, _ = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), labels)
    o_loss, _ = oracle.ppo_actor_loss(o_lp, prox, old, adv, 0.2, mask, 0.28, 3.0)
    o_loss.backward()
    assert float(loss.detach()) == pytest.approx(float(o_loss.detach()), rel=1e-3)
    assert cosine(h_d.grad.cpu(), h_o.grad) > 0.9999 and cosine(w_d.grad.cpu(), w_o.grad) > 0.9999
    assert_same_magnitude(h_d.grad, h_o.grad, what="d(hidden)")
    assert_same_magnitude(w_d.grad, w_o.grad, what="d(W)")


# ---------------------------------------------------------------------------------------------------------------
# Full-size configurations.  The oracle cannot run these whole, so they are checked on token slices (every token's
# log-prob, entropy and d(hidden) row depend only on that token's hidden state and the full weight matrix) and
# through properties that hold at any size: determinism, log-prob <= 0, 0 <= entropy <= log V, and linearity of
# d(W) in the upstream gradient, which ties the full-size weight gradient to a slice the oracle can compute.
# ---------------------------------------------------------------------------------------------------------------
def _cos_dev(a, b, device):
    a, b = a.to(device).double().reshape(-1), b.to(device).double().reshape(-1)
    return float(a @ b / (a.norm() * b.norm()))


def _oracle_slice(case, idx, g_slice):
    h = case.hidden[idx].cpu().float().requires_grad_(True)
    w = case.weight.cpu().float().requires_grad_(True)
    lp, ent = oracle.logprobs_entropy(oracle.lmhead_logits(h, w), case.labels[idx].cpu(), case.temperature)
    (lp * g_slice).sum().backward()
    return lp.detach(), ent.detach(), h.grad, w.grad


@pytest.mark.parametrize("name", ["cfg2", "cfg4", "cfg3"])
def test_full_size_configuration(device, name):
    from areal_amd import synth

    case = getattr(synth, {"cfg2": "config2", "cfg3": "config3", "cfg4": "config4"}[name])(device, seed=0)
    T, H = case.hidden.shape
    V = case.weight.shape[0]
    print(f"full-size {name}: T={T} H={H} V={V}", flush=True)
    n_s = 48
    idx = torch.cat([torch.arange(0, 16), torch.arange(T // 2 - 8, T // 2 + 8), torch.arange(T - 16, T)]).to(device)
    g = torch.Generator().manual_seed(11)
    g_slice = torch.randn(n_s, generator=g)
    g_rest = (torch.randn(T, generator=g) * case.loss_mask.cpu().float()).to(device)
    g_rest[idx] = 0.0
    g_only = torch.zeros(T, device=device)
    g_only[idx] = g_slice.to(device)

    def run(gvec):
        h = case.hidden.detach().requires_grad_(True)
        w = case.weight.detach().requires_grad_(True)
        lp, ent = areal_amd.lm_head_logprobs_entropy(h, w, case.labels, case.temperature)
        (lp * gvec).sum().backward()
        return lp.detach(), ent.detach(), h.grad, w.grad

    lp, ent, dh_only, dw_only = run(g_only)
    assert bool((lp <= 1e-6).all()) and bool((ent >= -1e-4).all()) and bool((ent <= math.log(V) + 1e-4).all())
    o_lp, o_ent, o_dh, o_dw = _oracle_slice(case, idx, g_slice)
    assert_within(lp[idx], o_lp, 2e-3, "log-prob")  # stated tolerance
    assert_within(ent[idx], o_ent, 2e-3, "entropy")
    assert cosine(dh_only[idx].cpu().float(), o_dh) > 0.9999
    assert_same_magnitude(dh_only[idx], o_dh, what="d(hidden)")
    assert float(dh_only.float().abs().sum()) == pytest.approx(float(dh_only[idx].float().abs().sum()), rel=1e-6)
    # the full-size weight gradient with only the slice's tokens switched on is the oracle's slice gradient
    assert _cos_dev(dw_only, o_dw, device) > 0.9999
    assert abs(float(dw_only.float().norm()) / float(o_dw.norm()) - 1.0) < 1e-2
    del o_dw
    # determinism and linearity of d(W), d(hidden) in the upstream gradient
    lp2, ent2, dh_rest, dw_rest = run(g_rest)
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2)
    _, _, dh_all, dw_all = run(g_rest + g_only)
    assert _cos_dev(dw_rest.float() + dw_only.float(), dw_all, device) > 0.9999
    assert _cos_dev(dh_rest.float() + dh_only.float(), dh_all, device) > 0.9999
    _, _, dh_again, dw_again = run(g_rest + g_only)
    assert torch.equal(dh_all, dh_again) and torch.equal(dw_all, dw_again)


@pytest.mark.parametrize("T,H,V", [(300, 128, 1088), (CHUNK + 72, 64, 640)])  # one chunk; two chunks
def test_weight_gradient_dtypes_through_the_c_abi(device, T, H, V):
    """aa_lmhead_bwd with d_weight as fp32 and as bf16: the fp32 result against autograd of the oracle, and the bf16
    result equal to it up to one rounding (the sum over tokens is kept in fp32 in both)."""
    import ctypes as C

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    hidden, weight, labels = _case(T, H, V, seed=T + H, w_std=0.3)
    g = torch.Generator().manual_seed(1)
    gl = torch.randn(T, generator=g) / T
    h_o = hidden.float().requires_grad_(True)
    w_o = weight.float().requires_grad_(True)
    o_lp, _ = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), labels)
    (o_lp * gl).sum().backward()

    hd, wd, ld, gd = hidden.to(device), weight.to(device), labels.to(device), gl.to(device)
    f32 = dict(dtype=torch.float32, device=device)
    logp, ent, lse, ez = (torch.empty(T, **f32) for _ in range(4))
    ws = F._lmhead_workspace(T, H, V, device)
    st = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    N.check(lib.aa_lmhead_fwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(logp), F._ptr(ent), F._ptr(lse),
                              F._ptr(ez), None, None, F._ptr(ws), ws.numel(), st), "aa_lmhead_fwd")
    out = {}
    for dt, code in ((torch.float32, N.AA_F32), (torch.bfloat16, N.AA_BF16)):
        dh = torch.empty_like(hd)
        dw = torch.full((V, H), float("nan"), dtype=dt, device=device)
        N.check(lib.aa_lmhead_bwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(lse), F._ptr(ez), F._ptr(gd),
                                  None, None, None, F._ptr(dh), F._ptr(dw), code, F._ptr(ws), ws.numel(), st), "aa_lmhead_bwd")
        out[dt] = (dh.cpu().float(), dw.cpu().float())
    dh32, dw32 = out[torch.float32]
    dh16, dw16 = out[torch.bfloat16]
    assert cosine(dw32, w_o.grad) > 0.9999 and cosine(dh32, h_o.grad) > 0.9999
    assert torch.equal(dh32, dh16)
    scale = float(dw32.abs().max())
    assert float((dw16 - dw32).abs().max()) <= scale * 2.0 ** -8 * 1.01     # half a bf16 step at the largest magnitude
    assert cosine(dw16, dw32) > 0.99999
    # an unknown dtype code is refused
    rc = lib.aa_lmhead_bwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(lse), F._ptr(ez), F._ptr(gd), None,
                           None, None, F._ptr(dh), F._ptr(dw), N.AA_F16, F._ptr(ws), ws.numel(), st)
    assert rc == 2  # AA_ERR_UNSUPPORTED


def test_backward_leaves_out_rows_without_gradient(device):
    """lm_head_logprobs_entropy backward with many zero upstream gradients (two chunks, one of them all zero) against
    the same call through the C ABI with every row multiplied through."""
    import ctypes as C

    from areal_amd import _native as N
    from areal_amd import functional as F

    T, H, V = CHUNK + 520, 64, 1088
    hidden, weight, labels = _case(T, H, V, seed=77, w_std=0.3)
    g = torch.Generator().manual_seed(78)
    gl = torch.randn(T, generator=g) * (torch.rand(T, generator=g) < 0.4)
    gh = 0.2 * torch.randn(T, generator=g) * (torch.rand(T, generator=g) < 0.1)
    gl[CHUNK:] = 0.0
    gh[CHUNK:] = 0.0                                   # the second chunk has no gradient at all
    h_d = hidden.to(device).requires_grad_(True)
    w_d = weight.to(device).requires_grad_(True)
    lp, ent = areal_amd.lm_head_logprobs_entropy(h_d, w_d, labels.to(device))
    ((lp * gl.to(device)).sum() + (ent * gh.to(device)).sum()).backward()
    # dense reference through the C ABI
    lib = N.load()
    hd, wd, ld = hidden.to(device), weight.to(device), labels.to(device)
    f32 = dict(dtype=torch.float32, device=device)
    logp, e, lse, ez = (torch.empty(T, **f32) for _ in range(4))
    ws = F._lmhead_workspace(T, H, V, device)
    st = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    N.check(lib.aa_lmhead_fwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(logp), F._ptr(e), F._ptr(lse),
                              F._ptr(ez), None, None, F._ptr(ws), ws.numel(), st), "aa_lmhead_fwd")
    dh, dw = torch.empty_like(hd), torch.empty_like(wd)
    gld, ghd = gl.to(device), gh.to(device)
    N.check(lib.aa_lmhead_bwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(lse), F._ptr(ez), F._ptr(gld),
                              F._ptr(ghd), None, None, F._ptr(dh), F._ptr(dw), N.AA_BF16, F._ptr(ws), ws.numel(), st),
            "aa_lmhead_bwd")
    off = ((gl == 0) & (gh == 0)).to(device)
    assert float(h_d.grad[off].float().abs().max()) == 0.0 and float(dh[off].float().abs().max()) == 0.0
    for a, b in ((h_d.grad.float(), dh.float()), (w_d.grad.float(), dw.float())):
        assert float((a - b).abs().max()) <= float(b.abs().max()) * 2.0 ** -7
        assert cosine(a.cpu(), b.cpu()) > 0.99999
    # mismatched pair of arguments
    rc = lib.aa_lmhead_bwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(lse), F._ptr(ez), F._ptr(gld),
                           F._ptr(ghd), F._ptr(off.view(torch.uint8)), None, F._ptr(dh), F._ptr(dw), N.AA_BF16, F._ptr(ws),
                           ws.numel(), st)
    assert rc == 1  # AA_ERR_INVALID_ARGUMENT


def test_token_mask_runs_only_the_selected_tokens(device):
    T, H, V = 700, 128, 1088
    hidden, weight, labels = _case(T, H, V, seed=91, w_std=0.3)
    g = torch.Generator().manual_seed(92)
    sel = torch.rand(T, generator=g) < 0.4
    gl = torch.randn(T, generator=g)
    hd, wd, ld = hidden.to(device), weight.to(device), labels.to(device)
    h0, w0 = hd.clone().requires_grad_(True), wd.clone().requires_grad_(True)
    lp0, ent0 = areal_amd.lm_head_logprobs_entropy(h0, w0, ld, 0.9)
    ((lp0 * gl.to(device) + 0.1 * ent0) * sel.to(device)).sum().backward()
    h1, w1 = hd.clone().requires_grad_(True), wd.clone().requires_grad_(True)
    lp1, ent1 = areal_amd.lm_head_logprobs_entropy(h1, w1, ld, 0.9, token_mask=sel.to(device))
    (lp1 * gl.to(device) + 0.1 * ent1).sum().backward()
    s = sel.to(device)
    assert torch.allclose(lp1[s], lp0[s].detach(), atol=1e-6) and torch.allclose(ent1[s], ent0[s].detach(), atol=1e-6)
    assert float(lp1.detach()[~s].abs().sum()) == 0.0 and float(ent1.detach()[~s].abs().sum()) == 0.0
    assert cosine(h1.grad.cpu(), h0.grad.cpu()) > 0.99999 and cosine(w1.grad.cpu(), w0.grad.cpu()) > 0.99999
    assert float(h1.grad[~s].float().abs().sum()) == 0.0
    none = torch.zeros(T, dtype=torch.bool, device=device)
    lp2, ent2 = areal_amd.lm_head_logprobs_entropy(hd, wd, ld, token_mask=none)
    assert float(lp2.abs().sum()) == 0.0 and lp2.shape == (T,)


def test_row_counts_that_disagree_with_the_mask_stay_in_bounds(device):
    """kept_per_chunk comes from the host.  Too small: the rows beyond it count as rows without gradient.  Too large:
    the result is meaningless but every access stays inside the buffers (the call returns, the device stays usable)."""
    import ctypes as C

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    T, H, V = 900, 64, 1088
    hidden, weight, labels = _case(T, H, V, seed=5, w_std=0.3)
    hd, wd, ld = hidden.to(device), weight.to(device), labels.to(device)
    g = torch.Generator().manual_seed(6)
    gl = (torch.randn(T, generator=g) * (torch.rand(T, generator=g) < 0.5)).to(device)
    f32 = dict(dtype=torch.float32, device=device)
    logp, e, lse, ez = (torch.empty(T, **f32) for _ in range(4))
    ws = F._lmhead_workspace(T, H, V, device)
    st = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    N.check(lib.aa_lmhead_fwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(logp), F._ptr(e), F._ptr(lse),
                              F._ptr(ez), None, None, F._ptr(ws), ws.numel(), st), "aa_lmhead_fwd")
    has = (gl != 0)
    n = int(has.sum())

    def run(g_vec, rows, count):
        dh, dw = torch.empty_like(hd), torch.empty_like(wd)
        N.check(lib.aa_lmhead_bwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(lse), F._ptr(ez), F._ptr(g_vec),
                                  None, F._ptr(rows.view(torch.uint8)), (C.c_int64 * 1)(count), F._ptr(dh), F._ptr(dw),
                                  N.AA_BF16, F._ptr(ws), ws.numel(), st), "aa_lmhead_bwd")
        torch.cuda.synchronize()
        return dh.float(), dw.float()

    dh_small, dw_small = run(gl, has, n - 5)
    last5 = has.nonzero().squeeze(-1)[-5:]
    gl_cut = gl.clone()
    gl_cut[last5] = 0.0
    dh_ref, dw_ref = run(gl_cut, gl_cut != 0, n - 5)
    assert torch.equal(dh_small, dh_ref) and torch.equal(dw_small, dw_ref)
    run(gl, has, n + 7)                                   # must simply come back
    dh_ok, _ = run(gl, has, n)
    assert bool(torch.isfinite(dh_ok).all()) and float(dh_ok[~has].abs().sum()) == 0.0


def test_forward_needs_no_panel(device):
    """The forward writes nothing of size T x V: its workspace is the softmax partials only, and it runs with exactly
    that much."""
    import ctypes as C

    from areal_amd import _native as N
    from areal_amd import functional as F

    lib = N.load()
    T, H, V = 16384, 4096, 151936
    assert lib.aa_lmhead_fwd_workspace_bytes(T, H, V) < 0.05 * (2 * T * V)          # bf16 logits would be 2 T V bytes
    assert lib.aa_lmhead_fwd_workspace_bytes(T, H, V) < lib.aa_lmhead_workspace_bytes(T, H, V) / 20
    T, H, V = 600, 128, 1088
    hidden, weight, labels = _case(T, H, V, seed=3, w_std=0.3)
    hd, wd, ld = hidden.to(device), weight.to(device), labels.to(device)
    n = lib.aa_lmhead_fwd_workspace_bytes(T, H, V)
    ws = torch.empty(n, dtype=torch.uint8, device=device)
    f32 = dict(dtype=torch.float32, device=device)
    logp, ent = torch.empty(T, **f32), torch.empty(T, **f32)
    st = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    N.check(lib.aa_lmhead_fwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(logp), F._ptr(ent), None, None,
                              None, None, F._ptr(ws), n, st), "aa_lmhead_fwd")
    r_lp, r_ent = oracle.logprobs_entropy_f64(oracle.lmhead_logits(hidden, weight), labels, 1.0)
    assert_within(logp, r_lp, 2e-3, "log-prob")
    assert_within(ent, r_ent, 2e-3, "entropy")
    assert lib.aa_lmhead_fwd(F._ptr(hd), F._ptr(wd), T, H, V, F._ptr(ld), 1.0, F._ptr(logp), F._ptr(ent), None, None,
                             None, None, F._ptr(ws), n - 1, st) == 1                                # AA_ERR_INVALID_ARGUMENT


@pytest.mark.parametrize("T,H,V,temperature", [(300, 128, 1088, 1.0), (203, 72, 1097, 0.7), (CHUNK + 70, 64, 640, 1.3)])
def test_vocabulary_extrema_of_the_logits(device, T, H, V, temperature):
    """vocab_min_logits / vocab_max_logits, which the engine reads from materialised logits and hands to the loss
    function (areal/engine/fsdp_engine.py:1893-1906), here from the tiles: extrema of the raw (not temperature-scaled)
    fp32 logits.  Tolerance: the order of the fp32 accumulation (1e-5 of the largest logit)."""
    hidden, weight, labels = _case(T, H, V, seed=3 * T + V, w_std=0.3)
    lp, ent, vmin, vmax = areal_amd.lm_head_logprobs_entropy_stats(
        hidden.to(device), weight.to(device), labels.to(device), temperature)
    logits = oracle.lmhead_logits(hidden, weight)
    scale = float(logits.abs().max())
    assert float((vmax.cpu() - logits.max(-1).values).abs().max()) <= 1e-5 * scale
    assert float((vmin.cpu() - logits.min(-1).values).abs().max()) <= 1e-5 * scale
    assert not vmin.requires_grad and not vmax.requires_grad
    lp2, ent2 = areal_amd.lm_head_logprobs_entropy(hidden.to(device), weight.to(device), labels.to(device), temperature)
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2)  # asking for the extrema changes nothing else


# ---------------------------------------------------------------------------------------------------------------
# backward="carry" of the stand-alone op: the forward keeps p_v / p_label of the tokens that may get a gradient, the
# backward is two plain GEMMs (aa_lmhead_fwd_carry / aa_lmhead_bwd_carry).  Same oracle, same tolerances.
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,H,V,temperature,with_mask,counts_from_host", [
    (300, 128, 1088, 1.0, True, False),
    (203, 72, 1097, 0.7, True, True),          # vocabulary no multiple of 8
    (CHUNK + 200, 64, 640, 1.3, True, True),   # two token chunks
    (CHUNK + 72, 64, 640, 1.0, False, False),  # every token kept
    (300, 128, 16643, 1.0, True, False),       # d(hidden) cut into parts along the vocabulary
])
def test_carried_backward_matches_autograd_of_oracle(device, T, H, V, temperature, with_mask, counts_from_host):
    hidden, weight, labels = _case(T, H, V, seed=5 * T + V, w_std=0.3)
    g = torch.Generator().manual_seed(3)
    mask = (torch.rand(T, generator=g) < 0.6) if with_mask else torch.ones(T, dtype=torch.bool)
    gl = torch.randn(T, generator=g) * mask.float()
    gl[::7] = 0.0                                  # a named token may still have no gradient
    kept = [int(mask[i:i + CHUNK].sum()) for i in range(0, T, CHUNK)] if counts_from_host else None

    def run(backward):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        lp, ent = areal_amd.lm_head_logprobs_entropy(
            h, w, labels.to(device), temperature, backward=backward,
            grad_token_mask=mask.to(device) if with_mask else None, kept_per_chunk=kept if backward == "carry" else None)
        (lp * gl.to(device)).sum().backward()
        return lp.detach(), ent.detach(), h.grad, w.grad

    lp_c, ent_c, dh_c, dw_c = run("carry")
    lp_r, ent_r, dh_r, dw_r = run("recompute")
    assert torch.equal(lp_c, lp_r) and torch.equal(ent_c, ent_r)     # the same tiles, the same merge
    h_o = hidden.float().requires_grad_(True)
    w_o = weight.float().requires_grad_(True)
    o_lp, _ = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), labels, temperature)
    (o_lp * gl).sum().backward()
    assert_within(lp_c, o_lp.detach(), 2e-3, "log-prob")
    for name, got, other, want in (("d(hidden)", dh_c, dh_r, h_o.grad), ("d(W)", dw_c, dw_r, w_o.grad)):
        assert got.dtype == torch.bfloat16
        assert cosine(got.cpu(), want) > 0.9999, name
        assert_same_magnitude(got, want, what=name)
        assert cosine(got.cpu().float(), other.cpu().float()) > 0.99999, name
    assert float(dh_c[~mask.to(device)].float().abs().sum()) == 0.0   # tokens outside the mask: no gradient


def test_carried_backward_edge_cases(device):
    T, H, V = 400, 64, 1088
    hidden, weight, labels = _case(T, H, V, seed=77, w_std=0.3)
    g = torch.Generator().manual_seed(1)
    gl, gh = torch.randn(T, generator=g), 0.3 * torch.randn(T, generator=g)
    args = (hidden.to(device), weight.to(device), labels.to(device))

    def grads(backward, with_entropy, **kw):
        h, w = args[0].clone().requires_grad_(True), args[1].clone().requires_grad_(True)
        lp, ent = areal_amd.lm_head_logprobs_entropy(h, w, args[2], 0.9, backward=backward, **kw)
        obj = (lp * gl.to(device)).sum() + ((ent * gh.to(device)).sum() if with_entropy else 0.0)
        obj.backward(retain_graph=True)
        return h, w, obj

    # an entropy gradient is no multiple of the stored rows: the backward forms the logits again, same bits as recompute
    hc, wc, _ = grads("carry", True)
    hr, wr, _ = grads("recompute", True)
    assert torch.equal(hc.grad, hr.grad) and torch.equal(wc.grad, wr.grad)
    # the stored rows serve one backward
    _, _, obj = grads("carry", False)
    with pytest.raises(RuntimeError, match="already used by a backward"):
        obj.backward()
    # no gradient asked for: the plain forward, nothing kept
    with torch.no_grad():
        lp, _ = areal_amd.lm_head_logprobs_entropy(*args, 0.9, backward="carry")
    assert not lp.requires_grad
    # tokens outside grad_token_mask get no gradient even if the loss gives them one
    mask = torch.zeros(T, dtype=torch.bool)
    mask[50:200] = True
    hm, wm, _ = grads("carry", False, grad_token_mask=mask.to(device))
    assert float(hm.grad[:50].float().abs().sum()) == 0.0 and float(hm.grad[200:].float().abs().sum()) == 0.0
    assert float(hm.grad[50:200].float().abs().sum()) > 0.0
    with pytest.raises(ValueError, match="backward must be one of"):
        areal_amd.lm_head_logprobs_entropy(*args, backward="panel")


def test_carried_backward_redoes_a_chunk_that_does_not_fit(device):
    """Labels with a log-prob below -80 in the first chunk: its rows are redone from the logits tiles (decided on the
    device); the second chunk stays on the carried rows.  Both against the oracle and against recompute."""
    T, H, V = CHUNK + 300, 64, 1088
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(T, H, generator=g)
    hidden[:CHUNK] *= 12.0
    hidden = hidden.bfloat16()
    weight = (0.5 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    ref_lp = oracle.logprobs(oracle.lmhead_logits(hidden, weight), labels)
    assert int((ref_lp[:CHUNK] < -80).sum()) > 100 and float(ref_lp[CHUNK:].min()) > -60
    mask = torch.rand(T, generator=g) < 0.7
    gl = torch.randn(T, generator=g) * mask.float()

    def run(backward):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        lp, _ = areal_amd.lm_head_logprobs_entropy(h, w, labels.to(device), backward=backward,
                                                   grad_token_mask=mask.to(device))
        (lp * gl.to(device)).sum().backward()
        return h.grad.float(), w.grad.float()

    got, ref = run("carry"), run("recompute")
    h_o = hidden.float().requires_grad_(True)
    w_o = weight.float().requires_grad_(True)
    o_lp, _ = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), labels)
    (o_lp * gl).sum().backward()
    for name, a, b, o in (("d(hidden)", got[0], ref[0], h_o.grad), ("d(W)", got[1], ref[1], w_o.grad)):
        assert torch.isfinite(a).all(), name
        assert cosine(a.cpu(), o) > 0.9999, name
        assert_same_magnitude(a, o, what=name)
    assert torch.equal(got[0][:CHUNK], ref[0][:CHUNK])   # the redone chunk: the rows of the recompute mode, bit for bit


@pytest.mark.parametrize("T,H,V,density", [
    (300, 128, 1088, 0.6),
    (CHUNK + 200, 64, 640, 0.6),       # two token chunks: the second one's rows start a whole chunk further on
    (CHUNK + 200, 64, 8256, 0.004),    # a handful of rows: d(hidden) is cut along the vocabulary, chosen on the device
    (CHUNK + 200, 64, 640, 0.0),       # no token named at all
])
def test_carried_backward_with_the_rows_counted_on_the_device(device, T, H, V, density):
    """``count_on_device=True``: nothing is read back, the stored rows keep room for every token and the kernels stop
    at the rows in use.  The same log-probs and d(hidden) bits as with the counts read back, d(W) up to the order of
    the sums (the rows of a chunk are the same, in the same order), and both against the oracle."""
    hidden, weight, labels = _case(T, H, V, seed=3 * T + V, w_std=0.3)
    g = torch.Generator().manual_seed(9)
    mask = torch.rand(T, generator=g) < density
    gl = torch.randn(T, generator=g) * mask.float()

    def run(**kw):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        lp, _ = areal_amd.lm_head_logprobs_entropy(h, w, labels.to(device), 0.9, backward="carry",
                                                   grad_token_mask=mask.to(device), **kw)
        (lp * gl.to(device)).sum().backward()
        return lp.detach(), h.grad, w.grad

    on_device, read_back = run(count_on_device=True), run()
    assert torch.equal(on_device[0], read_back[0]) and torch.equal(on_device[1], read_back[1])
    assert torch.isfinite(on_device[2].float()).all()
    if mask.any():
        assert cosine(on_device[2].float().cpu(), read_back[2].float().cpu()) > 0.9999999
        assert_same_magnitude(on_device[2].float(), read_back[2].float(), rel=1e-4)
        h_o = hidden.float().requires_grad_(True)
        w_o = weight.float().requires_grad_(True)
        o_lp, _ = oracle.logprobs_entropy(oracle.lmhead_logits(h_o, w_o), labels, 0.9)
        (o_lp * gl).sum().backward()
        assert cosine(on_device[1].cpu(), h_o.grad) > 0.9999 and cosine(on_device[2].cpu(), w_o.grad) > 0.9999
        assert_same_magnitude(on_device[1], h_o.grad, what="d(hidden)")
        assert_same_magnitude(on_device[2], w_o.grad, what="d(W)")
    else:
        assert float(on_device[1].float().abs().max()) == 0.0 and float(on_device[2].float().abs().max()) == 0.0


def test_carried_backward_redoes_a_chunk_with_the_rows_counted_on_the_device(device):
    """The chunk that does not fit the stored form is redone from the logits tiles over the rows in use only; the
    rows of the recompute mode, bit for bit."""
    T, H, V = CHUNK + 300, 64, 1088
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(T, H, generator=g)
    hidden[:CHUNK] *= 12.0
    hidden = hidden.bfloat16()
    weight = (0.5 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    mask = torch.rand(T, generator=g) < 0.3
    gl = torch.randn(T, generator=g) * mask.float()

    def run(backward, **kw):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        lp, _ = areal_amd.lm_head_logprobs_entropy(h, w, labels.to(device), backward=backward,
                                                   grad_token_mask=mask.to(device), **kw)
        (lp * gl.to(device)).sum().backward()
        return h.grad.float(), w.grad.float()

    got, host, ref = run("carry", count_on_device=True), run("carry"), run("recompute")
    assert torch.isfinite(got[0]).all() and torch.isfinite(got[1]).all()
    assert torch.equal(got[0], host[0]) and torch.equal(got[0][:CHUNK], ref[0][:CHUNK])
    assert cosine(got[1].cpu(), host[1].cpu()) > 0.9999999
    assert_same_magnitude(got[1], host[1], rel=1e-4)


def test_sequence_level_step_reads_nothing_back(device):
    """GSPO through the lm_head (``fused_lm_head_ppo_loss(importance_sampling_level="sequence")``): the op keeps its
    rows with the count on the device (default) or read back; same loss, same gradients."""
    T, H, V = 700, 64, 1088
    hidden, weight, labels = _case(T, H, V, seed=21, w_std=0.3)
    g = torch.Generator().manual_seed(2)
    ref = oracle.logprobs(oracle.lmhead_logits(hidden, weight), labels)
    prox, old = ref + 0.05 * torch.randn(T, generator=g), ref + 0.05 * torch.randn(T, generator=g)
    adv = torch.randn(T, generator=g)
    mask = torch.rand(T, generator=g) < 0.5
    cu = torch.tensor([0, 130, 400, 700], dtype=torch.int32, device=device)

    def run(**kw):
        h = hidden.to(device).requires_grad_(True)
        w = weight.to(device).requires_grad_(True)
        loss, _ = areal_amd.fused_lm_head_ppo_loss(h, w, labels.to(device), prox.to(device), old.to(device), adv.to(device),
                                                   eps_clip=0.2, loss_mask=mask.to(device), cu_seqlens=cu,
                                                   importance_sampling_level="sequence", **kw)
        loss.backward()
        return loss.detach(), h.grad, w.grad

    a, b = run(), run(count_on_device=False)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert cosine(a[2].float().cpu(), b[2].float().cpu()) > 0.9999999
    assert float(a[1].float().abs().sum()) > 0.0
