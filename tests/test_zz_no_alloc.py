"""aa_lmhead_fwd_static, the forward of the lm_head path for callers that cannot allocate, called through the C-ABI
and held against aa_lmhead_fwd on the same inputs.  Both run the same kernels over the same per-token arithmetic (only
the home of the softmax partials and the number of tokens per pass differ), so the outputs must be bit-equal; the
oracle's 2e-3 bound on every token is checked as well.  Two calls in a row, the second smaller: the library's array
keeps the first call's contents and nothing of them may leak into the second."""
import ctypes

import pytest
import torch

import oracle
from areal_amd import _native as N
from helpers import assert_within

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _case(T, H, V, seed, device):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    return hidden.to(device), weight.to(device), labels.to(device)


def _outputs(T, device):
    # NaN-filled so that an element the library does not write shows
    return [torch.full((T,), float("nan"), dtype=torch.float32, device=device) for _ in range(4)]


def _fwd(lib, hidden, weight, labels, inv_t):
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    n = lib.aa_lmhead_fwd_workspace_bytes(T, H, V)
    assert n > 0
    ws = torch.empty(n, dtype=torch.uint8, device=dev)
    out = _outputs(T, dev)
    N.check(lib.aa_lmhead_fwd(_ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), inv_t, *[_ptr(o) for o in out], None, None,
                              _ptr(ws), ws.numel(), _stream(dev)), "aa_lmhead_fwd")
    return out


def _fwd_static(lib, hidden, weight, labels, inv_t):
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    out = _outputs(T, dev)
    N.check(lib.aa_lmhead_fwd_static(_ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), inv_t, *[_ptr(o) for o in out],
                                     _stream(dev)), "aa_lmhead_fwd_static")
    return out


def _check(lib, T, H, V, seed, temperature, device):
    hidden, weight, labels = _case(T, H, V, seed, device)
    inv_t = 1.0 / temperature
    got = _fwd_static(lib, hidden, weight, labels, inv_t)
    want = _fwd(lib, hidden, weight, labels, inv_t)
    torch.cuda.synchronize(device)
    for name, g, w in zip(("logp", "entropy", "row_lse", "row_ez"), got, want):
        assert not torch.isnan(g).any(), name
        assert torch.equal(g, w), f"{name}: max |diff| {float((g - w).abs().max())}"
    r_lp, r_ent = oracle.logprobs_entropy_f64(oracle.lmhead_logits(hidden.cpu(), weight.cpu()), labels.cpu(), temperature)
    assert_within(got[0], r_lp, 2e-3, "log-prob")
    assert_within(got[1], r_ent, 2e-3, "entropy")


def test_two_calls_in_a_row_second_smaller(device):
    lib = N.load()
    with torch.cuda.device(device):
        # V = 151936 leaves room for 2304 tokens a pass: 5000 tokens take three passes, the last of them ragged
        _check(lib, 5000, 128, 151936, seed=1, temperature=1.0, device=device)
        _check(lib, 300, 192, 1088, seed=2, temperature=0.7, device=device)
        _check(lib, 37, 64, 576, seed=3, temperature=1.3, device=device)


def test_sizes_beyond_the_array_are_refused(device):
    lib = N.load()
    assert lib.aa_lmhead_fwd_static_scratch_bytes() == 32 << 20
    v_max = lib.aa_lmhead_fwd_static_max_vocab()
    assert v_max == 1398016
    T, H, V = 8, 8, v_max + 8
    with torch.cuda.device(device):
        hidden = torch.zeros(T, H, dtype=torch.bfloat16, device=device)
        weight = torch.zeros(V, H, dtype=torch.bfloat16, device=device)
        labels = torch.zeros(T, dtype=torch.int64, device=device)
        out = _outputs(T, device)
        rc = lib.aa_lmhead_fwd_static(_ptr(hidden), _ptr(weight), T, H, V, _ptr(labels), 1.0, *[_ptr(o) for o in out],
                                      _stream(device))
        assert rc == N.AA_ERR_UNSUPPORTED
        with pytest.raises(N.NativeLibraryError, match="aa_lmhead_fwd_static"):
            N.check(rc, "aa_lmhead_fwd_static")
        torch.cuda.synchronize(device)
        assert all(torch.isnan(o).all() for o in out)  # nothing was launched
        # the largest vocabulary it takes: zero weights make every row uniform over V
        weight = torch.zeros(v_max, H, dtype=torch.bfloat16, device=device)
        N.check(lib.aa_lmhead_fwd_static(_ptr(hidden), _ptr(weight), T, H, v_max, _ptr(labels), 1.0,
                                         *[_ptr(o) for o in out], _stream(device)), "aa_lmhead_fwd_static")
        torch.cuda.synchronize(device)
        import math

        assert torch.allclose(out[0], torch.full_like(out[0], -math.log(v_max)), atol=1e-5)
        assert torch.allclose(out[1], torch.full_like(out[1], math.log(v_max)), atol=1e-5)
