"""Shared comparison helpers for the parity tests."""
import torch


def check_partial(actual: torch.Tensor, expected, atol=1e-5, rtol=1e-5, exact=False):
    """Compare ``actual`` with a nested list that may hold ``None`` for entries nobody asserts."""
    flat_a = actual.detach().cpu().reshape(-1).tolist()

    def flatten(x):
        if isinstance(x, list):
            for v in x:
                yield from flatten(v)
        else:
            yield x

    flat_e = list(flatten(expected))
    assert len(flat_a) == len(flat_e), (len(flat_a), len(flat_e))
    for i, (a, e) in enumerate(zip(flat_a, flat_e)):
        if e is None:
            continue
        if exact:
            assert a == e, f"entry {i}: {a} != {e}"
        else:
            assert abs(a - e) <= atol + rtol * abs(e), f"entry {i}: {a} vs {e}"


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.double().reshape(-1)
    b = b.double().reshape(-1)
    den = a.norm() * b.norm()
    if den == 0:
        return 1.0 if a.norm() == b.norm() else 0.0
    return float((a @ b) / den)


def assert_within(got: torch.Tensor, want: torch.Tensor, tol: float = 2e-3, what: str = ""):
    """Every entry of ``got`` within ``tol`` (absolute) of ``want``."""
    err = (got.detach().double().cpu() - want.detach().double().cpu()).abs().reshape(-1)
    if err.numel():
        assert float(err.max()) < tol, f"{what}: worst entry off by {float(err.max())} (allowed {tol})"


def assert_within_one_bf16_logit_step(got: torch.Tensor, want: torch.Tensor, logit_scale: float, what: str = ""):
    """Per-token quantities of the lm_head path (fp32 logits tiles) against the reference pipeline whose lm_head
    output is rounded to bf16: that rounding moves a logit by up to 2^-8 of its magnitude (half a bf16 step), the label
    logit and the row's logsumexp each by at most that much, so no token may be further off than twice that at the
    largest logit."""
    err = (got.detach().double().cpu() - want.detach().double().cpu()).abs().reshape(-1)
    if err.numel() == 0:
        return
    assert float(err.max()) <= logit_scale * 2.0 ** -7, f"{what}: worst token off by {float(err.max())}"


def assert_same_magnitude(got: torch.Tensor, want: torch.Tensor, rel: float = 1e-2, what: str = ""):
    """Norm ratio within ``rel`` and every entry within one bf16 step of the largest one: catches a wrong global factor
    (1/n, a loss scale, a temperature), which a cosine cannot see."""
    a, b = got.detach().double().cpu().reshape(-1), want.detach().double().cpu().reshape(-1)
    nb = float(b.norm())
    if nb == 0.0:
        assert float(a.norm()) == 0.0, f"{what}: expected all zeros"
        return
    assert abs(float(a.norm()) / nb - 1.0) < rel, f"{what}: norm ratio {float(a.norm()) / nb}"
    assert float((a - b).abs().max()) <= float(b.abs().max()) * 2.0 ** -7 + 1e-12, f"{what}: entry off by {float((a - b).abs().max())}"


class Cfg:
    """Attribute bag standing in for a rejection-sampling config in oracle calls."""

    def __init__(self, level="token", action="mask", metric="ratio", agg="mean", upper=5.0, lower=None):
        self.level, self.action, self.metric, self.agg, self.upper, self.lower = level, action, metric, agg, upper, lower
        if action == "clamp" and lower is None:
            self.lower = 0.0
