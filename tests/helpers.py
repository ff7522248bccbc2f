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


class Cfg:
    """Attribute bag standing in for a rejection-sampling config in oracle calls."""

    def __init__(self, level="token", action="mask", metric="ratio", agg="mean", upper=5.0, lower=None):
        self.level, self.action, self.metric, self.agg, self.upper, self.lower = level, action, metric, agg, upper, lower
        if action == "clamp" and lower is None:
            self.lower = 0.0
