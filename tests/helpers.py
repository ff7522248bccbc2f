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


def assert_close_up_to_logit_rounding(got: torch.Tensor, want: torch.Tensor, tol: float = 2e-3, what: str = ""):
    """Per-token quantities of the lm_head path against an oracle that formed its bf16 logits with another GEMM.

    Two fp32 sums of the same products in a different order can land on either side of a bf16 rounding boundary; the
    logit then differs by one bf16 step (2^-8 of its magnitude), and so does the token's log-prob if it is the label.
    With logits of magnitude up to ~8 that is up to 0.03, far above the stated tolerance, for about one token in a
    few thousand.  So: all but a handful of tokens within ``tol``, and no token further off than one bf16 step of a
    logit."""
    err = (got.detach().double().cpu() - want.detach().double().cpu()).abs().reshape(-1)
    if err.numel() == 0:
        return
    allowed = max(2, err.numel() // 200)
    assert int((err >= tol).sum()) <= allowed, f"{what}: {int((err >= tol).sum())} of {err.numel()} tokens beyond {tol}"
    assert float(err.max()) < 0.06, f"{what}: worst token off by {float(err.max())}"
    assert float(err.median()) < tol / 20, f"{what}: median error {float(err.median())}"


class Cfg:
    """Attribute bag standing in for a rejection-sampling config in oracle calls."""

    def __init__(self, level="token", action="mask", metric="ratio", agg="mean", upper=5.0, lower=None):
        self.level, self.action, self.metric, self.agg, self.upper, self.lower = level, action, metric, agg, upper, lower
        if action == "clamp" and lower is None:
            self.lower = 0.0
