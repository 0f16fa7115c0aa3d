"""Error metrics shared by the parity tests."""
import os

import torch

# Acceptance tolerances: bf16 outputs and fp32 states against the fp32 oracle.
TOL_BF16 = 2e-2
TOL_STATE = 1e-3


# (test id, tensor name, tolerance asked for, measured statistics) of every assert_close of the session; conftest.py
# writes them out at the end of a GPU run so that the margins to the bounds are on record.
RECORDS = []


def err_stats(actual: torch.Tensor, expected: torch.Tensor):
    a, e = actual.detach().float().cpu(), expected.detach().float().cpu()
    diff = (a - e).abs()
    scale = e.abs().max().clamp_min(1e-30)
    return dict(max_abs=float(diff.max()), max_ref=float(scale), rel_max=float(diff.max() / scale),
                rms_rel=float(diff.pow(2).mean().sqrt() / e.pow(2).mean().sqrt().clamp_min(1e-30)))


def assert_close(actual, expected, tol, name="tensor"):
    """|a - e| <= tol + tol * |e| element-wise (the reference's allclose(rtol=tol, atol=tol) form,
    examples/flash_gated_delta_rule.py:1738-1761) and max error <= tol * max|e| + tol."""
    a, e = actual.detach().float().cpu(), expected.detach().float().cpu()
    assert a.shape == e.shape, f"{name}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    assert torch.isfinite(a).all(), f"{name}: non-finite values"
    st = err_stats(a, e)
    RECORDS.append(dict(test=os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0], name=name, tol=tol, **st))
    ok = torch.allclose(a, e, rtol=tol, atol=tol)
    assert ok, f"{name}: not within tol={tol}: {st}"
    return st
