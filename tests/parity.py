"""Shared parity check of the GPU tests.

Element-wise closeness alone says little on long rows of random data: with N(0, 1) values and
near-uniform probabilities an output element shrinks like 1/sqrt(kv_len) and falls under any
fixed absolute tolerance (a row of 30000 tokens has elements of ~0.008).  Every comparison with
the oracle therefore also bounds the error of each output row (one query token, one head)
relative to that row's own size:

    || got - want ||_2  <=  rel * || want ||_2

rel = 1e-2 for 16-bit caches and 3e-2 for fp8 caches.  A kernel that drops a tile of a long row,
mixes up a merge weight or mis-scales a partial row changes the row by far more than that.
"""

import torch

BF16_TOL = dict(rtol=2e-2, atol=2e-2)
FP8_TOL = dict(rtol=5e-2, atol=5e-2)
BF16_REL = 1e-2
FP8_REL = 3e-2


def row_rel_error(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    g, w = got.double(), want.double()
    return (g - w).norm(dim=-1) / w.norm(dim=-1).clamp_min(1e-30)


def assert_parity(got, want, *, rtol, atol, rel=None):
    """`got`, `want`: [..., D] outputs; rows are the last dimension."""
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got, want, rtol=rtol, atol=atol)
    if rel is None:
        rel = BF16_REL if atol <= 2e-2 else FP8_REL
    err = row_rel_error(got, want)
    worst = int(err.argmax())
    assert float(err.max()) <= rel, (
        f"row-relative error {float(err.max()):.3e} > {rel:g} at row {worst} of {err.numel()} "
        f"(|want| = {float(want.reshape(-1, want.shape[-1])[worst].norm()):.3e})")
