"""Shared test helpers: a duck-typed gradient bucket and the comparison used for fp32 parity."""
import numpy as np
import torch

REL_TOL = 1e-5   # the parity bar for floating-point results: 1e-5 relative, fp32


class FakeGradBucket:
    """What a DDP GradBucket shows a hook: one flat buffer and per-parameter views into it."""

    def __init__(self, flat, shapes, index=0, is_last=True):
        self._flat, self._shapes, self._index, self._is_last = flat, list(shapes), index, is_last
        self._views = None

    def buffer(self):
        return self._flat

    def gradients(self):
        if self._views is None:          # made once: the reducer's bucket hands its views over without Python work
            out, off = [], 0
            for s in self._shapes:
                c = int(np.prod(s))
                out.append(self._flat[off:off + c].view(*s))
                off += c
            self._views = out
        return list(self._views)

    def index(self):
        return self._index

    def is_last(self):
        return self._is_last


class OldApiGradBucket(FakeGradBucket):
    """Same bucket under the method names the reference hooks call (torch 1.9 pre-release)."""
    buffer = gradients = index = is_last = None

    def get_tensor(self):
        return FakeGradBucket.buffer(self)

    def get_per_parameter_tensors(self):
        return FakeGradBucket.gradients(self)

    def get_index(self):
        return FakeGradBucket.index(self)

    def is_the_last_bucket_to_allreduce(self):
        return FakeGradBucket.is_last(self)


def to_np(t):
    return t.detach().cpu().numpy() if isinstance(t, torch.Tensor) else np.asarray(t)


def assert_close(got, want, rel=REL_TOL, what=""):
    """|got - want| <= rel * max|want| elementwise, and the relative L2 error <= rel.
    Sums whose terms cancel cannot be compared entry by entry in relative terms once the order
    of accumulation differs, hence the norm-wise form."""
    got, want = to_np(got).astype(np.float64), to_np(want).astype(np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all() == np.isfinite(want).all(), what
    scale = np.abs(want).max() if want.size else 0.0
    if scale == 0.0:
        assert np.abs(got).max(initial=0.0) == 0.0, what
        return
    err = np.abs(got - want).max()
    assert err <= rel * scale, "%s: max abs err %.3e > %.1e * %.3e" % (what, err, rel, scale)
    l2 = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert l2 <= rel, "%s: relative L2 error %.3e" % (what, l2)


def heavy_tail_gradient(numel, seed, sigma=1e-3, tail_frac=0.01, tail_scale=1e-2):
    """N(0, sigma^2) with a Bernoulli(tail_frac) mask of Laplace(0, tail_scale) entries."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(numel, generator=g) * sigma
    mask = torch.rand(numel, generator=g) < tail_frac
    u = torch.rand(numel, generator=g) - 0.5
    lap = -tail_scale * torch.sign(u) * torch.log1p(-2 * u.abs())
    return torch.where(mask, lap, x).float()
