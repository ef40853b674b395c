"""Shared helpers for the GPU parity tests: one context per session, numpy <-> device moves."""
import numpy as np
import pytest

_ctx = None


def ctx():
    """The process-wide argus_hip context (created on first use; needs a GPU)."""
    global _ctx
    if _ctx is None:
        import argus_hip
        _ctx = argus_hip.Context(0)
    return _ctx


_env_ctx = {}


def env_ctx(name, value):
    """A context created under the environment switch `name=value` (switches are read at creation)."""
    key = (name, value)
    if key not in _env_ctx:
        import os
        import argus_hip
        old = os.environ.get(name)
        os.environ[name] = value
        try:
            _env_ctx[key] = argus_hip.Context(0)
        finally:
            if old is None:
                del os.environ[name]
            else:
                os.environ[name] = old
    return _env_ctx[key]


_direct_ctx = None


def direct_ctx():
    """A second context created under ARGUS_HIP_SCORES=direct (the switches are read when a context
    is created): its score-emitting decode calls store their logits from inside the token loop."""
    global _direct_ctx
    if _direct_ctx is None:
        import os
        import argus_hip
        old = os.environ.get("ARGUS_HIP_SCORES")
        os.environ["ARGUS_HIP_SCORES"] = "direct"
        try:
            _direct_ctx = argus_hip.Context(0)
        finally:
            if old is None:
                del os.environ["ARGUS_HIP_SCORES"]
            else:
                os.environ["ARGUS_HIP_SCORES"] = old
    return _direct_ctx


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.cpu().numpy()


def normal(shape, seed, dtype=np.float32):
    return np.random.default_rng(seed).standard_normal(shape, dtype=np.float32).astype(dtype)


def check_attention_out(got, ref, what=""):
    """Required tolerance for attention outputs: <= 2e-3 max-abs and <= 1e-3 mean-abs."""
    diff = np.abs(np.asarray(got, np.float64) - np.asarray(ref, np.float64))
    assert np.all(np.isfinite(got)), what
    assert diff.max() <= 2e-3, "%s max-abs %g" % (what, diff.max())
    assert diff.mean() <= 1e-3, "%s mean-abs %g" % (what, diff.mean())
    return diff.max()


def check_scores(got, ref, what=""):
    """Required tolerance for H2O score vectors: <= 1e-4 relative (element-wise, with an
    absolute floor at the f32 underflow scale of a softmax over <= 64K tokens)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    err = np.abs(got - ref)
    tol = 1e-4 * np.abs(ref) + 1e-12
    bad = err > tol
    assert not bad.any(), "%s: %d scores off, worst rel %g" % (
        what, bad.sum(), (err / np.maximum(np.abs(ref), 1e-30)).max())
