"""Shared helpers for the GPU parity tests (run with -m gpu on an MI355X)."""
import sys

import numpy as np

import foundry_attn as fa

_ctx = None


def ctx():
    """One context per test process."""
    global _ctx
    if _ctx is None:
        _ctx = fa.Foundry(0)
    return _ctx


def announce(*parts):
    """Names the case before any GPU work so a crashed run still shows what was running."""
    print("[case]", *parts, flush=True)
    sys.stdout.flush()


def h16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16)


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))))
