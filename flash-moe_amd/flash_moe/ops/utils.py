"""Small host helpers shared by the ops."""
from __future__ import annotations

import functools

import torch


def next_power_of_2(n: int) -> int:
    """Smallest power of two >= n (1 for n <= 1)."""
    return 1 if n <= 1 else 1 << (int(n) - 1).bit_length()


def ensure_contiguous(fn):
    """Decorator for ``autograd.Function`` static methods: every tensor argument is made contiguous
    before the call (the reference applies the same rule to its forward and backward methods,
    flash_moe/ops/utils.py:35-45)."""

    @functools.wraps(fn)
    def wrapper(ctx, *args, **kwargs):
        fix = lambda a: a.contiguous() if isinstance(a, torch.Tensor) else a
        return fn(ctx, *[fix(a) for a in args], **{k: fix(v) for k, v in kwargs.items()})

    return wrapper
