"""Runtime glue with the behaviour of the reference's ``fla.utils`` for this path:
``tensor_cache`` (fla/utils/_decorators.py:31-82), ``input_guard`` (:99-165),
``assert_close`` / ``get_err_ratio`` / ``get_abs_err`` (fla/utils/_testing.py:19-41)."""
from __future__ import annotations

import contextlib
import functools
import inspect
import logging
import os
import warnings
from collections import deque
from typing import Any, Callable

import torch

logger = logging.getLogger(__name__)

FLA_CI_ENV = os.environ.get('FLA_CI_ENV') == '1'
FLA_DISABLE_TENSOR_CACHE = os.environ.get('FLA_DISABLE_TENSOR_CACHE') == '1'
FLA_TENSOR_CACHE_SIZE = int(os.environ.get('FLA_TENSOR_CACHE_SIZE', '4'))


def tensor_cache(fn: Callable[..., Any]) -> Callable[..., Any]:
    """Memoise the last few results by ARGUMENT IDENTITY (``is``), as the reference does for
    its index helpers: calling again with the very same tensor objects returns the cached
    result; equal-valued but distinct tensors recompute.  A tensor argument that has been written
    in place since (its version counter moved: a serving loop that refills a persistent
    ``cu_seqlens`` buffer) recomputes as well - what is cached here includes bounds checks."""
    entries: deque = deque(maxlen=FLA_TENSOR_CACHE_SIZE)

    def versions(args, kwargs):
        # (tensors created in inference mode keep no version counter: calls with one are not memoised)
        return tuple(None if x.is_inference() else x._version for x in (*args, *kwargs.values()) if isinstance(x, torch.Tensor))

    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        if FLA_DISABLE_TENSOR_CACHE or os.environ.get('FLA_DISABLE_TENSOR_CACHE') == '1':
            return fn(*args, **kwargs)
        now = versions(args, kwargs)
        if None in now:
            return fn(*args, **kwargs)
        for a0, k0, v0, r0 in entries:
            if len(a0) == len(args) and k0.keys() == kwargs.keys() \
                    and all(x is y for x, y in zip(args, a0)) \
                    and all(kwargs[key] is k0[key] for key in kwargs) \
                    and v0 == now:
                return r0
        out = fn(*args, **kwargs)
        entries.append((args, kwargs, now, out))
        return out

    return wrapper


def input_guard(fn: Callable | None = None, *, no_guard_contiguous=False):
    """Make every tensor argument contiguous (optionally skipping named ones) and run ``fn``
    with the first tensor's device as the current device."""

    def decorate(f):
        names = list(inspect.signature(f).parameters)
        skip_all = no_guard_contiguous is True
        skip = set(no_guard_contiguous) if isinstance(no_guard_contiguous, (list, tuple, set)) else set()

        def fix(name, x):
            if isinstance(x, torch.Tensor) and not skip_all and name not in skip:
                return x.contiguous()
            return x

        @functools.wraps(f)
        def wrapper(*args, **kwargs):
            new_args = [fix(names[i] if i < len(names) else f'__arg_{i}', a) for i, a in enumerate(args)]
            new_kwargs = {k: fix(k, v) for k, v in kwargs.items()}
            first = next((a for a in list(args) + list(kwargs.values()) if isinstance(a, torch.Tensor)), None)
            if first is not None and first.is_cuda:
                ctx = torch.cuda.device(first.device.index)
            else:
                ctx = contextlib.nullcontext()
            with ctx:
                return f(*new_args, **new_kwargs)

        return wrapper

    return decorate(fn) if fn is not None else decorate


contiguous = input_guard


def get_abs_err(x: torch.Tensor, y: torch.Tensor) -> float:
    return (x.detach() - y.detach()).flatten().abs().max().item()


def get_err_ratio(x: torch.Tensor, y: torch.Tensor) -> float:
    err = (x.detach() - y.detach()).flatten().square().mean().sqrt().item()
    base = x.detach().flatten().square().mean().sqrt().item()
    return err / (base + 1e-8)


def assert_close(prefix: str, ref: torch.Tensor, tri: torch.Tensor, ratio: float, warning: bool = False,
                 err_atol: float = 1e-6) -> None:
    """Test helper with the call signature of the reference's (fla/utils/_testing.py:29-41): passes when
    the largest absolute difference is at most ``err_atol`` or the relative RMS error is below ``ratio``;
    NaNs on either side fail; ``warning=True`` (or the lenient CI mode, ``FLA_CI_ENV``, for results that are
    close: relative error < 1 % or absolute difference <= 0.3) reports a miss as a warning instead."""
    worst, rel = get_abs_err(ref, tri), get_err_ratio(ref, tri)
    report = f'{prefix:>16} diff: {worst:.6f} ratio: {rel:.6f}'
    logger.info(report)
    if worst <= err_atol:
        return
    for name, x in (('ref', ref), ('tri', tri)):
        assert not torch.isnan(x).any(), f'{prefix}: NaN detected in {name}'
    if rel < ratio:
        return
    lenient = warning or (FLA_CI_ENV and (rel < 0.01 or worst <= 0.3))
    if not lenient:
        raise AssertionError(report)
    if rel > ratio:
        warnings.warn(report)


__all__ = ['tensor_cache', 'input_guard', 'contiguous', 'get_abs_err', 'get_err_ratio', 'assert_close']
