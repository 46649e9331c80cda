"""Plugin boundary with the semantics of the reference's ``fla/ops/backends/__init__.py``:
``BaseBackend`` (:33-88), ``BackendRegistry`` (:96-157) and the ``@dispatch`` decorator
(:160-220).

A backend is an object whose class carries ``backend_type``, ``package_name``, ``env_var``,
``default_enable`` and ``priority`` (lower wins, default 5).  For an overridable function
``f`` it may define ``f(*args, **kw)`` and ``f_verifier(*args, **kw) -> (ok, reason)``.
``@dispatch('<operation>')`` tries the registered backends of that operation in priority
order (registration order breaks ties), skips those that are unavailable, disabled or whose
verifier rejects or raises, and otherwise falls through to the decorated default.
``FLA_DISABLE_BACKEND_DISPATCH=1`` (read at import) turns the decorator into the identity.
"""
from __future__ import annotations

import contextlib
import importlib
import importlib.util
import logging
import os
import threading
from functools import wraps
from typing import Any, Callable, ClassVar

import torch

logger = logging.getLogger(__name__)

_DISPATCH_DISABLED = os.environ.get('FLA_DISABLE_BACKEND_DISPATCH') == '1'

_spec_cache: dict[str, bool] = {}


def _has_package(name: str) -> bool:
    if name not in _spec_cache:
        try:
            _spec_cache[name] = importlib.util.find_spec(name) is not None
        except (ImportError, ValueError):
            _spec_cache[name] = False
    return _spec_cache[name]


class BaseBackend:
    backend_type: ClassVar[str] = 'base'
    package_name: ClassVar[str | None] = None
    env_var: ClassVar[str | None] = None
    default_enable: ClassVar[bool] = True
    priority: ClassVar[int] = 5

    @classmethod
    def is_available(cls) -> bool:
        return True if cls.package_name is None else _has_package(cls.package_name)

    @classmethod
    def is_enabled(cls) -> bool:
        if cls.env_var is None:
            return True
        return os.environ.get(cls.env_var, '1' if cls.default_enable else '0') != '0'

    @classmethod
    def can_use(cls) -> bool:
        return cls.is_available() and cls.is_enabled()

    def verify(self, func_name: str, *args, **kwargs) -> tuple[bool, str | None]:
        verifier = getattr(self, f'{func_name}_verifier', None)
        if verifier is None:
            return True, None
        try:
            return verifier(*args, **kwargs)
        except Exception as exc:       # a verifier that raises is a rejection, not an error
            return False, str(exc)


# operation name -> module whose import registers that operation's backends
_OPERATION_BACKEND_MODULES: dict[str, str] = {}


class BackendRegistry:
    _registries: ClassVar[dict[str, 'BackendRegistry']] = {}
    _initialized: ClassVar[set[str]] = set()
    _init_lock: ClassVar[threading.Lock] = threading.Lock()

    def __init__(self, operation_name: str):
        self.operation_name = operation_name
        self._backends: dict[str, BaseBackend] = {}
        self._active: BaseBackend | None = None
        self._lock = threading.RLock()
        self._logged: set[str] = set()
        BackendRegistry._registries[operation_name] = self

    def register(self, backend: BaseBackend) -> None:
        with self._lock:
            self._backends[backend.backend_type] = backend
            self._active = next((b for b in self._get_sorted_backends() if b.can_use()), self._active)

    def _get_sorted_backends(self) -> list[BaseBackend]:
        order = list(self._backends.values())
        return [b for _, _, b in sorted((b.priority, i, b) for i, b in enumerate(order))] \
            if all(isinstance(b.priority, int) for b in order) else order

    def get_active(self) -> BaseBackend | None:
        return self._active

    @classmethod
    def ensure_initialized(cls, operation: str) -> None:
        if operation in cls._initialized:
            return
        with cls._init_lock:
            if operation in cls._initialized:
                return
            module = _OPERATION_BACKEND_MODULES.get(operation, f'fla_hip.ops.{operation}.backends')
            with contextlib.suppress(ImportError):
                importlib.import_module(module)
            cls._initialized.add(operation)


def dispatch(operation: str) -> Callable[[Callable], Callable]:
    def decorator(func: Callable) -> Callable:
        if _DISPATCH_DISABLED:
            return func
        name = func.__name__

        @wraps(func)
        def wrapper(*args, **kwargs) -> Any:
            BackendRegistry.ensure_initialized(operation)
            registry = BackendRegistry._registries.get(operation)
            if registry is None:
                return func(*args, **kwargs)
            for be in registry._get_sorted_backends():
                if not (be.is_available() and be.is_enabled()):
                    continue
                ok, reason = be.verify(name, *args, **kwargs)
                if not ok:
                    key = f'{operation}:{name}:{be.backend_type}:fail'
                    if key not in registry._logged:
                        registry._logged.add(key)
                        logger.info('[FLA Backend] %s.%s -> %s rejected: %s', operation, name, be.backend_type, reason)
                    continue
                impl = getattr(be, name, None)
                if impl is None:
                    continue
                out = impl(*args, **kwargs)
                key = f'{operation}:{name}:{be.backend_type}'
                if key not in registry._logged:
                    registry._logged.add(key)
                    logger.info('[FLA Backend] %s.%s -> %s', operation, name, be.backend_type)
                return out
            return func(*args, **kwargs)

        return torch.compiler.disable(wrapper)

    return decorator


__all__ = ['BackendRegistry', 'BaseBackend', 'dispatch']
