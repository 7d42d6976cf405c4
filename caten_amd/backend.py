"""Backend registry: mirror of `define-backend` (source/codegen/backend.lisp:16-48).

A backend is five things looked up by keyword: a Buffer class, a Runtime class,
a Renderer class, an auto-scheduler configuration and whether it JIT-compiles.
"""
from __future__ import annotations

import os

_BACKENDS: dict = {}


def define_backend(name: str, buffer_class, runtime_class, renderer_class, auto_scheduler_class, is_jit_p: bool):
    """(define-backend name buffer-class runtime-class renderer-class auto-scheduler-class is-jit-p)"""
    _BACKENDS[name.upper()] = dict(buffer=buffer_class, runtime=runtime_class, renderer=renderer_class,
                                   auto_scheduler=auto_scheduler_class, jit=bool(is_jit_p))


def _get(backend, slot):
    key = (backend or os.environ.get("BACKEND", "HIP")).upper().lstrip(":")
    if key not in _BACKENDS:
        raise KeyError(f"No backend named :{key} is defined (known: {sorted(_BACKENDS)})")
    return _BACKENDS[key][slot]


def get_backend_buffer(backend=None):
    return _get(backend, "buffer")


def get_backend_runtime(backend=None):
    return _get(backend, "runtime")


def get_backend_renderer(backend=None):
    return _get(backend, "renderer")


def get_backend_auto_scheduler(backend=None):
    return _get(backend, "auto_scheduler")


def get_backend_jit_p(backend=None):
    return _get(backend, "jit")


def jit_mode_p(backend=None) -> bool:
    return get_backend_jit_p(backend)


def get_buffer_type(backend=None):
    return get_backend_buffer(backend)


def get_runtime_type(backend=None):
    return get_backend_runtime(backend)
