"""Constants and the torch.library shim of the reference package
(custom_models/sba/stickbreaking_attention/utils.py:5-39): every host launcher is also
registered as ``stickbreaking_attention::<name>`` with ``mutates_args``, and that
registered form is taken only while ``torch.compile`` is tracing, so that the ctypes call
into the HIP library is an opaque node of the graph."""
from __future__ import annotations

from typing import Callable, Iterable

import torch

PACKAGE_NAME = "stickbreaking_attention"


def _dispatch(func: Callable, compileable_fn: Callable, *args, **kwargs):
    if torch.compiler.is_compiling():
        return compileable_fn(*args, **kwargs)
    return func(*args, **kwargs)


def custom_op(name: str, mutates_args: Iterable[str]) -> Callable:
    compileable_name = f"{PACKAGE_NAME}::{name}"

    def _inner(func: Callable):
        compileable_func = torch.library.custom_op(compileable_name, func, mutates_args=tuple(mutates_args))

        def _run(*args, **kwargs):
            return _dispatch(func, compileable_func, *args, **kwargs)

        _run.__name__ = func.__name__
        _run.op = compileable_func
        return _run

    return _inner
