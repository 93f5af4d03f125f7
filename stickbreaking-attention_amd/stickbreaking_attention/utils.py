"""Constants and the torch.compile hook, with the names of the reference's stickbreaking_attention/utils.py:7-40."""
import math
from typing import Callable, Iterable, Sequence

import torch

PACKAGE_NAME = "stickbreaking_attention"
log2 = math.log(2)
inv_log2 = 1 / log2          # the kernels work in base 2: logits are scaled by inv_temp * inv_log2 (utils.py:8-9)


def _dispatch(func: Callable, compileable_fn: Callable, *args, **kwargs):
    """Eager calls go straight to the launcher; under torch.compile the registered operator is called so that
    the graph holds one opaque node (utils.py:12-17)."""
    if torch.compiler.is_compiling():
        return compileable_fn(*args, **kwargs)
    return func(*args, **kwargs)


def custom_op(name: str = None, mutates_args: str | Iterable[str] = None,
              device_types: str | Sequence[str] | None = None, schema: str | None = None) -> Callable:
    """Registers ``func`` as ``stickbreaking_attention::<name>`` (utils.py:20-40).  The launchers registered
    with it are out-parameter functions that return None, so no fake implementation is needed."""
    compileable_name = f"{PACKAGE_NAME}::{name}"

    def _inner(func: Callable):
        compileable_func = torch.library.custom_op(compileable_name, func, mutates_args=mutates_args,
                                                   device_types=device_types, schema=schema)

        def _run(*args, **kwargs):
            return _dispatch(func, compileable_func, *args, **kwargs)

        _run.__name__ = getattr(func, "__name__", name)
        _run.compileable = compileable_func
        return _run

    return _inner
