"""Module specs: how the model's constructor arguments name the layers to build.

A spec is either a callable (``nn.ReLU``, ``nn.InstanceNorm3d``) or a sequence whose first
item is a callable and whose other items pre-bind arguments -- dicts as keyword arguments,
other sequences as runs of positional arguments, anything else as one positional argument:
``(nn.GroupNorm, (8,))``, ``(nn.Conv3d, {"kernel_size": 2})``.  Same convention as the
reference's ``partialize`` (``deconver/utils/helpers.py:91-128``), so its configurations can
be passed unchanged.
"""

from __future__ import annotations

import functools
from typing import Any, Callable, Sequence

__all__ = ["as_tuple", "partialize", "build"]


def _is_plain_sequence(obj: Any) -> bool:
    return isinstance(obj, Sequence) and not isinstance(obj, str)


def as_tuple(obj: Any) -> tuple:
    """``obj`` as a tuple: sequences (strings excepted) item by item, anything else wrapped
    (``deconver/utils/helpers.py:36-51``)."""
    return tuple(obj) if _is_plain_sequence(obj) else (obj,)


def partialize(spec: Any) -> Callable:
    """The callable a spec stands for, with its pre-bound arguments applied."""
    if callable(spec):
        return spec
    if not (_is_plain_sequence(spec) and len(spec) > 0 and callable(spec[0])):
        raise TypeError(f"Expected a callable or valid tuple, got {type(spec).__name__}")
    positional: list = []
    keywords: dict = {}
    for item in spec[1:]:
        if isinstance(item, dict):
            keywords.update(item)
        elif _is_plain_sequence(item):
            positional.extend(item)
        else:
            positional.append(item)
    return functools.partial(spec[0], *positional, **keywords)


def build(spec: Any, *args: Any, **kwargs: Any) -> Any:
    """Instantiate a spec: ``partialize(spec)(*args, **kwargs)``."""
    return partialize(spec)(*args, **kwargs)
