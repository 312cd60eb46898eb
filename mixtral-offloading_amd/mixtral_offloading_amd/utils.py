"""Helpers for walking nested containers of tensors, and a default-dtype guard.

The expert slab layout depends on one property only: nested dicts are
visited in sorted-key order (reference ``src/utils.py:34-45``), so that
``w1`` comes before ``w2`` and ``W_q`` before ``meta``."""
from __future__ import annotations

from contextlib import contextmanager

import torch


def is_namedtuple(x) -> bool:
    t = type(x)
    return (tuple in t.__bases__ and len(t.__bases__) == 1 and isinstance(getattr(t, "_fields", None), tuple)
            and all(isinstance(f, str) for f in t._fields))


def nested_flatten(t):
    """Leaves of a nested list / tuple / dict structure, dict values in sorted-key order."""
    stack = [t]
    while stack:
        cur = stack.pop()
        if isinstance(cur, dict):
            stack.extend(cur[k] for k in sorted(cur, reverse=True))
        elif isinstance(cur, (list, tuple)):
            stack.extend(reversed(cur))
        else:
            yield cur


def nested_pack(flat, structure):
    """Inverse of ``nested_flatten``: refill ``structure`` with the items of ``flat``."""
    it = iter(flat)

    def build(s):
        if is_namedtuple(s):
            return type(s)(*[build(v) for v in s])
        if isinstance(s, (list, tuple)):
            return type(s)(build(v) for v in s)
        if isinstance(s, dict):
            return {k: build(s[k]) for k in sorted(s)}
        return next(it)

    return build(structure)


@contextmanager
def with_default_dtype(dtype):
    saved = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        yield
    finally:
        torch.set_default_dtype(saved)
