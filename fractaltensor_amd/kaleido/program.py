"""Stand-ins for the reference's program-capture decorators.

In the reference `@kaleido.function(ctx)` parses the function into an IR that
is only analysed and plotted, and then calls the original Python function
unchanged (kaleido/parser/__init__.py:85-104); `@kaleido.params(ctx)` wraps a
NamedTuple class (:106-122).  Neither is on the data path, so here both are
pass-through decorators that keep the example programs runnable verbatim,
including their `ctx[-1].ir_block.propagate_storage()` and plotting calls.
"""
from __future__ import annotations

import functools


class _IrBlock:
    def propagate_storage(self):
        return None

    def __getattr__(self, name):
        return lambda *a, **k: None


class _Entry:
    def __init__(self, name):
        self.name = name
        self.ir_block = _IrBlock()


class Context:
    def __init__(self):
        self._entries = []

    def _register(self, name):
        self._entries.append(_Entry(name))

    def __getitem__(self, i):
        return self._entries[i]

    def __len__(self):
        return len(self._entries)


def function(ctx: Context):
    def decorate(fn):
        ctx._register(fn.__name__)

        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            return fn(*args, **kwargs)
        return wrapper
    return decorate


def params(ctx: Context):
    def decorate(cls):
        ctx._register(cls.__name__)
        return cls
    return decorate


class PlotProgram:
    """The reference renders the IR with graphviz; there is no IR here."""

    def plot(self, *args, **kwargs):
        return None
