"""Values derived from a few tensors (a stack of weights, scaled random matrices), kept until one
of the tensors changes.

An entry remembers, for every source tensor, a weak reference to the tensor object and its version
counter, storage address, dtype, shape and device.  It answers only for the very same objects in the
very same state: an in-place update moves the version counter, ``p.data = ...`` moves the address,
and a tensor that has died cannot be impersonated by a new one that the allocator put at its
address (or that Python gave its id), because the weak reference is dead.
"""
from __future__ import annotations

import weakref
from typing import Callable, Optional, Sequence

from torch import Tensor


def _state(t: Optional[Tensor]):
    return None if t is None else (t._version, t.data_ptr(), t.dtype, tuple(t.shape), str(t.device))


class _Entry:
    __slots__ = ("refs", "state", "extra", "value")

    def __init__(self, sources, state, extra, value):
        self.refs = tuple(None if t is None else weakref.ref(t) for t in sources)
        self.state, self.extra, self.value = state, extra, value

    def answers(self, sources, state, extra) -> bool:
        if self.state != state or self.extra != extra or len(self.refs) != len(sources):
            return False
        return all((r is None and t is None) or (r is not None and t is not None and r() is t)
                   for r, t in zip(self.refs, sources))

    def alive(self) -> bool:
        return all(r is None or r() is not None for r in self.refs)


def derived(slot: dict, name, sources: Sequence[Optional[Tensor]], extra, make: Callable, limit: int = 0):
    """``make()`` for these source tensors, from ``slot[name]`` if that entry was made from the same
    tensor objects in the same state (and the same ``extra``), else made and stored there.  With
    ``limit`` > 0 the slot is first cleared of entries whose sources have died and, if it is still
    that full, emptied."""
    state = tuple(_state(t) for t in sources)
    e = slot.get(name)
    if e is not None and e.answers(sources, state, extra):
        return e.value
    value = make()
    if limit and len(slot) >= limit:
        for k in [k for k, v in slot.items() if not v.alive()]:
            del slot[k]
        if len(slot) >= limit:
            slot.clear()
    slot[name] = _Entry(sources, state, extra, value)
    return value
