"""Sequence cache of hybrid models: a paged pool for what attention layers keep per token
and fixed state slots for what recurrent layers carry per sequence.

Every layer declares what it needs (``Mixer.cache_spec``; a mixer made of several gives a
list):
  * ``("paged", width)``  -- one vector of ``width`` numbers per token, stored in pages of
    ``PAGE`` tokens drawn from the shared ``PageAllocator`` (page 0 is the null page); a
    sequence's token t lives at ``pages[t // PAGE] * PAGE + t % PAGE`` in every paged layer;
  * ``("state", {name: shape})`` -- fp32 tensors per sequence slot, overwritten in place by
    the layer's kernels; a portion that starts at position 0 ignores what the slot held.
A sequence holds one state slot and a growing list of pages; both return to the free lists
when it closes and are handed to later sequences as they are (no clearing is needed: a new
sequence starts from zero state by position, and never reads a token it has not written).
"""
from __future__ import annotations

import torch

from ..ops import PAGE
from .kv_cache import PageAllocator, pages_for


def layer_specs(specs: list):
    """(layer, kind, what) for every declaration; a layer may give one spec, a list of specs
    (a mixer made of several) or None."""
    for i, spec in enumerate(specs):
        if not spec:
            continue
        for kind, what in (spec if isinstance(spec, list) else [spec]):
            yield i, kind, what


class SlotAllocator:
    def __init__(self, n: int):
        if n < 1:
            raise ValueError("need at least one state slot")
        self.n = n
        self._free = list(range(n - 1, -1, -1))

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise MemoryError("no free state slot (%d sequences are live)" % self.n)
        return self._free.pop()

    def free(self, s: int):
        if s < 0 or s >= self.n or s in self._free:
            raise ValueError("bad state slot %d" % s)
        self._free.append(s)


class Sequence:
    __slots__ = ("key", "slot", "pages", "length")

    def __init__(self, key, slot):
        self.key, self.slot, self.pages, self.length = key, slot, [], 0


class SequenceCache:
    def __init__(self, specs: list, num_pages: int, num_slots: int, device, dtype):
        """specs: one ``cache_spec()`` per layer (None for a layer that keeps nothing)."""
        self.device = torch.device(device)
        self.num_pages, self.num_slots = num_pages, num_slots
        self.allocator = PageAllocator(num_pages)
        self.slots = SlotAllocator(num_slots)
        self.paged, self.state = {}, {}
        for i, kind, what in layer_specs(specs):
            if kind == "paged":
                if i in self.paged:
                    raise ValueError("layer %d declares two paged pools" % i)
                self.paged[i] = torch.zeros(num_pages * PAGE, int(what), device=self.device,
                                            dtype=dtype)
            elif kind == "state":
                # one slot more than the allocator hands out: the null slot, where padding rows
                # of a bucketed (graph-captured) step keep their state, like the null page
                st = self.state.setdefault(i, {})
                for k, s in what.items():
                    if k in st:
                        raise ValueError("layer %d declares state %r twice" % (i, k))
                    st[k] = torch.zeros((num_slots + 1,) + tuple(s), device=self.device,
                                        dtype=torch.float32)
            else:
                raise ValueError("unknown cache kind %r" % kind)
        self.null_slot = num_slots
        self._live = {}

    # ------------------------------------------------------------ sequences
    def open(self, key) -> Sequence:
        if key in self._live:
            raise KeyError("sequence %r is already live" % (key,))
        seq = self._live[key] = Sequence(key, self.slots.alloc())
        return seq

    def get(self, key) -> Sequence:
        return self._live[key]

    def __contains__(self, key):
        return key in self._live

    @property
    def live(self) -> int:
        return len(self._live)

    def reserve(self, seq: Sequence, tokens: int):
        """Make the sequence's pages cover ``tokens`` tokens."""
        need = pages_for(tokens) - len(seq.pages)
        if need > 0:
            seq.pages += self.allocator.alloc(need)

    def close(self, key):
        seq = self._live.pop(key)
        if seq.pages:
            self.allocator.free(seq.pages)
        self.slots.free(seq.slot)

    def bytes_per_page(self) -> int:
        return sum(t.shape[1] * t.element_size() * PAGE for t in self.paged.values())

    def bytes_per_slot(self) -> int:
        return sum(t[0].numel() * 4 for d in self.state.values() for t in d.values())
