"""State slots for layers that carry a recurrent state from token to token (selective scans,
delta rules, short convolutions): the counterpart of the paged KV pool for state that does not
grow with the sequence.

* ``StatePool``   - the device side: for every state tensor of every stateful layer one
  allocation [num_slots, *shape]; layers get their views through ``bind_state``.
* ``StateSlots``  - the host side: which running sequence owns which slot.
* ``StatefulBlockManager`` - the block manager the scheduler sees for such a model: a sequence
  holds pages (attention layers) AND one slot; ``grow`` is all or nothing over both, ``free``
  returns both, so preemption and admission follow whichever runs out. Prefix reuse is off:
  a cached page says nothing about the scan state at its end.

A slot is not cleared when it changes hands: the first portion of a sequence (start 0) runs
with ``seq_init`` 0 and the kernels start from zero instead of reading the slot.
"""
from __future__ import annotations

import torch


class StatePool:
    def __init__(self, layers, num_slots: int, device):
        self.num_slots = num_slots
        self.tensors = []
        for layer in layers:
            ts = [torch.zeros((num_slots,) + tuple(shape), dtype=dt, device=device)
                  for shape, dt in layer.state_shapes()]
            layer.bind_state(ts)
            self.tensors.append(ts)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for ts in self.tensors for t in ts)


class StateSlots:
    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._of: dict[int, int] = {}

    def num_free(self) -> int:
        return len(self._free)

    def has(self, seq_id) -> bool:
        return seq_id in self._of

    def slot_of(self, seq_id) -> int:
        return self._of[seq_id]

    def acquire(self, seq_id) -> int:
        if seq_id in self._of:
            return self._of[seq_id]
        if not self._free:
            raise RuntimeError("no free state slot")
        s = self._of[seq_id] = self._free.pop()
        return s

    def release(self, seq_id):
        s = self._of.pop(seq_id, None)
        if s is not None:
            self._free.append(s)

    def check_invariants(self):
        assert sorted(self._free + list(self._of.values())) == list(range(self.num_slots))


class SlotTables(dict):
    """seq_id -> block table, with each sequence's state slot in ``slots``."""

    def __init__(self, tables: dict, slots: dict):
        super().__init__(tables)
        self.slots = slots


class StatefulBlockManager:
    def __init__(self, pages, num_slots: int):
        self.pages = pages
        self.slots = StateSlots(num_slots)
        self.block_size = pages.block_size
        self.num_blocks = pages.num_blocks

    # ---- admission
    def lookup(self, toks, extra) -> int:
        return 0

    def acquire(self, seq_id, toks, extra) -> int:
        got = self.pages.acquire(seq_id, toks, extra, 0)
        assert got == 0, "stateful models do not reuse cached prefixes"
        return 0

    def can_allocate(self, n: int) -> bool:
        return self.pages.can_allocate(n) and self.slots.num_free() > 0

    def grow(self, seq_id, total_tokens: int) -> bool:
        if not self.slots.has(seq_id) and self.slots.num_free() == 0:
            return False
        if not self.pages.grow(seq_id, total_tokens):
            return False
        self.slots.acquire(seq_id)
        return True

    def commit(self, seq_id, toks, num_computed: int):
        pass

    def free(self, seq_id):
        self.pages.free(seq_id)
        self.slots.release(seq_id)

    def allocate_remote(self, seq_id, num_tokens, extra):
        raise RuntimeError("stateful models do not take remote KV (the scan state is not transferred)")

    # ---- tables
    def has_seq(self, seq_id) -> bool:
        return self.pages.has_seq(seq_id)

    def block_table(self, seq_id):
        return self.pages.block_table(seq_id)

    def state_slot(self, seq_id) -> int:
        return self.slots.slot_of(seq_id)

    def num_seq_blocks(self, seq_id) -> int:
        return self.pages.num_seq_blocks(seq_id)

    def fill_block_tables(self, ids, out):
        self.pages.fill_block_tables(ids, out)

    # ---- accounting
    def num_free(self) -> int:
        return self.pages.num_free()

    def num_cached(self) -> int:
        return 0

    def usage(self) -> float:
        return max(self.pages.usage(), 1.0 - self.slots.num_free() / max(1, self.slots.num_slots))

    def reset_prefix_cache(self):
        pass

    def take_events(self):
        return []

    def take_evicted(self):
        return []

    def prefix_stats(self):
        return self.pages.prefix_stats()

    def cached_block_for(self, h):
        return None

    def check_invariants(self):
        self.pages.check_invariants()
        self.slots.check_invariants()
