"""Slots for per-request state of fixed size.

Every live request holds one slot index, valid in the state tensor of every
site that declared a StateNeed ([n_slots, *shape] each).  The Llama architecture
declares none; the slot still exists (the index is part of every step's
metadata) so that a mixer with a recurrent state can be added without touching
the cache manager.  The reference has nothing like it.
"""


class StateSlots:
    def __init__(self, n_slots):
        if n_slots <= 0:
            raise ValueError("need at least one state slot")
        self.n_slots = n_slots
        self.free = list(reversed(range(n_slots)))
        self.owner = {}

    def acquire(self, request):
        if request in self.owner:
            raise ValueError(f"request {request!r} already holds a state slot")
        if not self.free:
            raise MemoryError("no free state slot")
        slot = self.free.pop()
        self.owner[request] = slot
        return slot

    def release(self, request):
        self.free.append(self.owner.pop(request))

    def slot_of(self, request):
        return self.owner[request]

    def check(self):
        held = list(self.owner.values())
        assert len(held) == len(set(held)), "a state slot is held twice"
        assert not (set(held) & set(self.free)), "a held state slot is on the free list"
        assert len(self.free) == len(set(self.free)), "a state slot is freed twice"
        assert len(held) + len(self.free) == self.n_slots, "a state slot is lost"
