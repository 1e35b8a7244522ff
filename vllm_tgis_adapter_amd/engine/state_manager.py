"""Per-sequence state slots.

Some layers carry a fixed-size state per sequence next to the paged cache
(the last inputs of a short causal convolution, a recurrent state).  Such
state lives in slot-indexed tensors owned by the worker; this manager hands
out the slot ids.  A request holds one slot from admission until it finishes,
is aborted or is preempted; a freed slot is handed to the next admission
as is — the kernels never read state rows that lie before the start of the
sequence, so slots need no clearing.
"""

from __future__ import annotations

from collections import deque

from .request import Request


class StateSlotManager:
    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free: deque[int] = deque(range(num_slots))

    @property
    def num_free_slots(self) -> int:
        return len(self._free)

    def can_allocate(self, request: Request) -> bool:
        return request.state_slot is not None or bool(self._free)

    def allocate(self, request: Request) -> bool:
        if request.state_slot is not None:
            return True
        if not self._free:
            return False
        request.state_slot = self._free.popleft()
        return True

    def free(self, request: Request) -> None:
        if request.state_slot is not None:
            self._free.append(request.state_slot)
            request.state_slot = None
