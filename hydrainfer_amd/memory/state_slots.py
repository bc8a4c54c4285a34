"""State slots: the rows a sequence carries from one step to the next beside its paged cache (a token-shift model keeps
the mixer input of the sequence's last token, one row per layer run).  One device tensor [n_slots, rows, width] of
float32; a sequence owns one slot from its first step to its end, and slots are handed out again, lowest first.  A new
owner needs no clearing: a sequence's first token (position 0) never reads the slot."""
from typing import List

import torch


class StateSlotManager:
    def __init__(self, n_slots: int, rows: int, width: int, device, dtype: torch.dtype = torch.float32):
        if n_slots < 1 or rows < 1 or width < 1:
            raise ValueError("state slots: n_slots, rows and width must be positive")
        self.n_slots, self.rows, self.width = n_slots, rows, width
        self.device = torch.device(device)
        self.state = torch.zeros((n_slots, rows, width), dtype=dtype, device=self.device)
        self.free_slots: List[int] = list(range(n_slots - 1, -1, -1))
        self.n_allocated_total = 0

    def get_num_available_slots(self) -> int:
        return len(self.free_slots)

    def allocate(self) -> int:
        """A free slot, or -1 when every slot has an owner."""
        if not self.free_slots:
            return -1
        self.n_allocated_total += 1
        return self.free_slots.pop()

    def free(self, slot: int) -> None:
        if not 0 <= slot < self.n_slots or slot in self.free_slots:
            raise ValueError(f"state slot {slot} is not in use")
        self.free_slots.append(slot)
        self.free_slots.sort(reverse=True)
