"""StateSlotManager — per-sequence recurrent state beside the paged KV pool.

Layers that carry a fixed-size state from token to token (a recurrence's matrix, the last inputs of a causal convolution)
keep it in a SLOT: one row of an fp32 pool [num_slots, floats per slot], laid out by the model (`add_region` hands out
offsets). A sequence gets the lowest free slot when it first brings tokens and gives it back when it is released; slots are
reused without clearing — kernels take "position 0" as the start from the zero state and never read carried inputs of
positions before the sequence's start.

Carried convolution inputs are double-buffered by PARITY: a step reads the buffer the previous step wrote and writes the
other one, so the kernel that convolves a step's tokens never reads what it writes. `begin_step` returns, per sequence,
`slot * 2 + parity` (what the kernels take per token) and flips the parity of every sequence that takes part.

Sequences that are swapped out keep their state in host memory (`swap_out` / `swap_in`), so the number of slots bounds the
sequences that RUN together, not the ones the scheduler knows.
"""
from typing import Dict, List, Sequence

import numpy as np
import torch


class StateSlotManager:
    def __init__(self, num_slots: int, device="cuda"):
        self.num_slots = int(num_slots)
        self.device = torch.device(device)
        self.slot_floats = 0
        self.pool = None
        self._free = list(range(self.num_slots - 1, -1, -1))       # pop() hands out the lowest id
        self._slot_of: Dict[int, int] = {}
        self._parity: Dict[int, int] = {}
        self._swapped: Dict[int, tuple] = {}

    # ---- layout (before allocate) ------------------------------------------------------------------------------------
    def add_region(self, floats: int) -> int:
        """Reserve `floats` fp32 words in every slot; returns their offset (16-byte aligned)."""
        off = self.slot_floats
        self.slot_floats += -(-int(floats) // 4) * 4
        return off

    def allocate(self):
        self.pool = torch.zeros((self.num_slots, max(self.slot_floats, 4)), dtype=torch.float32, device=self.device)

    @property
    def slot_stride(self) -> int:
        return self.pool.shape[1]

    @property
    def num_free_slots(self) -> int:
        return len(self._free)

    def slot_of(self, seq_id: int) -> int:
        return self._slot_of[seq_id]

    # ---- per step ----------------------------------------------------------------------------------------------------
    def begin_step(self, seq_ids: Sequence[int], starts: Sequence[int]) -> np.ndarray:
        """Codes `slot * 2 + parity` of the sequences of a step. A sequence that starts at position 0 gets a slot (a fresh
        one, or its own again); one that continues must have one."""
        codes = np.empty(len(seq_ids), dtype=np.int32)
        for i, (sid, start) in enumerate(zip(seq_ids, starts)):
            slot = self._slot_of.get(sid)
            if slot is None:
                if start != 0:
                    raise RuntimeError(f"sequence {sid} continues at position {start} but holds no state slot")
                if not self._free:
                    raise RuntimeError(f"no free state slot ({self.num_slots} in total): too many sequences run together")
                slot = self._free.pop()
                self._slot_of[sid] = slot
                self._parity[sid] = 0
            par = self._parity[sid]
            codes[i] = slot * 2 + par
            self._parity[sid] = par ^ 1
        return codes

    def release(self, seq_ids: Sequence[int]):
        for sid in seq_ids:
            slot = self._slot_of.pop(sid, None)
            self._parity.pop(sid, None)
            self._swapped.pop(sid, None)
            if slot is not None:
                self._free.append(slot)
        self._free.sort(reverse=True)

    # ---- swapping ----------------------------------------------------------------------------------------------------
    def swap_out(self, seq_ids: Sequence[int]):
        """Move the state of the given sequences to host memory and free their slots."""
        for sid in seq_ids:
            slot = self._slot_of.pop(sid, None)
            if slot is None:
                continue
            self._swapped[sid] = (self.pool[slot].to("cpu"), self._parity.pop(sid))
            self._free.append(slot)
        self._free.sort(reverse=True)

    def swap_in(self, seq_ids: Sequence[int]):
        for sid in seq_ids:
            saved = self._swapped.pop(sid, None)
            if saved is None:
                continue
            if not self._free:
                raise RuntimeError(f"no free state slot ({self.num_slots} in total) to swap sequence {sid} in")
            slot = self._free.pop()
            self.pool[slot].copy_(saved[0])
            self._slot_of[sid] = slot
            self._parity[sid] = saved[1]

    def snapshot(self, seq_ids: Sequence[int]):
        """A copy of the slots of the given sequences (to undo a step that has to run twice)."""
        rows = torch.tensor(sorted({self._slot_of[s] for s in seq_ids}), dtype=torch.long, device=self.pool.device)
        return rows, self.pool.index_select(0, rows)

    def restore(self, saved):
        rows, data = saved
        self.pool.index_copy_(0, rows, data)

    def live_sequences(self) -> List[int]:
        return sorted(self._slot_of)
