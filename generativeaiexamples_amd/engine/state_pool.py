"""Per-sequence recurrent state slots (the counterpart of the paged KV cache for layers whose memory of the past is a
fixed-size state: linear attention, WKV, delta rule, short convolutions, token shift).

A model registers its state tensors once (``add``): each gets a leading - or, with ``slot_dim``, an inner - axis of
``n_slots + 1`` entries in fp32. A live sequence owns one slot index across all of them; ``slot(sid, fresh)`` hands the
index out (allocating on first use) and zero-fills the sequence's entries when it starts from position 0;
``release(sid)`` returns the index for reuse. The last index is the pad slot: rows of a padded decode graph write
there. Kernels address states through a device vector of slot indices, so a step updates them in place.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch


class StatePool:
    def __init__(self, n_slots: int, device):
        self.n_slots = int(n_slots)
        self.device = torch.device(device)
        self.tensors: Dict[str, Tuple[torch.Tensor, int]] = {}
        self.slot_of: Dict[int, int] = {}
        self.free_slots: List[int] = list(range(self.n_slots))[::-1]

    @property
    def pad_slot(self) -> int:
        return self.n_slots

    def clear(self) -> None:
        """Drop every registered tensor and every assignment (weights reloaded)."""
        self.tensors.clear()
        self.slot_of.clear()
        self.free_slots = list(range(self.n_slots))[::-1]

    def add(self, name: str, shape, slot_dim: int = 0, dtype=torch.float32) -> torch.Tensor:
        """Register a zero-filled state tensor: `shape` with an axis of n_slots + 1 inserted at slot_dim."""
        full = list(shape)
        full.insert(slot_dim, self.n_slots + 1)
        t = torch.zeros(*full, dtype=dtype, device=self.device)
        self.tensors[name] = (t, slot_dim)
        return t

    def slot(self, sid: int, fresh: bool = False) -> int:
        s = self.slot_of.get(sid)
        if s is None:
            if not self.free_slots:
                raise RuntimeError("state slot pool exhausted: raise GAI_LINEAR_STATE_SLOTS or lower max_num_seqs")
            s = self.slot_of[sid] = self.free_slots.pop()
            fresh = True
        if fresh:
            for t, d in self.tensors.values():
                t.select(d, s).zero_()
        return s

    def release(self, sid: int) -> None:
        s = self.slot_of.pop(sid, None)
        if s is not None:
            self.free_slots.append(s)

    @property
    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t, _ in self.tensors.values())
