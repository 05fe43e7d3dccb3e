"""Per-sequence recurrent state slots, the fixed-size counterpart of the paged
KV cache.

Layers whose memory does not grow with the sequence (matrix-state linear
recurrences, short-convolution tails, the previous token of a token shift)
keep it in a *slot*: one row of a float32 arena ``[num_slots, floats_per_slot]``.
A model declares named buffers per layer (``{"S": (H, D, Dv), ...}``); each
becomes a strided view ``[num_slots, *shape]`` into the arena, so a slot's
whole state is one contiguous row (one copy to checkpoint or migrate it) and
the kernels address it with a slot stride. Slots are handed out on admission
and returned when a request ends. A returned slot is not cleared: every
state-carrying op ignores what it finds there for a sequence that starts at
position 0, so a reused slot cannot leak its previous owner's state.
"""

from typing import Dict, List, Optional, Sequence, Tuple

import torch

__all__ = ["StateCacheManager"]


class StateCacheManager:
    def __init__(self, layer_buffers: Sequence[Optional[Dict[str, Tuple[int, ...]]]], num_slots: int, device=None):
        self.num_slots = num_slots
        self.device = device or ("cuda" if torch.cuda.is_available() else "cpu")
        offsets, total = [], 0
        for spec in layer_buffers:
            layout = {}
            for name, shape in (spec or {}).items():
                n = 1
                for s in shape:
                    n *= int(s)
                layout[name] = (total, n, tuple(int(s) for s in shape))
                total += (n + 3) // 4 * 4  # keep every buffer 16-byte aligned inside a slot row
            offsets.append(layout)
        self.floats_per_slot = max(total, 4)
        self.arena = torch.zeros(num_slots, self.floats_per_slot, dtype=torch.float32, device=self.device)
        self.layers: List[Dict[str, torch.Tensor]] = [
            {name: self.arena[:, off : off + n].view(num_slots, *shape) for name, (off, n, shape) in layout.items()}
            for layout in offsets
        ]
        self._free: List[int] = list(range(num_slots - 1, -1, -1))
        self._owner: Dict[int, int] = {}  # seq id -> slot

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def can_allocate(self) -> bool:
        return bool(self._free)

    def allocate(self, seq_id) -> int:
        assert self._free, "no free state slot"
        assert seq_id not in self._owner, f"sequence {seq_id!r} already holds a slot"
        self._owner[seq_id] = self._free.pop()
        return self._owner[seq_id]

    def slot(self, seq_id) -> int:
        return self._owner[seq_id]

    def free(self, seq_id) -> None:
        slot = self._owner.pop(seq_id, None)
        if slot is not None:
            self._free.append(slot)

    def buffer(self, layer: int, name: str) -> torch.Tensor:
        return self.layers[layer][name]
