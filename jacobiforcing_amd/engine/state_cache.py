"""Storage behind the ragged step: a pool of key/value pages per attention layer run and a table of recurrent-state slots per
recurrent layer run.  Which page or slot a request uses is bookkeeping elsewhere (``BlockManager`` hands out page ids, the
runner hands out slots); this class only owns the memory, sized once.

A *layer run* is one execution of a layer in a forward: a model that repeats a span of layers with the same weights has one
run — and therefore one cache or state of its own — per repetition."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass
class RunSpec:
    """Memory one layer run needs.  kind "kv": ``k_width`` / ``v_width`` elements per cached token (all key/value heads side by
    side; ``v_width`` 0: the values are read out of the key rows, there is no second pool).  kind "state": a float tensor of
    ``state_shape`` per slot.  kind None: nothing.  Beside either, ``tail_shape`` (when not empty) is a small float tensor per slot
    for what a layer carries from step to step whatever its mixer is (the last inputs of a short convolution); a layer that carries
    several such things of different shapes names them in ``tails`` (name -> shape per slot)."""
    kind: Optional[str]
    k_width: int = 0
    v_width: int = 0
    state_shape: tuple = ()
    tail_shape: tuple = ()
    tails: Dict[str, tuple] = field(default_factory=dict)


class PagedStateCache:
    def __init__(self, specs: List[RunSpec], num_pages: int, page_size: int, num_slots: int, device, dtype):
        self.num_pages, self.page_size, self.num_slots = int(num_pages), int(page_size), int(num_slots)
        self.P = self.num_slots                      # a live request owns one slot: the scheduler's admission limit
        tokens = self.num_pages * self.page_size
        self.k: List[Optional[torch.Tensor]] = []
        self.v: List[Optional[torch.Tensor]] = []
        self.state: List[Optional[torch.Tensor]] = []
        self.tail: List[Optional[torch.Tensor]] = []
        self.tails: List[Dict[str, torch.Tensor]] = []
        for s in specs:
            kv = s.kind == "kv"
            self.k.append(torch.zeros((tokens, s.k_width), dtype=dtype, device=device) if kv else None)
            self.v.append(torch.zeros((tokens, s.v_width), dtype=dtype, device=device) if kv and s.v_width else None)
            self.tail.append(torch.zeros((self.num_slots, *s.tail_shape), dtype=torch.float32, device=device)
                             if s.tail_shape and all(int(d) > 0 for d in s.tail_shape) else None)
            self.state.append(torch.zeros((self.num_slots, *s.state_shape), dtype=torch.float32, device=device) if s.kind == "state" else None)
            self.tails.append({k: torch.zeros((self.num_slots, *shape), dtype=torch.float32, device=device)
                               for k, shape in s.tails.items() if shape and all(int(d) > 0 for d in shape)})

    def bytes(self) -> int:
        return (sum(t.numel() * t.element_size() for ts in (self.k, self.v, self.state, self.tail) for t in ts if t is not None) +
                sum(t.numel() * t.element_size() for d in self.tails for t in d.values()))
