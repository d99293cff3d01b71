"""What a step hands to the parts: the batch's metadata on the GPU and scratch memory."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional

import numpy as np
import torch


@dataclass(frozen=True)
class Env:
    """Build-time facts that every part may need."""
    dtype: torch.dtype          # dtype of activations and matrices: float32 or bfloat16
    device: torch.device


class Workspace:
    """Bump allocator over one GPU buffer; ``reset`` gives everything back at once.

    When a step needs more than the buffer holds, a further chunk is allocated; the next
    reset merges the chunks into one buffer of the total size, so that a warmed-up engine
    allocates nothing during a step.
    """
    ALIGN = 256

    def __init__(self, device, nbytes: int = 1 << 20):
        self.device = device
        self._chunks = [torch.empty(max(nbytes, self.ALIGN), dtype=torch.uint8, device=device)]
        self._off = 0
        self.generation = 0          # counts reallocations: addresses handed out earlier are stale after one

    def reset(self):
        if len(self._chunks) > 1:
            total = sum(c.numel() for c in self._chunks)
            self._chunks = [torch.empty(total, dtype=torch.uint8, device=self.device)]
            self.generation += 1
        self._off = 0

    def mark(self) -> int:
        """Where the next ``take`` starts; ``rewind`` goes back there (within one generation)."""
        return self._off

    def rewind(self, mark: int) -> None:
        self._off = mark

    def take(self, shape, dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        item = torch.empty((), dtype=dtype).element_size()
        nbytes = n * item
        cur = self._chunks[-1]
        start = (self._off + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        if start + nbytes > cur.numel():
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("workspace would grow while a graph is captured; warm the step up first")
            cur = torch.empty(max(nbytes + self.ALIGN, 2 * cur.numel()), dtype=torch.uint8, device=self.device)
            self._chunks.append(cur)
            self.generation += 1
            start = 0
        self._off = start + nbytes
        if n == 0:
            return torch.empty(tuple(shape), dtype=dtype, device=self.device)
        return cur[start:start + nbytes].view(dtype).view(tuple(shape))


@dataclass
class LayerCache:
    """The cache as one layer call sees it."""
    k_pages: Optional[torch.Tensor]       # [n_pages, G, page_size, hd]
    v_pages: Optional[torch.Tensor]
    slot_map: Optional[torch.Tensor]      # int32 [T]: cache row of each token of the step
    block_table: Optional[torch.Tensor]   # int32 [n_seqs, max_blocks]
    page_size: int
    write: bool                           # this call fills the cache (else it reads another layer's)
    state: Optional[torch.Tensor] = None  # [max_requests, ...]: per-request state of the layer
    tiled: bool = False                   # pages in the MFMA attention kernels' operand order, not row-major


@dataclass
class HostBatch:
    """The step's metadata as numpy arrays, for parts that walk requests on the host."""
    slots: np.ndarray          # [n_seqs] request slot of each entry
    starts: np.ndarray         # [n_seqs] position of its first token
    counts: np.ndarray         # [n_seqs] number of tokens
    cu_seqlens: np.ndarray     # [n_seqs+1]


@dataclass
class StepContext:
    T: int
    n_seqs: int
    token_ids: torch.Tensor      # int32 [T]
    positions: torch.Tensor      # int32 [T]
    seq_of_token: torch.Tensor   # int32 [T]: index of the token's entry in the step
    cu_seqlens: torch.Tensor     # int32 [n_seqs+1]
    seq_slots: torch.Tensor      # int32 [n_seqs]
    seq_starts: torch.Tensor     # int32 [n_seqs]
    logit_rows: torch.Tensor     # int32 [n_out]: token rows whose logits are wanted
    n_out: int
    host: HostBatch
    ws: Any = None               # Workspace of the layer call that runs
    decode_only: bool = False    # every entry holds one token
    max_count: int = 0           # longest portion of the step
    derived: dict = field(default_factory=dict)   # step arrays that parts asked for: name -> (device array, info)
    extras: dict = field(default_factory=dict)
