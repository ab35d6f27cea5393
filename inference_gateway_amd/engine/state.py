"""Per-layer cache and state buffers.

A model describes what each layer keeps between steps; the engine
allocates it once and passes layer i's buffer to layer i:

  ("paged_kv", heads, head_dim)  (K, V) pair [blocks, heads, block, dim]
  ("paged_k_vt", heads, kdim, vdim)  K [blocks, heads, block, kdim] and
                                 V TRANSPOSED inside the page [blocks,
                                 heads, vdim, block]: the keys of a page
                                 are contiguous per value entry, which is
                                 the operand layout of the P.V matrix
                                 product (no transpose staging)
  ("latent", width)              one paged row per token
                                 [blocks, block, width], compute dtype
  ("state", width)               one fp32 vector per SEQUENCE SLOT
                                 [slots, width] — recurrent layers

Paged buffers are addressed through BlockManager block ids, slot buffers
through Sequence.slot (the scheduler's persistent per-sequence slot), so
both are recycled by the same admission / finish / preemption paths.
A recurrent state needs no clearing on reuse: a sequence whose first row
is position 0 starts from zero whatever the slot held (ops.mingru_scan).
"""
from __future__ import annotations

from typing import List

import torch


class LayerCaches(list):
    """list of per-layer buffers + the spec each was built from."""

    def __init__(self, buffers, specs):
        super().__init__(buffers)
        self.specs = list(specs)

    def copy_block(self, src: int, dst: int) -> None:
        """Duplicate one page in every paged layer (forked sequences
        copy their partially filled tail page)."""
        for buf, spec in zip(self, self.specs):
            if spec[0] in ("paged_kv", "paged_k_vt"):
                for t in buf:
                    t[dst].copy_(t[src])
            elif spec[0] == "latent":
                buf[dst].copy_(buf[src])

    def copy_slot(self, src: int, dst: int) -> None:
        """Duplicate one sequence slot's recurrent state in every
        stateful layer (a fork continues from its parent's state)."""
        for buf, spec in zip(self, self.specs):
            if spec[0] == "state":
                buf[dst].copy_(buf[src])

    def bytes(self) -> int:
        n = 0
        for buf in self:
            for t in (buf if isinstance(buf, tuple) else (buf,)):
                n += t.numel() * t.element_size()
        return n


def allocate_caches(specs: List[tuple], num_blocks: int, block_size: int,
                    num_slots: int, dtype, device) -> LayerCaches:
    bufs = []
    for spec in specs:
        kind = spec[0]
        if kind == "paged_kv":
            shape = (num_blocks, spec[1], block_size, spec[2])
            bufs.append((torch.zeros(shape, dtype=dtype, device=device),
                         torch.zeros(shape, dtype=dtype, device=device)))
        elif kind == "paged_k_vt":
            kshape = (num_blocks, spec[1], block_size, spec[2])
            vshape = (num_blocks, spec[1], spec[3], block_size)
            bufs.append((torch.zeros(kshape, dtype=dtype, device=device),
                         torch.zeros(vshape, dtype=dtype, device=device)))
        elif kind == "latent":
            bufs.append(torch.zeros((num_blocks, block_size, spec[1]),
                                    dtype=dtype, device=device))
        elif kind == "state":
            bufs.append(torch.zeros((num_slots, spec[1]),
                                    dtype=torch.float32, device=device))
        else:
            raise ValueError(f"unknown cache kind {kind!r}")
    return LayerCaches(bufs, specs)
