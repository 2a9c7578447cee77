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
  ("slot_i32", width)            one int32 vector per sequence slot
                                 (token ids a layer remembers)
  ("paged_k_v", heads, kdim, vdim)  K [blocks, heads, block, kdim] and
                                 V [blocks, heads, block, vdim]
  ("group", [spec, ...])         a layer that keeps several buffers: a
                                 tuple of the above, in order

Paged buffers are addressed through BlockManager block ids, slot buffers
through Sequence.slot (the scheduler's persistent per-sequence slot), so
both are recycled by the same admission / finish / preemption paths.
A recurrent state needs no clearing on reuse: a sequence whose first row
is position 0 starts from zero whatever the slot held (ops.mingru_scan).
"""
from __future__ import annotations

from typing import List

import torch


PAGED_PAIR_KINDS = ("paged_kv", "paged_k_vt", "paged_k_v")
SLOT_KINDS = ("state", "slot_i32")


def _leaves(buf, spec):
    """(tensor, kind) for every tensor of one layer's buffer."""
    if spec[0] == "group":
        for b, s in zip(buf, spec[1]):
            yield from _leaves(b, s)
    elif isinstance(buf, tuple):
        for t in buf:
            yield t, spec[0]
    else:
        yield buf, spec[0]


class LayerCaches(list):
    """list of per-layer buffers + the spec each was built from."""

    def __init__(self, buffers, specs):
        super().__init__(buffers)
        self.specs = list(specs)

    def _all(self):
        for buf, spec in zip(self, self.specs):
            yield from _leaves(buf, spec)

    def copy_block(self, src: int, dst: int) -> None:
        """Duplicate one page in every paged layer (forked sequences
        copy their partially filled tail page)."""
        for t, kind in self._all():
            if kind in PAGED_PAIR_KINDS or kind == "latent":
                t[dst].copy_(t[src])

    def copy_slot(self, src: int, dst: int) -> None:
        """Duplicate one sequence slot's recurrent state in every
        stateful layer (a fork continues from its parent's state)."""
        for t, kind in self._all():
            if kind in SLOT_KINDS:
                t[dst].copy_(t[src])

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t, _k in self._all())


def _allocate(spec, num_blocks, block_size, num_slots, dtype, device):
    kind = spec[0]

    def z(shape, dt=dtype):
        return torch.zeros(shape, dtype=dt, device=device)

    if kind == "group":
        return tuple(_allocate(s, num_blocks, block_size, num_slots, dtype,
                               device) for s in spec[1])
    if kind == "paged_kv":
        shape = (num_blocks, spec[1], block_size, spec[2])
        return z(shape), z(shape)
    if kind == "paged_k_v":
        return (z((num_blocks, spec[1], block_size, spec[2])),
                z((num_blocks, spec[1], block_size, spec[3])))
    if kind == "paged_k_vt":
        return (z((num_blocks, spec[1], block_size, spec[2])),
                z((num_blocks, spec[1], spec[3], block_size)))
    if kind == "latent":
        return z((num_blocks, block_size, spec[1]))
    if kind == "state":
        return z((num_slots, spec[1]), torch.float32)
    if kind == "slot_i32":
        return z((num_slots, spec[1]), torch.int32)
    raise ValueError(f"unknown cache kind {kind!r}")


def allocate_caches(specs: List[tuple], num_blocks: int, block_size: int,
                    num_slots: int, dtype, device) -> LayerCaches:
    return LayerCaches(
        [_allocate(spec, num_blocks, block_size, num_slots, dtype, device)
         for spec in specs], specs)
