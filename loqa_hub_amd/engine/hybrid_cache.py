"""Cache and state manager of the hybrid decoders, beside ``PagedKVCache``.

Two kinds of per-sequence memory share one sequence table:

* **pages**: per caching attention layer either one tensor [blocks, BLK,
  width] (latent attention: the normalised latent row and the rotated shared
  key part of each token) or a key tensor [blocks, BLK, heads x size] and a
  transposed value tensor [blocks, heads x size, BLK] (``kv``), or key and
  value tensors that are both [blocks, BLK, heads x size] (``kv_rows``). The
  keys of these dictionaries are whatever the model's step function uses to
  find its storage: a layer index, or the index of a layer RUN when a model
  runs a stretch of layers several times and each pass caches for itself. The
  pages of all of them follow ONE block table per sequence,
  handed out by the same block pool the Llama KV cache uses (native
  ``BlockPool``);
* **state slots**: one slot per live sequence (the last slot is the write
  target of padding rows) in every per-layer state tensor: a recurrent layer's
  matrix state [slots + 1, H, D, Dv] f32 (``state``), or named f32 rows of any
  shape [slots + 1, ...] (``rows``: a previous token's activations, the tail
  of a short convolution). A slot is taken when a sequence is added and
  returned with its pages when the sequence is freed; the kernels treat the
  state of a sequence at position 0 as zero, so a reused slot needs no
  clearing.

Recurrent state cannot be rebuilt from shared prefix pages, so sequences of a
model with state slots never enter the pool's prefix cache.
"""
from __future__ import annotations

import torch

from .kv_cache import make_block_pool


class SlotPool:
    """Free list of state slots keyed by sequence id."""

    def __init__(self, n: int):
        self.n = n
        self._free = list(range(n))[::-1]
        self._of: dict[int, int] = {}

    def take(self, seq_id: int) -> int:
        if seq_id in self._of:
            raise KeyError(f"sequence {seq_id} already holds a state slot")
        if not self._free:
            raise RuntimeError("no free state slot")
        s = self._free.pop()
        self._of[seq_id] = s
        return s

    def give(self, seq_id: int) -> None:
        s = self._of.pop(seq_id, None)
        if s is not None:
            self._free.append(s)

    def slot(self, seq_id: int) -> int:
        return self._of[seq_id]

    def free_slots(self) -> int:
        return len(self._free)


class _SeqPool:
    """The block pool's interface with the state slots tied to it: adding a
    sequence takes a slot, freeing it gives slot and pages back."""

    def __init__(self, blocks, slots: SlotPool | None):
        self._b, self._s = blocks, slots
        self.num_blocks, self.block_size = blocks.num_blocks, blocks.block_size

    def add_seq(self, seq_id: int, toks) -> int:
        # never a prefix hit when the model carries state (see the module text)
        hit = self._b.add_seq(seq_id, [] if self._s is not None else toks)
        if hit >= 0 and self._s is not None:
            try:
                self._s.take(seq_id)
            except Exception:
                self._b.free_seq(seq_id)
                raise
        return hit

    def free_seq(self, seq_id: int) -> None:
        if self._s is not None:
            self._s.give(seq_id)
        self._b.free_seq(seq_id)

    def cache_prefix(self, seq_id: int, toks) -> None:
        if self._s is None:
            self._b.cache_prefix(seq_id, toks)

    def __getattr__(self, name):          # append / step_meta / seq_len / truncate / ...
        return getattr(self._b, name)


class HybridCache:
    def __init__(self, spec: dict, num_blocks: int, block_size: int, max_seqs: int, device,
                 dtype=torch.bfloat16):
        dev = torch.device(device)
        self.block_size, self.num_blocks, self.max_seqs = block_size, num_blocks, max_seqs
        self.latent = {li: torch.zeros(num_blocks, block_size, width, dtype=dtype, device=dev)
                       for li, width in spec["latent"].items()}
        self.state = {li: torch.zeros(max_seqs + 1, H, D, Dv, dtype=torch.float32, device=dev)
                      for li, (H, D, Dv) in spec["state"].items()}
        # key pages and transposed value pages of plain (uncompressed) attention
        # layers: the value product sums over a page's keys, so its kernels want
        # a column's keys side by side
        self.kv = {li: (torch.zeros(num_blocks, block_size, kw, dtype=dtype, device=dev),
                        torch.zeros(num_blocks, vw, block_size, dtype=dtype, device=dev))
                   for li, (kw, vw) in spec.get("kv", {}).items()}
        # key pages and value pages in the same row-major layout (softmax
        # attention: its kernels stage both through LDS tile by tile)
        self.kv_rows = {li: (torch.zeros(num_blocks, block_size, kw, dtype=dtype, device=dev),
                             torch.zeros(num_blocks, block_size, vw, dtype=dtype, device=dev))
                        for li, (kw, vw) in spec.get("kv_rows", {}).items()}
        # named per-sequence rows
        self.rows = {li: {name: torch.zeros(max_seqs + 1, *shape, dtype=torch.float32, device=dev)
                          for name, shape in named.items()}
                     for li, named in spec.get("rows", {}).items()}
        self.slots = SlotPool(max_seqs) if (self.state or self.rows) else None
        self.pool = _SeqPool(make_block_pool(num_blocks, block_size,
                                             require_native=dev.type == "cuda"), self.slots)

    @property
    def trash_slot(self) -> int:
        return self.max_seqs

    def state_slots(self, seq_ids: list[int], B_pad: int):
        """int32 list of each sequence's state slot, padded with the trash slot."""
        if self.slots is None:
            return [0] * B_pad
        return [self.slots.slot(s) for s in seq_ids] + [self.trash_slot] * (B_pad - len(seq_ids))

    def nbytes(self) -> int:
        ts = [*self.latent.values(), *self.state.values()]
        ts += [t for pair in (*self.kv.values(), *self.kv_rows.values()) for t in pair]
        ts += [t for named in self.rows.values() for t in named.values()]
        return sum(t.numel() * t.element_size() for t in ts)
