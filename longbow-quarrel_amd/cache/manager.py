"""The cache: a slot for each live sequence, keys and values for each layer
with each sequence's own length, and fixed-size state per sequence beside it.

Layers are grouped by what their mixers need (`KVNeed`: kv heads, head size,
window; `StateNeed`: a shape; or a need class of the model's own).  Every need builds its
group (`CacheNeed.make_group`) and every group has storage of its own: for keys and values a pool of
blocks of BLOCK_SIZE positions and a block table per slot, so a group that keeps
all positions and a group that keeps a window of them never share rows.  The
reference has one contiguous ring per layer for its single sequence
(internal/engine/kv_cache_sliding_window.go:16-185) and a block-table variant
it does not use (internal/engine/kv_cache_paged.go:17-278); a full cache here is
an error, never an overwrite of old rows (internal/engine/kv_cache.go:121-124).

Layouts of one layer of a group, chosen for the attention kernels:
  K [blocks, kv_heads, BLOCK_SIZE, head_dim]   V [blocks, kv_heads, head_dim, BLOCK_SIZE]
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Tuple

import torch

from ..parts.base import CacheNeed, KVNeed, LayerCache, StateNeed
from .slots import BLOCK_SIZE, CacheFull, FreeList


def blocks_for(tokens: int) -> int:
    return (tokens + BLOCK_SIZE - 1) // BLOCK_SIZE


class CacheGroup:
    """Storage of the runs of the schedule that share one need: what `CacheManager` asks of it.

    A group that grows with a sequence's length takes blocks from a pool of its own and answers
    `blocks_missing` / `free_blocks` / `blocks_for` truthfully, so that `CacheManager.reserve` can refuse
    a step before anything has changed; a group of fixed size per slot keeps the defaults."""

    layers: List[int]  # the runs of the schedule that the group serves

    def layer_view(self, layer: int):
        """What the mixer of run `layer` receives as `cache` (a `LayerCache`, or an object of the
        group's own; it needs `read_only()` if another run may read it through `cache_of`)."""
        raise NotImplementedError

    def free_blocks(self) -> int:
        """Blocks the pool can still hand out (a group without a pool: no limit)."""
        return 1 << 60

    def taken_blocks(self) -> int:
        return 0

    def blocks_for(self, tokens: int) -> int:
        """Blocks a sequence of `tokens` tokens holds at most."""
        return 0

    def blocks_missing(self, slot: int, new_len: int) -> int:
        """Blocks the slot still lacks for positions < new_len."""
        return 0

    def ensure(self, slot: int, new_len: int) -> None:
        """Room for positions < new_len (the manager has checked `blocks_missing` against `free_blocks`)."""

    def reserved(self) -> None:
        """Every `ensure` of one `CacheManager.reserve` has been made."""

    def trim(self, slot: int, length: int) -> None:
        """The slot holds `length` tokens now; what no later token can reach may go back."""

    def release(self, slot: int) -> None:
        """The sequence has ended: everything it holds goes back."""

    def clear(self, slot: int) -> None:
        """A new sequence starts in the slot."""


class KVGroup(CacheGroup):
    """Storage of the layers that share one KVNeed."""

    def __init__(self, need: KVNeed, layers: List[int], n_blocks: int, max_slots: int,
                 dtype: torch.dtype, device: torch.device) -> None:
        self.need = need
        self.layers = list(layers)
        self.n_blocks = int(n_blocks)
        self.max_slots = int(max_slots)
        self.blocks = FreeList(self.n_blocks, "cache block")
        shape_k = (len(layers), self.n_blocks, need.kv_heads, BLOCK_SIZE, need.head_dim)
        shape_v = (len(layers), self.n_blocks, need.kv_heads, need.head_dim, BLOCK_SIZE)
        # reads are bounded by each sequence's length, but kernels load whole tiles of a block and
        # mask afterwards: what they load must at least be finite numbers
        self.k = torch.zeros(shape_k, dtype=dtype, device=device)
        self.v = torch.zeros(shape_v, dtype=dtype, device=device)
        self.table_width = max(1, self.n_blocks)
        # The host's copy is pinned: new entries go up without a wait for the device, so a step queued ahead
        # stays queued when a sequence crosses a block's edge.  A row is only ever appended to while its
        # sequence lives; before a row is written from its start again (the slot has a new sequence) the
        # uploads asked for so far are waited for (`_uploaded`), since they read this memory when they run.
        self.table_host = torch.zeros((self.max_slots, self.table_width), dtype=torch.int32,
                                      pin_memory=device.type == "cuda")
        self._uploaded: Optional["torch.cuda.Event"] = None
        self._uploads_pending = False
        self.table_dev = torch.zeros((self.max_slots, self.table_width), dtype=torch.int32, device=device)
        # per slot: physical block of each logical block (None once trimmed away)
        self.owned: List[List[Optional[int]]] = [[] for _ in range(self.max_slots)]

    def layer_view(self, layer: int) -> LayerCache:
        i = self.layers.index(layer)
        return LayerCache(write=True, k=self.k[i], v=self.v[i], block_table=self.table_dev,
                          block_size=BLOCK_SIZE)

    def free_blocks(self) -> int:
        return self.blocks.free_count

    def taken_blocks(self) -> int:
        return self.blocks.taken_count

    def blocks_for(self, tokens: int) -> int:
        return blocks_for(tokens)

    def blocks_missing(self, slot: int, new_len: int) -> int:
        return max(0, blocks_for(new_len) - len(self.owned[slot]))

    def ensure(self, slot: int, new_len: int) -> None:
        """Blocks for positions < new_len.  The caller has checked that enough are free."""
        owned = self.owned[slot]
        first = len(owned)
        want = blocks_for(new_len)
        if want <= first:
            return
        if want > self.table_width:
            raise CacheFull(f"a sequence of {new_len} tokens needs {want} blocks, the table holds {self.table_width}")
        owned.extend(self.blocks.take_many(want - first))
        if first == 0 and self._uploaded is not None:
            self._uploaded.synchronize()
            self._uploaded = None
        self.table_host[slot, first:want] = torch.tensor(owned[first:want], dtype=torch.int32)
        self.table_dev[slot, first:want].copy_(self.table_host[slot, first:want], non_blocking=True)
        self._uploads_pending = True

    def reserved(self) -> None:
        if self._uploads_pending and self.table_dev.is_cuda:
            self._uploaded = torch.cuda.Event()
            self._uploaded.record()
        self._uploads_pending = False

    def trim(self, slot: int, length: int) -> None:
        """A windowed group gives back the blocks no later query can reach."""
        w = self.need.window
        if w <= 0:
            return
        first_needed = max(0, length - w + 1) // BLOCK_SIZE
        owned = self.owned[slot]
        for b in range(min(first_needed, len(owned))):
            if owned[b] is not None:
                self.blocks.give(owned[b])
                owned[b] = None

    def release(self, slot: int) -> None:
        for b in self.owned[slot]:
            if b is not None:
                self.blocks.give(b)
        self.owned[slot] = []


class StateGroup(CacheGroup):
    """Fixed-size state of the layers that share one StateNeed: [layers, slots, *shape]."""

    def __init__(self, need: StateNeed, layers: List[int], max_slots: int, device: torch.device) -> None:
        self.need = need
        self.layers = list(layers)
        self.data = torch.zeros((len(layers), max_slots) + tuple(need.shape), dtype=need.dtype, device=device)

    def layer_view(self, layer: int) -> LayerCache:
        return LayerCache(write=True, state=self.data[self.layers.index(layer)])

    def clear(self, slot: int) -> None:
        self.data[:, slot].zero_()


class CacheManager:
    """Slots, key/value groups and state groups of one engine."""

    def __init__(self, needs: Mapping[int, object], max_tokens: int, max_slots: int,
                 dtype: torch.dtype, device: torch.device) -> None:
        if max_tokens <= 0 or max_slots <= 0:
            raise ValueError("the cache needs a positive number of tokens and slots")
        self.max_tokens = int(max_tokens)
        self.n_blocks = blocks_for(self.max_tokens)
        self.max_slots = int(min(max_slots, self.n_blocks))
        self.slots = FreeList(self.max_slots, "slot")
        self.lengths = [0] * self.max_slots
        self.groups: List[CacheGroup] = []
        self._owner: Dict[int, CacheGroup] = {}
        by_need: Dict[object, List[int]] = {}
        for layer in sorted(needs):
            by_need.setdefault(needs[layer], []).append(layer)
        for need, layers in by_need.items():
            if not isinstance(need, CacheNeed):
                raise TypeError(f"run {layers[0]} of the schedule: {need!r} is no CacheNeed "
                                "(a need builds its own group: CacheNeed.make_group)")
            g = need.make_group(layers, self.n_blocks, self.max_slots, dtype, device)
            self.groups.append(g)
            for layer in layers:
                self._owner[layer] = g

    @property
    def kv_groups(self) -> List[KVGroup]:
        return [g for g in self.groups if isinstance(g, KVGroup)]

    @property
    def state_groups(self) -> List[StateGroup]:
        return [g for g in self.groups if isinstance(g, StateGroup)]

    # ---- slots ------------------------------------------------------------------------
    def acquire(self) -> int:
        slot = self.slots.take()
        self.lengths[slot] = 0
        for g in self.groups:
            g.clear(slot)
        return slot

    def release(self, slot: int) -> None:
        self.slots.give(slot)  # raises if the slot is not in use
        for g in self.groups:
            g.release(slot)
        self.lengths[slot] = 0

    def length(self, slot: int) -> int:
        if not self.slots.is_taken(slot):
            raise ValueError(f"slot {slot} is not in use")
        return self.lengths[slot]

    # ---- growth ---------------------------------------------------------------------------
    def reserve(self, growth: Mapping[int, int]) -> None:
        """Makes room for `growth[slot]` more tokens in every slot named, or raises CacheFull
        before anything has changed.  What a group uploads for it (new block-table entries) is queued on the
        current stream without a wait: call this with the stream current on which the step's kernels run."""
        for g in self.groups:
            missing = sum(g.blocks_missing(slot, self.lengths[slot] + n) for slot, n in growth.items())
            if missing > g.free_blocks():
                raise CacheFull(
                    f"the cache is full: {missing} more blocks of {BLOCK_SIZE} tokens are needed, "
                    f"{g.free_blocks()} of {self.n_blocks} are free")
        for g in self.groups:
            for slot, n in growth.items():
                g.ensure(slot, self.lengths[slot] + n)
            g.reserved()

    def advance(self, growth: Mapping[int, int]) -> None:
        for slot, n in growth.items():
            self.lengths[slot] += n
            for g in self.groups:
                g.trim(slot, self.lengths[slot])

    def free_blocks(self) -> int:
        """Blocks that every group can still hand out."""
        return min((g.free_blocks() for g in self.groups), default=1 << 60)

    def blocks_for(self, tokens: int) -> int:
        """Blocks a sequence of `tokens` tokens takes from the fullest-growing group."""
        return max((g.blocks_for(tokens) for g in self.groups), default=0)

    # ---- views --------------------------------------------------------------------------------
    def layer_views(self) -> Dict[int, object]:
        return {layer: g.layer_view(layer) for layer, g in self._owner.items()}

    def tokens_held(self) -> int:
        """Tokens of live sequences, each rounded up to whole blocks (largest over the groups)."""
        return max((g.taken_blocks() for g in self.groups), default=0) * BLOCK_SIZE
