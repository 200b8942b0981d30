"""Paged KV cache + block manager (the resident per-knight memory).

Layout per layer (see ``ops/reference.py``): ``K [num_blocks, Hkv, BS, D]`` and
``V [num_blocks, Hkv, D, BS]`` — both one allocation ``[L, num_blocks, Hkv, BS*D]``.
Blocks are handed out from a free list with reference counts, so a sequence can be
forked (copy-on-write share of a prefix: ``fork``) and truncated back to any token
count (``truncate``), which is how a knight's cache is rolled back to the longest
common prefix with its next prompt.

Sizing for 288 GB HBM: the cache takes ``kv_cache_fraction`` of what is free after
weights, e.g. ~230 GB on an 8B knight's GPU = 1.8M tokens at 128 KiB/token — every
knight's whole discussion stays resident across rounds with room to spare.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


class KVCacheOOM(RuntimeError):
    """Raised when the block pool is exhausted (classified as ``oom`` by the orchestrator)."""


class BlockAllocator:
    def __init__(self, num_blocks: int):
        self.num_blocks = num_blocks
        self.free: List[int] = list(range(num_blocks - 1, -1, -1))
        self.ref = [0] * num_blocks

    def alloc(self) -> int:
        if not self.free:
            raise KVCacheOOM("KV cache out of memory: no free blocks")
        b = self.free.pop()
        self.ref[b] = 1
        return b

    def incref(self, b: int) -> None:
        self.ref[b] += 1

    def release(self, b: int) -> None:
        self.ref[b] -= 1
        if self.ref[b] == 0:
            self.free.append(b)
        elif self.ref[b] < 0:  # pragma: no cover - logic error guard
            raise RuntimeError(f"double free of KV block {b}")

    @property
    def num_free(self) -> int:
        return len(self.free)


@dataclass
class SeqState:
    """One knight's resident sequence: the token ids whose K/V are in ``blocks``."""
    key: str
    tokens: List[int] = field(default_factory=list)
    blocks: List[int] = field(default_factory=list)
    # models with a running per-sequence state (input convolutions): the state slot, and how many
    # tokens the state in it has seen (it is only valid for exactly that prefix)
    slot: Optional[int] = None
    state_len: int = 0

    @property
    def length(self) -> int:
        return len(self.tokens)


class PagedKVCache:
    def __init__(self, n_layers: int, n_kv_heads: int, head_dim: int, num_blocks: int, block_size: int,
                 device, dtype=torch.bfloat16):
        self.n_layers, self.n_kv_heads, self.head_dim = n_layers, n_kv_heads, head_dim
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.device = device
        self.dtype = dtype
        shape = (n_layers, num_blocks, n_kv_heads, block_size * head_dim)
        # zero-init: masked tail keys of a partial block must be finite (0 * NaN = NaN in P.V)
        self.k = torch.zeros(shape, dtype=dtype, device=device)
        self.v = torch.zeros(shape, dtype=dtype, device=device)
        self.alloc = BlockAllocator(num_blocks)
        self.seqs: Dict[str, SeqState] = {}

    # views in the kernel layouts
    def k_layer(self, l: int) -> torch.Tensor:
        return self.k[l].view(self.num_blocks, self.n_kv_heads, self.block_size, self.head_dim)

    def v_layer(self, l: int) -> torch.Tensor:
        return self.v[l].view(self.num_blocks, self.n_kv_heads, self.head_dim, self.block_size)

    @staticmethod
    def bytes_per_block(n_layers, n_kv_heads, head_dim, block_size, dtype_bytes=2) -> int:
        return 2 * n_layers * n_kv_heads * head_dim * block_size * dtype_bytes

    # ---- sequence management ------------------------------------------------------------
    def seq(self, key: str) -> SeqState:
        s = self.seqs.get(key)
        if s is None:
            s = self.seqs[key] = SeqState(key)
        return s

    def blocks_needed(self, n_tokens: int) -> int:
        return (n_tokens + self.block_size - 1) // self.block_size

    # positions a sequence may reach (the model's RoPE table / position embeddings and the block
    # tables are sized by it); None = unbounded. Past it a kernel would index beyond those tables,
    # so the turn fails here, on the host, like any other KV exhaustion (kind "oom").
    max_tokens: Optional[int] = None

    def ensure_capacity(self, s: SeqState, n_tokens: int) -> None:
        """Grow ``s.blocks`` to hold ``n_tokens`` (copy-on-write if the tail block is shared)."""
        if self.max_tokens is not None and n_tokens > self.max_tokens:
            raise KVCacheOOM(f"context of {n_tokens} tokens exceeds the model's {self.max_tokens} positions")
        need = self.blocks_needed(n_tokens)
        if s.blocks and self.alloc.ref[s.blocks[-1]] > 1 and s.length % self.block_size:
            self._cow_tail(s)
        while len(s.blocks) < need:
            s.blocks.append(self.alloc.alloc())

    def _cow_tail(self, s: SeqState) -> None:
        old = s.blocks[-1]
        new = self.alloc.alloc()
        self.copy_blocks([old], [new])
        self.alloc.release(old)
        s.blocks[-1] = new

    def copy_blocks(self, src: List[int], dst: List[int]) -> None:
        """K8 (csrc/kv_copy.hip): whole-block copies across every layer of K and V, one launch."""
        from .. import ops
        ops.kv_block_copy(self.k.view(self.n_layers, self.num_blocks, -1),
                          self.v.view(self.n_layers, self.num_blocks, -1), src, dst)

    def truncate(self, s: SeqState, n_tokens: int) -> None:
        n_tokens = max(0, min(n_tokens, s.length))
        n_tokens = self._state_rollback(s, n_tokens)
        keep = self.blocks_needed(n_tokens)
        for b in s.blocks[keep:]:
            self.alloc.release(b)
        del s.blocks[keep:]
        del s.tokens[n_tokens:]

    def _state_rollback(self, s: SeqState, n_tokens: int) -> int:
        """Hook of caches with a running state: the token count a roll-back to ``n_tokens`` really
        lands on (a paged K/V cache alone can be cut anywhere)."""
        return n_tokens

    def _release_state(self, s: SeqState) -> None:
        pass

    def free_seq(self, key: str) -> None:
        s = self.seqs.pop(key, None)
        if s is not None:
            for b in s.blocks:
                self.alloc.release(b)
            self._release_state(s)

    def fork(self, src: str, dst: str, copy: bool = False) -> SeqState:
        """``dst`` starts as ``src``. Default: share the blocks (refcounted prefix sharing; a writer
        copies-on-write its tail). ``copy=True``: a deep snapshot in fresh blocks (K8 batch copy),
        e.g. a continuation branch that must survive the live sequence being rolled back."""
        self.free_seq(dst)
        a = self.seqs[src]
        if copy:
            new = [self.alloc.alloc() for _ in a.blocks]
            self.copy_blocks(list(a.blocks), new)
            b = self.seqs[dst] = SeqState(dst, list(a.tokens), new)
            return b
        b = self.seqs[dst] = SeqState(dst, list(a.tokens), list(a.blocks))
        for blk in b.blocks:
            self.alloc.incref(blk)
        return b

    def slots(self, s: SeqState, start: int, end: int) -> List[int]:
        bs = self.block_size
        return [s.blocks[p // bs] * bs + (p % bs) for p in range(start, end)]


class StateSlots:
    """Fixed pool of per-sequence state slots (the running state a model keeps beside its paged
    cache). A slot is handed out when a sequence first runs and returned when it is freed; a
    slot's old content is never read by its next owner (kernels treat a sequence at position 0
    as having an all-zero state)."""

    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self.free: List[int] = list(range(n_slots - 1, -1, -1))

    def take(self) -> int:
        if not self.free:
            raise KVCacheOOM(f"all {self.n_slots} sequence state slots are in use")
        return self.free.pop()

    def give(self, slot: int) -> None:
        self.free.append(slot)


class StatefulPagedCache(PagedKVCache):
    """A paged cache whose sequences also keep a running state in a slot of a fixed pool
    (``self.state``: :class:`StateSlots`). ``state_tensors()`` lists every tensor indexed by slot on
    its first axis. The state belongs to exactly ``state_len`` tokens of its sequence: rolling a
    sequence back to any other length drops it, and the sequence restarts from position 0."""

    state: StateSlots

    def state_tensors(self) -> List[torch.Tensor]:
        raise NotImplementedError

    def slot_of(self, s: SeqState) -> int:
        """The sequence's state slot (taken on first use)."""
        if s.slot is None:
            s.slot = self.state.take()
            s.state_len = 0
        return s.slot

    def _state_rollback(self, s: SeqState, n_tokens: int) -> int:
        if n_tokens == s.state_len or s.slot is None:
            return n_tokens
        s.state_len = 0         # the convolution inputs ahead of `n_tokens` are gone: start over
        return 0

    def _release_state(self, s: SeqState) -> None:
        if s.slot is not None:
            self.state.give(s.slot)
            s.slot = None

    def fork(self, src: str, dst: str, copy: bool = False) -> SeqState:
        b = super().fork(src, dst, copy=copy)
        a = self.seqs[src]
        if a.slot is not None and a.state_len == a.length:
            b.slot = self.state.take()
            b.state_len = a.state_len
            for c in self.state_tensors():
                c[b.slot].copy_(c[a.slot])
        else:
            self.truncate(b, 0)
        return b


class LatentKVCache(StatefulPagedCache):
    """Paged cache of latent-attention layers plus the input-convolution states.

    Per layer ``l`` one tensor ``rows[l]`` ``[num_blocks, block_size, row_l]``: token ``t`` of a
    sequence keeps ``row_l = kv_rank + rot_dim`` numbers (its normed latent, then the rotated key
    part all heads share) at ``slot = block * block_size + offset`` — keys AND values of every
    head are read from that one row, so a layer's cache line is 1 / (2 * heads) of a per-head
    K/V cache's. Layers may differ in row width.

    ``conv[l]`` ``[n_slots, 2, taps - 1, width]`` fp32: for each state slot the last ``taps - 1``
    inputs of layer ``l``'s two input convolutions (mixer, feed-forward), oldest first. The state
    belongs to exactly ``state_len`` tokens of its sequence: rolling a sequence back to any other
    length drops it, and the sequence restarts from position 0."""

    def __init__(self, row_dims, conv_width: int, taps: int, num_blocks: int, block_size: int, device,
                 dtype=torch.bfloat16, n_slots: int = 16):
        self.n_layers = len(row_dims)
        self.row_dims = list(row_dims)
        self.n_kv_heads, self.head_dim = 1, max(row_dims)
        self.block_size, self.num_blocks = block_size, num_blocks
        self.device, self.dtype = device, dtype
        # zero-init: tail rows of a partial block are masked, never skipped, so they must be finite
        self.rows = [torch.zeros(num_blocks, block_size, r, dtype=dtype, device=device) for r in row_dims]
        self.alloc = BlockAllocator(num_blocks)
        self.seqs = {}
        self.taps = taps
        self.state = StateSlots(n_slots)
        self.conv = [torch.zeros(n_slots, 2, max(taps - 1, 1), conv_width, dtype=torch.float32, device=device)
                     for _ in row_dims]

    @staticmethod
    def bytes_per_block(row_dims, block_size, dtype_bytes=2) -> int:   # type: ignore[override]
        return sum(row_dims) * block_size * dtype_bytes

    def layer_rows(self, l: int) -> torch.Tensor:
        return self.rows[l]

    def k_layer(self, l: int):      # the per-head views of a K/V cache do not exist here
        raise AttributeError("a latent cache has no per-head K blocks; use layer_rows()")

    v_layer = k_layer

    def copy_blocks(self, src: List[int], dst: List[int]) -> None:
        si = torch.tensor(src, dtype=torch.int64, device=self.device)
        di = torch.tensor(dst, dtype=torch.int64, device=self.device)
        for r in self.rows:
            r.index_copy_(0, di, r.index_select(0, si))

    def state_tensors(self) -> List[torch.Tensor]:
        return self.conv


class GroupedKVCache(StatefulPagedCache):
    """Paged keys and values of grouped-attention layers whose shapes differ from layer to layer,
    plus per-sequence running states.

    Layer run ``l``: ``k[l]`` ``[num_blocks, kv_heads_l, block_size, dim_l]`` and ``v[l]``
    ``[num_blocks, kv_heads_l, block_size, vdim_l]``; token ``t`` of a sequence lives at
    ``block_tables[t // block_size]``, offset ``t % block_size``. ``shapes`` gives
    ``(kv_heads, dim, vdim)`` per run. A run with ``matrix_layout`` keeps the layout of the
    matrix-core attention kernels instead: ``v[l]`` ``[num_blocks, kv_heads_l, vdim_l, block_size]``
    and each key block chunk-major (``ops/reference.py`` ``k_blocks``).

    A run whose mixer has no attention gives ``None`` as its shape and has no pages (``k[l]`` and
    ``v[l]`` are None): its memory per sequence is its state alone.

    States, fp32, one row per slot: ``shift[l]`` ``[n_slots, width]`` is the previous token's
    normed mixer input (token shift; None for a run without one when ``shift_layers`` says so);
    ``rec[l]`` ``[n_slots, rec_width_l]`` the state of the layer's recurrence — a channel vector,
    or the flattened matrix state per head of a wkv / delta-rule mixer (None for a layer without
    one). ``canon_taps`` > 1: ``conv[l]`` ``[n_slots, 2, canon_taps - 1, width]`` holds the last
    inputs of the layer's two input convolutions (mixer, feed-forward), oldest first.
    ``short_conv[l]`` = (channels, taps): ``sconv[l]`` ``[n_slots, taps - 1, channels]`` holds the
    last inputs of a short convolution inside the mixer (None for a layer without one).
    A sequence at position 0 never reads its slot, so a reused slot needs no clearing."""

    def __init__(self, shapes, width: int, rec_widths, num_blocks: int, block_size: int, device,
                 dtype=torch.bfloat16, n_slots: int = 16, matrix_layout=None, shift_layers=None,
                 canon_taps: int = 0, short_conv=None):
        shapes = [sh if sh is not None else (0, 0, 0) for sh in shapes]
        self.n_layers = len(shapes)
        # per run: the layout of the framework's matrix-core attention kernels (keys chunk-major
        # per block, values transposed [.., vdim, block_size]) instead of plain rows
        self.matrix = list(matrix_layout) if matrix_layout is not None else [False] * len(shapes)
        self.shapes = [tuple(int(x) for x in sh) for sh in shapes]
        self.n_kv_heads = max(1, max(sh[0] for sh in self.shapes))
        self.head_dim = max(1, max(max(sh[1], sh[2]) for sh in self.shapes))
        self.block_size, self.num_blocks = block_size, num_blocks
        self.device, self.dtype = device, dtype
        # zero-init: tail rows of a partial block are masked, never skipped, so they must be finite
        self.k = [torch.zeros(num_blocks, g, block_size, dk, dtype=dtype, device=device) if g else None
                  for g, dk, _ in self.shapes]
        self.v = [(torch.zeros((num_blocks, g, dv, block_size) if mx else (num_blocks, g, block_size, dv), dtype=dtype,
                               device=device) if g else None) for (g, _, dv), mx in zip(self.shapes, self.matrix)]
        self.alloc = BlockAllocator(num_blocks)
        self.seqs = {}
        self.state = StateSlots(n_slots)
        shift_layers = list(shift_layers) if shift_layers is not None else [True] * len(self.shapes)
        self.shift = [torch.zeros(n_slots, width, dtype=torch.float32, device=device) if on else None
                      for on in shift_layers]
        self.rec = [torch.zeros(n_slots, w, dtype=torch.float32, device=device) if w else None for w in rec_widths]
        self.canon_taps = canon_taps
        self.conv = [torch.zeros(n_slots, 2, max(canon_taps - 1, 1), width, dtype=torch.float32, device=device)
                     if canon_taps > 0 else None for _ in self.shapes]
        short_conv = list(short_conv) if short_conv is not None else [None] * len(self.shapes)
        self.sconv = [torch.zeros(n_slots, max(sc[1] - 1, 1), sc[0], dtype=torch.float32, device=device)
                      if sc is not None else None for sc in short_conv]

    @staticmethod
    def bytes_per_block(shapes, block_size, dtype_bytes=2) -> int:   # type: ignore[override]
        return sum(g * (dk + dv) for g, dk, dv in shapes if g) * block_size * dtype_bytes

    def k_layer(self, l: int) -> torch.Tensor:
        return self.k[l]

    def v_layer(self, l: int) -> torch.Tensor:
        return self.v[l]

    def copy_blocks(self, src: List[int], dst: List[int]) -> None:
        si = torch.tensor(src, dtype=torch.int64, device=self.device)
        di = torch.tensor(dst, dtype=torch.int64, device=self.device)
        for t in self.k + self.v:
            if t is not None:
                t.index_copy_(0, di, t.index_select(0, si))

    def state_tensors(self) -> List[torch.Tensor]:
        return [t for t in self.shift + self.rec + self.conv + self.sconv if t is not None]
