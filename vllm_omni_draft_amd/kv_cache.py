"""Paged KV cache storage and page allocation.

Page = 16 tokens of one KV head; layouts are documented in include/sd_amd.h.
The cache is zero-filled at allocation (the attention kernel reads unwritten
slots of a partly filled page and masks them, so they must be finite).
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .config import ModelConfig

PAGE = 16


class OutOfPages(RuntimeError):
    pass


class PageAllocator:
    """Free-list allocator of cache pages shared by the sequences of one model."""

    def __init__(self, num_pages: int):
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("KV cache is out of pages")
        return self._free.pop()

    def free(self, pages: List[int]) -> None:
        self._free.extend(pages)


class PagedKVCache:
    """K and V pages of every layer of one model, plus the block tables of the
    running batch as a device tensor."""

    def __init__(self, cfg: ModelConfig, num_pages: int, max_batch: int, max_seq_len: int,
                 device="cuda"):
        self.cfg = cfg
        self.num_pages = num_pages
        self.max_blocks_per_seq = (max_seq_len + PAGE - 1) // PAGE
        page_elems = cfg.head_dim * PAGE
        shape = (cfg.n_layers, num_pages, cfg.n_kv_heads, page_elems)
        self.k = torch.zeros(shape, dtype=torch.bfloat16, device=device)
        self.v = torch.zeros(shape, dtype=torch.bfloat16, device=device)
        self.layer_stride_bytes = num_pages * cfg.n_kv_heads * page_elems * 2
        self.allocator = PageAllocator(num_pages)
        self.block_tables = torch.zeros(max_batch, self.max_blocks_per_seq, dtype=torch.int32,
                                        device=device)
        self._host_tables: List[List[int]] = [[] for _ in range(max_batch)]

    def pages_of(self, slot: int) -> List[int]:
        return self._host_tables[slot]

    def ensure_capacity(self, slot: int, n_tokens: int, grow_to: int = 0) -> None:
        """Makes sure batch slot `slot` owns pages for positions 0..n_tokens-1.  When pages
        must be added anyway, grow_to > n_tokens takes pages for that many tokens at once
        (as far as free pages allow)."""
        need = (n_tokens + PAGE - 1) // PAGE
        if need > self.max_blocks_per_seq:
            raise OutOfPages(f"sequence of {n_tokens} tokens exceeds max_seq_len")
        tbl = self._host_tables[slot]
        if len(tbl) >= need:
            return
        first_new = len(tbl)
        while len(tbl) < need:
            tbl.append(self.allocator.alloc())
        want = min((grow_to + PAGE - 1) // PAGE, self.max_blocks_per_seq)
        while len(tbl) < want and self.allocator.num_free > 0:
            tbl.append(self.allocator.alloc())
        need = len(tbl)
        new = torch.tensor(tbl[first_new:], dtype=torch.int32)
        self.block_tables[slot, first_new:need].copy_(new, non_blocking=True)

    def release(self, slot: int) -> None:
        self.allocator.free(self._host_tables[slot])
        self._host_tables[slot] = []

    def move_slot(self, src: int, dst: int) -> None:
        """Batch slot `dst` (empty) takes over the pages of slot `src`."""
        if self._host_tables[dst]:
            raise ValueError(f"slot {dst} still owns pages")
        self._host_tables[dst] = self._host_tables[src]
        self._host_tables[src] = []
        self.block_tables[dst].copy_(self.block_tables[src])

    def swap_slots(self, a: int, b: int) -> None:
        """Batch slots a and b exchange their pages (either may be empty)."""
        if a == b:
            return
        self._host_tables[a], self._host_tables[b] = self._host_tables[b], self._host_tables[a]
        row = self.block_tables[a].clone()
        self.block_tables[a].copy_(self.block_tables[b])
        self.block_tables[b].copy_(row)

    @staticmethod
    def pages_for(cfg: ModelConfig, max_batch: int, max_seq_len: int) -> int:
        return max_batch * ((max_seq_len + PAGE - 1) // PAGE)

    def nbytes(self) -> int:
        return 2 * self.k.numel() * 2


# ---------------------------------------------------------------------------------------------
# Caches of layer-list models (config.SeqModelConfig): per-sequence recurrent states in slots, and
# pages of plain key / value rows (plus pooled rows) for windowed attention layers.
class OutOfSlots(RuntimeError):
    pass


class SlotAllocator:
    """Sequence slots: the row of a block table, and of every recurrent layer's state tensor."""

    def __init__(self, n: int):
        self.n = n
        self._free = list(range(n - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfSlots("every sequence slot is taken")
        return self._free.pop()

    def free(self, slot: int) -> None:
        if slot in self._free:
            raise ValueError(f"slot {slot} is free already")
        self._free.append(slot)


class SeqCache:
    """What the sequences of a layer-list model keep on the device.

    Recurrent layers: state[layer] f32 [slots, heads, dim, vdim]; a slot's state needs no clearing
    when the slot is taken again (a sequence that starts at position 0 starts from zero).
    Window layers: k / v [pages, kv_heads, PAGE, dim | vdim] in the serving dtype and the pooled
    means pk / pv f32 [pages, kv_heads, pooled slots per page, dim | vdim]; one page table per
    slot serves all window layers.  Latent attention keeps one row [kv_rank + rot_dim] per token
    in k only; a state-space recurrence keeps state[layer] [slots, heads, state, vdim] and the
    tail of its convolution's inputs conv[layer] f32 [slots, taps - 1, channels].  The tensors are
    keyed by the layer's place in the order of running (cfg.runs): a layer that runs several
    times over keeps a cache for every pass.  A softmax attention with several score maps per head
    keeps that many key rows per kv head and token (cache head = kv head * maps + map) and one value
    row; a layer that reads another layer's keys and values owns no tensors: kv_source names the
    run whose tensors it reads."""

    def __init__(self, cfg, dtype: torch.dtype, max_seqs: int, num_pages: int, max_seq_len: int,
                 device="cuda"):
        from . import ops
        self.cfg, self.dtype = cfg, dtype
        self.page = PAGE
        self.slots = SlotAllocator(max_seqs)
        self.allocator = PageAllocator(num_pages)
        self.max_blocks_per_seq = max(1, (max_seq_len + PAGE - 1) // PAGE)
        self.block_tables = torch.zeros(max_seqs, self.max_blocks_per_seq, dtype=torch.int32, device=device)
        self._host_tables: List[List[int]] = [[] for _ in range(max_seqs)]
        self.state: Dict[int, torch.Tensor] = {}
        self.k: Dict[int, torch.Tensor] = {}
        self.v: Dict[int, torch.Tensor] = {}
        self.pk: Dict[int, torch.Tensor] = {}
        self.pv: Dict[int, torch.Tensor] = {}
        self.conv: Dict[int, torch.Tensor] = {}
        self.kv_source: Dict[int, int] = {}
        self.has_pages = False
        run_of = {li: i for i, (li, _) in enumerate(cfg.runs)}   # (a layer others read runs once)
        for i, (li, _) in enumerate(cfg.runs):
            m = cfg.layers[li].mixer
            if m.kv_from >= 0:
                self.has_pages = True
                self.kv_source[i] = run_of[m.kv_from]
                continue
            if m.kind == "latent_attention":
                # one row per token serves as key and value: the latent, then the shared rotated part
                self.has_pages = True
                self.k[i] = torch.zeros(num_pages, 1, PAGE, m.kv_rank + m.rot_dim, dtype=dtype, device=device)
            elif m.kind == "parallel":
                self.has_pages = True
                sd = m.ssd
                self.k[i] = torch.zeros(num_pages, m.kv_heads, PAGE, m.dim, dtype=dtype, device=device)
                self.v[i] = torch.zeros(num_pages, m.kv_heads, PAGE, m.vdim, dtype=dtype, device=device)
                self.state[i] = torch.zeros(max_seqs, sd.heads, sd.state, sd.vdim, dtype=torch.float32, device=device)
                self.conv[i] = torch.zeros(max_seqs, max(sd.taps - 1, 1), sd.conv_channels, dtype=torch.float32,
                                           device=device)
            elif m.kind == "softmax_attention":
                self.has_pages = True
                self.k[i] = torch.zeros(num_pages, m.kv_heads * m.maps, PAGE, m.dim, dtype=dtype, device=device)
                self.v[i] = torch.zeros(num_pages, m.kv_heads, PAGE, m.vdim, dtype=dtype, device=device)
            elif m.kind == "attention":
                self.has_pages = True
                ps = ops.pooled_slots_per_page(PAGE, m.pool)
                self.k[i] = torch.zeros(num_pages, m.kv_heads, PAGE, m.dim, dtype=dtype, device=device)
                self.v[i] = torch.zeros(num_pages, m.kv_heads, PAGE, m.vdim, dtype=dtype, device=device)
                self.pk[i] = torch.zeros(num_pages, m.kv_heads, ps, m.dim, dtype=torch.float32, device=device)
                self.pv[i] = torch.zeros(num_pages, m.kv_heads, ps, m.vdim, dtype=torch.float32, device=device)
            else:
                self.state[i] = torch.zeros(max_seqs, m.heads, m.dim, m.vdim, dtype=torch.float32, device=device)

    def keys_of(self, run: int):
        """The key cache run `run` reads: its own, or the one of the run it shares with."""
        return self.k.get(self.kv_source.get(run, run))

    def values_of(self, run: int):
        return self.v.get(self.kv_source.get(run, run))

    def pages_of(self, slot: int) -> List[int]:
        return self._host_tables[slot]

    def ensure_capacity(self, slot: int, n_tokens: int) -> None:
        """Slot `slot` owns pages for positions 0..n_tokens-1 afterwards (window layers only)."""
        if not self.has_pages:
            return
        need = (n_tokens + PAGE - 1) // PAGE
        if need > self.max_blocks_per_seq:
            raise OutOfPages(f"sequence of {n_tokens} tokens exceeds max_seq_len")
        tbl = self._host_tables[slot]
        if len(tbl) >= need:
            return
        if need - len(tbl) > self.allocator.num_free:
            raise OutOfPages("KV cache is out of pages")
        first_new = len(tbl)
        while len(tbl) < need:
            tbl.append(self.allocator.alloc())
        self.block_tables[slot, first_new:need].copy_(torch.tensor(tbl[first_new:], dtype=torch.int32),
                                                      non_blocking=False)

    def release(self, slot: int) -> None:
        self.allocator.free(self._host_tables[slot])
        self._host_tables[slot] = []
        self.slots.free(slot)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for d in (self.state, self.k, self.v, self.pk, self.pv, self.conv)
                   for t in d.values())
