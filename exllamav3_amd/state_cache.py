"""
Slot state manager for models whose per-sequence memory is bounded: every sequence that is alive holds one SLOT, and a slot holds, for
each layer, what that layer's mixer declares -- a ring buffer of the last `window` keys and values for sliding-window attention, a
float32 matrix per head for a recurrent (linear-attention) layer.  Slots are handed out on admission, given back when a sequence ends
and used again by the next one; the pool grows by doubling when every slot is taken.  Nothing in a slot has to be cleared on reuse: a
mixer starts a sequence (position 0) from its own initial state and reads only what the sequence's length says is valid.

A mixer whose memory grows with the sequence (attention without a window) declares `PagedSpec` buffers instead: per layer a POOL of pages of
`page_size` tokens shared by all sequences, and one table [slots, pages per slot] that lists, in order, the pages a sequence owns (the same for every
layer: they all hold the same tokens).  Pages are handed out as a sequence grows (in `begin_step`), given back with its slot and used again; the pool
and the table grow by doubling.  Nothing is cleared: a reader takes the sequence's length from the step.

`StepBatch` describes one step of the engine over these slots: the packed rows of all sequences in the step, and where each sequence
stands.  The generator's scheduler and the trace runner both build it through `SlotStateCache.begin_step`.
"""
from __future__ import annotations
from dataclasses import dataclass, field
import torch


@dataclass
class StateSpec:
    """One per-slot buffer of a layer: name, shape per slot, element type."""
    name: str
    shape: tuple
    dtype: torch.dtype


@dataclass
class PagedSpec:
    """One per-token buffer of a layer, kept in pages: name, shape per token, element type.  The pool is [pages, page_size, *shape]."""
    name: str
    shape: tuple
    dtype: torch.dtype


@dataclass
class StepBatch:
    n: int                      # rows in the step
    batch: int                  # sequences in the step
    decode: bool                # every sequence brings exactly one row (mixers read their caches); otherwise every sequence starts at position 0
    max_rows: int               # longest sequence of the step
    tokens: torch.Tensor        # int32 [n]
    cu: torch.Tensor            # int32 [batch + 1], first row of each sequence
    tok_seq: torch.Tensor       # int32 [n]
    tok_pos: torch.Tensor       # int32 [n]
    slots: torch.Tensor         # int32 [batch]
    pos0: torch.Tensor          # int32 [batch], length before the step
    len_after: torch.Tensor     # int32 [batch], length after the step
    want_rows: torch.Tensor | None = None     # int32 [m]: rows whose logits are asked for (may be empty)
    host_lens: list = field(default_factory=list)
    buffer: torch.Tensor | None = None        # the one device array that the tensors above are views of


class SlotStateCache:
    def __init__(self, layer_specs: list[list], device, slots: int = 4, page_size: int = 64, tokens: int = 0):
        """tokens: the most tokens that live sequences hold at once, if known -- sizes the page pools (they grow when it was too small)."""
        self.device = torch.device(device)
        self.layer_specs = [[s for s in specs if isinstance(s, StateSpec)] for specs in layer_specs]
        self.paged_specs = [[s for s in specs if isinstance(s, PagedSpec)] for specs in layer_specs]
        self.capacity = 0
        self.layers: list[dict[str, torch.Tensor]] = [dict() for _ in layer_specs]
        self.free: list[int] = []
        self.length: dict[int, int] = {}         # slot -> tokens held by the sequence that owns it
        self.generation = 0
        self.paged = any(self.paged_specs)
        self.page_size = int(page_size)
        self.num_pages, self.free_pages, self.pages_of = 0, [], {}         # pages_of: slot -> its pages, in order
        self.table_width = 0
        self.page_table = self._table_host = None
        self._grow(max(1, slots))
        if self.paged:
            if self.page_size < 1:
                raise RuntimeError("pages hold at least one token")
            want = -(-int(tokens) // self.page_size) + max(1, slots) if tokens > 0 else 16
            self._grow_table(max(1, -(-int(tokens) // self.page_size)) if tokens > 0 else 4)
            self._grow_pages(want)

    def bytes_per_slot(self) -> int:
        total = 0
        for specs in self.layer_specs:
            for s in specs:
                nel = 1
                for d in s.shape:
                    nel *= d
                total += nel * torch.empty((), dtype=s.dtype).element_size()
        return total

    def _grow(self, new_capacity: int):
        for li, specs in enumerate(self.layer_specs):
            for s in specs:
                buf = torch.zeros((new_capacity,) + tuple(s.shape), dtype=s.dtype, device=self.device)
                old = self.layers[li].get(s.name)
                if old is not None:
                    buf[: self.capacity].copy_(old)
                self.layers[li][s.name] = buf
        self.free.extend(range(new_capacity - 1, self.capacity - 1, -1))      # lowest number on top of the stack
        self.capacity = new_capacity
        self.generation += 1                   # the buffers moved: whoever holds their addresses (captured graphs) starts over
        if self.paged and self.table_width:
            self._grow_table(self.table_width)

    def _grow_table(self, width: int):
        """The page table for `capacity` slots of `width` pages each (host copy + device copy; entries beyond a sequence's pages are 0 and never read)."""
        host = torch.zeros((self.capacity, width), dtype=torch.int32)
        if self._table_host is not None:
            r, c = self._table_host.shape
            host[:r, :c] = self._table_host
        self._table_host, self.table_width = host, width
        self.page_table = host.to(self.device)
        for li, specs in enumerate(self.paged_specs):
            if specs:
                self.layers[li]["page_table"] = self.page_table
        self.generation += 1

    def _grow_pages(self, new_pages: int):
        for li, specs in enumerate(self.paged_specs):
            for s in specs:
                buf = torch.zeros((new_pages, self.page_size) + tuple(s.shape), dtype=s.dtype, device=self.device)
                old = self.layers[li].get(s.name)
                if old is not None:
                    buf[: self.num_pages].copy_(old)
                self.layers[li][s.name] = buf
        self.free_pages.extend(range(new_pages - 1, self.num_pages - 1, -1))
        self.num_pages = new_pages
        self.generation += 1

    def reserve(self, entries: list[tuple[int, list[int]]]):
        """Pages for the tokens that `entries` (slot, next tokens) are about to add.  begin_step calls it; a caller that holds device addresses (captured
        graphs) calls it first and looks at `generation` afterwards."""
        if not self.paged:
            return
        changed = []
        for slot, toks in entries:
            need = -(-(self.length[slot] + len(toks)) // self.page_size)
            own = self.pages_of.setdefault(slot, [])
            if need <= len(own):
                continue
            if need > self.table_width:
                self._grow_table(max(need, 2 * self.table_width))
            while len(own) < need:
                if not self.free_pages:
                    self._grow_pages(max(2 * self.num_pages, 1))
                pg = self.free_pages.pop()
                self._table_host[slot, len(own)] = pg
                own.append(pg)
            changed.append(slot)
        if changed:
            rows = torch.tensor(changed, dtype=torch.int64)
            self.page_table.index_copy_(0, rows.to(self.device), self._table_host[rows].to(self.device))

    def pages_in_use(self) -> int:
        return self.num_pages - len(self.free_pages)

    def alloc(self) -> int:
        if not self.free:
            self._grow(self.capacity * 2)
        slot = self.free.pop()
        self.length[slot] = 0
        return slot

    def release(self, slot: int):
        if slot not in self.length:
            raise RuntimeError(f"slot {slot} is not in use")
        del self.length[slot]
        self.free.append(slot)
        self.free_pages.extend(reversed(self.pages_of.pop(slot, [])))

    def in_use(self) -> int:
        return len(self.length)

    def begin_step(self, entries: list[tuple[int, list[int]]], want: list[list[int]] | None = None, into: StepBatch | None = None) -> StepBatch:
        """entries: (slot, the sequence's next tokens).  Either every sequence is at position 0 (a prompt step) or every sequence brings one
        token (a decode step).  want: per entry, the places among its tokens whose logits are asked for (None: every sequence's last).
        into: a StepBatch of the same layout (same row and sequence counts) whose device buffer is overwritten in place -- a captured graph keeps
        reading the same addresses."""
        lens = [len(t) for _, t in entries]
        if not entries or min(lens) < 1:
            raise RuntimeError("a step needs at least one token per sequence")
        pos0 = [self.length[s] for s, _ in entries]
        decode = all(l == 1 for l in lens) and any(p > 0 for p in pos0)
        if not decode and any(p > 0 for p in pos0):
            raise RuntimeError("a step either starts all its sequences or continues all of them by one token")
        self.reserve(entries)
        n, b = sum(lens), len(entries)
        cu = [0]
        for l in lens:
            cu.append(cu[-1] + l)
        tokens, tok_seq, tok_pos = [], [], []
        for i, (_, t) in enumerate(entries):
            tokens.extend(t)
            tok_seq.extend([i] * len(t))
            tok_pos.extend(range(pos0[i], pos0[i] + len(t)))
        slots = [s for s, _ in entries]
        after = [p + l for p, l in zip(pos0, lens)]
        if want is None:
            rows = [c - 1 for c in cu[1:]]
        else:
            rows = [cu[i] + p for i, w in enumerate(want) for p in w]
        # one host array, one copy: the pieces are views of it on the device
        flat = tokens + cu + tok_seq + tok_pos + slots + pos0 + after + rows
        host = torch.tensor(flat, dtype=torch.int32)
        if into is not None:
            if (into.n, into.batch, into.decode, into.want_rows.numel()) != (n, b, decode, len(rows)) or into.buffer.numel() != len(flat):
                raise RuntimeError("begin_step(into=...): the step has another layout than the one the buffer was made for")
            into.buffer.copy_(host)
            for (s, _), a in zip(entries, after):
                self.length[s] = a
            into.host_lens = lens
            return into
        dev = host.to(self.device, non_blocking=False)
        cuts, at = [], 0
        for ln in (n, b + 1, n, n, b, b, b, len(rows)):
            cuts.append(dev[at: at + ln]); at += ln
        for (s, _), a in zip(entries, after):
            self.length[s] = a
        return StepBatch(n=n, batch=b, decode=decode, max_rows=max(lens), tokens=cuts[0], cu=cuts[1], tok_seq=cuts[2], tok_pos=cuts[3], slots=cuts[4],
                         pos0=cuts[5], len_after=cuts[6], want_rows=cuts[7], host_lens=lens, buffer=dev)
