"""Paged KV-cache manager — HBM3E page pool + pinned-host checkpoints.

The MI355X replacement for the reference's "container keeps its
filesystem + Redis state" durability (SURVEY.md §2.3 "KV-cache manager"
row, §5 Checkpoint/resume):

  * One page pool per model layer in HBM (layouts match the attention
    kernels: k [P, n_kv, D/8, PS, 8], v [P, n_kv, PS, D]).
  * Sequences (= agent conversations) own page lists via a page table.
  * stop/offload gathers a sequence's pages into a contiguous GPU staging
    buffer (ops.gather_kv_pages) and streams it to PINNED host memory with
    a non-blocking copy (hipMemcpyAsync under torch); resume streams it
    back and rebuilds the page table. Checkpoints can also be serialized
    to disk for backup/export.

Sized for 288 GB HBM3E: by default the pool takes the configured fraction
of free device memory after weights.
"""

from __future__ import annotations

import threading
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from .. import ops


class OutOfPages(RuntimeError):
    pass


@dataclass
class Sequence:
    seq_id: str
    pages: List[int] = field(default_factory=list)
    length: int = 0  # tokens written


@dataclass
class KVCheckpoint:
    """Host-side image of one sequence's KV state."""

    length: int
    n_pages: int
    data: torch.Tensor  # pinned host [n_layers, n_pages, page_shorts] bf16
    # per-sequence recurrent state (layouts that keep one): host fp32
    # [n_layers, state_elems]
    state: Optional[torch.Tensor] = None


class GQALayout:
    """Per layer a K pool [P, n_kv, D/8, PS, 8] and a V pool [P, n_kv, PS, D]
    (the layouts the GQA attention kernels stream)."""

    def __init__(self, n_layers: int, n_kv: int, head_dim: int):
        assert head_dim % 8 == 0
        self.n_layers, self.n_kv, self.head_dim = n_layers, n_kv, head_dim

    def alloc(self, n_pages, page_size, device, dtype):
        return [(torch.zeros(n_pages, self.n_kv, self.head_dim // 8,
                             page_size, 8, dtype=dtype, device=device),
                 torch.zeros(n_pages, self.n_kv, page_size, self.head_dim,
                             dtype=dtype, device=device))
                for _ in range(self.n_layers)]

    def page_elems(self, page_size: int) -> int:
        return 2 * self.n_kv * self.head_dim * page_size

    def gather(self, entry, staging, page_ids):
        ops.gather_kv_pages(staging, entry[0], entry[1], page_ids)

    def scatter(self, entry, staging, page_ids):
        ops.scatter_kv_pages(entry[0], entry[1], staging, page_ids)


class LatentLayout:
    """Per layer ONE pool [P, PS, R_l] of cached attention latents (row =
    token); R_l may differ between layers. Checkpoint images are sized by
    the widest layer."""

    def __init__(self, ranks: List[int]):
        self.ranks = list(ranks)
        self.n_layers = len(self.ranks)

    def alloc(self, n_pages, page_size, device, dtype):
        return [(torch.zeros(n_pages, page_size, r, dtype=dtype,
                             device=device),) for r in self.ranks]

    def page_elems(self, page_size: int) -> int:
        return max(self.ranks) * page_size

    def gather(self, entry, staging, page_ids):
        pool = entry[0]
        n = pool.size(1) * pool.size(2)
        staging[:, :n] = pool.index_select(0, page_ids.long()).view(-1, n)

    def scatter(self, entry, staging, page_ids):
        pool = entry[0]
        n = pool.size(1) * pool.size(2)
        pool.index_copy_(0, page_ids.long(),
                         staging[:, :n].reshape(-1, pool.size(1),
                                                pool.size(2)))


class HeadKVLayout:
    """Per layer a K pool [P, G_l, PS, D_l] and a V pool [P, G_l, PS, Dv_l]:
    inside a page every kv head owns PS consecutive token rows, so the
    attention kernels stream one contiguous block per (page, head). The
    head count and the key / value sizes may differ from layer to layer
    and from each other. Checkpoint images are sized by the widest layer."""

    def __init__(self, shapes):
        # shapes: per layer (kv_heads, key_dim, value_dim)
        self.shapes = [tuple(int(v) for v in s) for s in shapes]
        self.n_layers = len(self.shapes)

    def alloc(self, n_pages, page_size, device, dtype):
        return [(torch.zeros(n_pages, g, page_size, d, dtype=dtype,
                             device=device),
                 torch.zeros(n_pages, g, page_size, dv, dtype=dtype,
                             device=device))
                for g, d, dv in self.shapes]

    def page_elems(self, page_size: int) -> int:
        return max(g * (d + dv) for g, d, dv in self.shapes) * page_size

    def gather(self, entry, staging, page_ids):
        ids = page_ids.long()
        nk = entry[0][0].numel()
        nv = entry[1][0].numel()
        staging[:, :nk] = entry[0].index_select(0, ids).view(-1, nk)
        staging[:, nk:nk + nv] = entry[1].index_select(0, ids).view(-1, nv)

    def scatter(self, entry, staging, page_ids):
        ids = page_ids.long()
        nk = entry[0][0].numel()
        nv = entry[1][0].numel()
        entry[0].index_copy_(0, ids, staging[:, :nk].reshape(
            -1, *entry[0].shape[1:]))
        entry[1].index_copy_(0, ids, staging[:, nk:nk + nv].reshape(
            -1, *entry[1].shape[1:]))


class HybridStateLayout:
    """Layers that cache per-token K/V pages, per-SEQUENCE state, or both.

    kv_shapes[l] is (kv_heads, key_dim, value_dim) — pools as in
    HeadKVLayout —, a 1-tuple (rank,) — one latent pool [P, PS, rank] as
    in LatentLayout, handed out as (pool, None) —, or None for a layer
    that caches nothing per token (no attention, or attention that reads
    another layer's pools). state_shapes[l]
    maps a name to the shape of one sequence's state tensor of that
    layer (a recurrent memory, the tail of a short convolution, the last
    token id); the manager allocates each as [slots, *shape], indexed by
    the sequence slot, so a sequence's state is addressed on the device by
    the same number as its page-table row. States are fp32 unless
    state_dtypes[l] names another dtype (integers below 2^24 survive the
    fp32 checkpoint image). The kernels treat a sequence that starts at
    position 0 as having zero state, so a slot needs no clearing when it
    is handed to the next sequence."""

    def __init__(self, kv_shapes, state_shapes, state_dtypes=None):
        self.kv_shapes = [None if s is None else tuple(int(v) for v in s)
                          for s in kv_shapes]
        self.state_shapes = [{k: tuple(int(x) for x in v)
                              for k, v in d.items()} for d in state_shapes]
        self.state_dtypes = (state_dtypes if state_dtypes is not None
                             else [{} for _ in self.state_shapes])
        assert len(self.kv_shapes) == len(self.state_shapes)
        assert len(self.state_dtypes) == len(self.state_shapes)
        self.n_layers = len(self.kv_shapes)

    def alloc(self, n_pages, page_size, device, dtype):
        out = []
        for s in self.kv_shapes:
            if s is None:
                out.append((None, None))
            elif len(s) == 1:
                out.append((torch.zeros(n_pages, page_size, s[0], dtype=dtype,
                                        device=device), None))
            else:
                g, d, dv = s
                out.append((torch.zeros(n_pages, g, page_size, d, dtype=dtype,
                                        device=device),
                            torch.zeros(n_pages, g, page_size, dv, dtype=dtype,
                                        device=device)))
        return out

    def alloc_state(self, n_slots, device):
        return [{k: torch.zeros(n_slots, *shape,
                                dtype=dt.get(k, torch.float32),
                                device=device) for k, shape in d.items()}
                for d, dt in zip(self.state_shapes, self.state_dtypes)]

    def page_elems(self, page_size: int) -> int:
        return max([s[0] if len(s) == 1 else s[0] * (s[1] + s[2])
                    for s in self.kv_shapes if s is not None] + [1]
                   ) * page_size

    def state_elems(self) -> int:
        """fp32 values of one sequence's state in the largest layer."""
        n = 0
        for d in self.state_shapes:
            tot = 0
            for shape in d.values():
                e = 1
                for x in shape:
                    e *= x
                tot += e
            n = max(n, tot)
        return n

    def state_bytes_per_seq(self) -> int:
        tot = 0
        for d in self.state_shapes:
            for shape in d.values():
                e = 4
                for x in shape:
                    e *= x
                tot += e
        return tot

    def gather(self, entry, staging, page_ids):
        if entry[0] is None:
            return
        if entry[1] is None:
            LatentLayout.gather(self, entry, staging, page_ids)
        else:
            HeadKVLayout.gather(self, entry, staging, page_ids)

    def scatter(self, entry, staging, page_ids):
        if entry[0] is None:
            return
        if entry[1] is None:
            LatentLayout.scatter(self, entry, staging, page_ids)
        else:
            HeadKVLayout.scatter(self, entry, staging, page_ids)

    def gather_state(self, state, slot: int, row: torch.Tensor) -> None:
        """One layer's state of `slot` -> flat fp32 row."""
        off = 0
        for k in sorted(state):
            t = state[k][slot].reshape(-1)
            row[off:off + t.numel()] = t.to(row.dtype)
            off += t.numel()

    def scatter_state(self, state, slot: int, row: torch.Tensor) -> None:
        off = 0
        for k in sorted(state):
            n = state[k][slot].numel()
            state[k][slot] = row[off:off + n].view(state[k].shape[1:]).to(
                device=state[k].device, dtype=state[k].dtype)
            off += n


class KVCacheManager:
    def __init__(self, n_layers: int, n_kv: int, head_dim: int, page_size: int,
                 n_pages: int, device="cpu", dtype=torch.bfloat16,
                 max_slots: int = 1024, max_pages_per_seq: int = 512,
                 mirrors: Optional[bool] = None, layout=None):
        # layout: what one layer caches per page (default: GQA K/V planes)
        self.layout = layout or GQALayout(n_layers, n_kv, head_dim)
        n_layers = self.layout.n_layers
        self.n_layers = n_layers
        self.n_kv = n_kv
        self.head_dim = head_dim
        self.page_size = page_size
        self.n_pages = n_pages
        self.device = device
        # dtype: bf16 (default) or float8_e4m3fn — fp8 halves KV bytes per
        # token (2x the agents per GPU) with OCP e4m3 storage, vLLM-style
        # scale-free semantics (e4m3 range +-448 covers post-norm K/V)
        self.dtype = dtype
        self.caches = self.layout.alloc(n_pages, page_size, device, dtype)
        # per-sequence-slot state (recurrent memories, convolution tails)
        # of layouts that keep one: per layer a dict name -> [slots, ...]
        self.states = (self.layout.alloc_state(max_slots, device)
                       if hasattr(self.layout, "alloc_state") else None)
        if isinstance(self.layout, GQALayout):
            self.k_caches: List[torch.Tensor] = [c[0] for c in self.caches]
            self.v_caches: List[torch.Tensor] = [c[1] for c in self.caches]
        # page 0 is reserved as the scratch page: hipGraph-padded decode rows
        # write their garbage K/V there (see llm.ModelInstance._device_decode)
        self._free: List[int] = list(range(n_pages - 1, 0, -1))
        self._seqs: Dict[str, Sequence] = {}
        # copy-on-write refcounts for SHARED pages (prefix sharing). A page
        # absent from the map has exactly one owner; adopt_prefix bumps the
        # count, release decrements and only returns a page to the pool when
        # its last owner lets go. Shared pages are never written: adopters
        # take only FULL pages, and appends always land at slot >= length,
        # which is past the shared region by construction.
        self._refs: Dict[int, int] = {}
        self._lock = threading.RLock()
        # shorts per page per layer: K plane + V plane
        self.page_shorts = self.layout.page_elems(page_size)
        # ---- device mirrors for the in-graph decode step ----
        # dev_page_table[slot] / dev_seq_lens[slot] are the ground truth the
        # captured decode graph reads; host bookkeeping mirrors them. On GPU
        # they live in HBM; `mirrors=True` on CPU materializes them as CPU
        # tensors so the device-decode path (and the async-TP protocol on
        # top of it) is testable without hardware.
        self.is_gpu = str(device) not in ("cpu",)
        self.mirrors = self.is_gpu if mirrors is None else bool(mirrors)
        self.max_slots = max_slots
        self.max_pages_per_seq = max_pages_per_seq
        if self.mirrors:
            self.dev_page_table = torch.zeros(max_slots, max_pages_per_seq,
                                              dtype=torch.int32, device=device)
            self.dev_seq_lens = torch.full((max_slots,), -1, dtype=torch.int32,
                                           device=device)
        else:
            self.dev_page_table = None
            self.dev_seq_lens = None
        # slots are assigned on CPU too: slot allocation is deterministic
        # across TP ranks (same create/free order), so the slot id doubles
        # as the wire identity of a sequence in binary step plans
        self._free_slots: List[int] = list(range(max_slots - 1, -1, -1))
        self._slot_of: Dict[str, int] = {}
        self._seq_of_slot: Dict[int, str] = {}

    # ---------- queries ----------

    @property
    def free_pages(self) -> int:
        with self._lock:
            return len(self._free)

    @property
    def used_pages(self) -> int:
        return self.n_pages - self.free_pages

    def kv_caches(self) -> List[Tuple[torch.Tensor, torch.Tensor]]:
        """Per layer what the model's forward reads and writes: the page
        pools, followed by the layer's state dict where the layout keeps
        per-sequence state."""
        if self.states is not None:
            return [tuple(c) + (st,) for c, st in zip(self.caches, self.states)]
        return list(self.caches)

    def has_seq(self, seq_id: str) -> bool:
        with self._lock:
            return seq_id in self._seqs

    def seq_len(self, seq_id: str) -> int:
        with self._lock:
            s = self._seqs.get(seq_id)
            return s.length if s else 0

    def seq_bytes(self, seq_id: str) -> int:
        with self._lock:
            s = self._seqs.get(seq_id)
            if not s:
                return 0
            return (len(s.pages) * self.page_shorts * self.n_layers *
                    torch.empty(0, dtype=self.dtype).element_size())

    # ---------- allocation ----------

    def create_seq(self, seq_id: str) -> Sequence:
        with self._lock:
            if seq_id in self._seqs:
                raise ValueError(f"sequence {seq_id} exists")
            if not self._free_slots:
                # check BEFORE registering: raising after the _seqs insert
                # left a zombie slotless entry behind (found by the
                # stateful fuzz in tests/test_kvcache_properties.py)
                raise OutOfPages("no free sequence slots")
            s = Sequence(seq_id)
            self._seqs[seq_id] = s
            slot = self._free_slots.pop()
            self._slot_of[seq_id] = slot
            self._seq_of_slot[slot] = seq_id
            if self.mirrors:
                self.dev_seq_lens[slot] = 0
            return s

    def slot(self, seq_id: str) -> int:
        return self._slot_of[seq_id]

    def seq_of_slot(self, slot: int) -> str:
        """Inverse of slot(): wire identity -> sequence (TP worker plans)."""
        with self._lock:
            return self._seq_of_slot[slot]

    def push_dev(self, seq_id: str) -> None:
        """Sync a sequence's page row + length to the device mirrors."""
        if not self.mirrors:
            return
        with self._lock:
            s = self._seqs[seq_id]
            slot = self._slot_of[seq_id]
            if s.pages:
                self.dev_page_table[slot, :len(s.pages)] = torch.tensor(
                    s.pages, dtype=torch.int32, device=self.device)
            self.dev_seq_lens[slot] = s.length

    def ensure_decode_page(self, seq_id: str) -> None:
        """Host half of the in-graph decode append: guarantee the page for
        the NEXT token exists (the graph computes the slot on device)."""
        with self._lock:
            s = self._seqs[seq_id]
            page_idx = s.length // self.page_size
            if page_idx >= self.max_pages_per_seq:
                raise OutOfPages("sequence exceeded max_pages_per_seq")
            if page_idx >= len(s.pages):
                if not self._free:
                    raise OutOfPages(f"KV pool exhausted ({self.n_pages} pages)")
                page = self._free.pop()
                s.pages.append(page)
                if self.mirrors:
                    self.dev_page_table[self._slot_of[seq_id], page_idx] = page

    def advance_host(self, seq_id: str) -> None:
        """Host length += 1 after an in-graph decode step incremented the
        device length."""
        with self._lock:
            self._seqs[seq_id].length += 1

    def decode_batch_prepare(self, seq_ids) -> list:
        """One-lock batch form of ensure_decode_page: guarantees each
        sequence's next-token page exists; returns the slot indices."""
        rows = []
        with self._lock:
            for seq_id in seq_ids:
                s = self._seqs[seq_id]
                page_idx = s.length // self.page_size
                if page_idx >= self.max_pages_per_seq:
                    raise OutOfPages("sequence exceeded max_pages_per_seq")
                if page_idx >= len(s.pages):
                    if not self._free:
                        raise OutOfPages(
                            f"KV pool exhausted ({self.n_pages} pages)")
                    page = self._free.pop()
                    s.pages.append(page)
                    if self.mirrors:
                        self.dev_page_table[self._slot_of[seq_id],
                                            page_idx] = page
                rows.append(self._slot_of[seq_id])
        return rows

    def advance_many(self, seq_ids) -> None:
        with self._lock:
            for seq_id in seq_ids:
                self._seqs[seq_id].length += 1

    def rollback_many(self, seq_ids) -> None:
        """Undo one speculative decode append per sequence (async decode:
        a row that turned out finished had a garbage token appended by the
        in-flight step). Device decrement is stream-ordered after that
        step's graph, so it lands exactly once the append has happened."""
        if not seq_ids:
            return
        with self._lock:
            slots = []
            for seq_id in seq_ids:
                self._seqs[seq_id].length -= 1
                if self.mirrors:
                    slots.append(self._slot_of[seq_id])
        if self.mirrors and slots:
            idx = torch.tensor(slots, dtype=torch.long, device=self.device)
            self.dev_seq_lens.index_add_(
                0, idx, torch.full((len(slots),), -1, dtype=torch.int32,
                                   device=self.device))

    def adopt_prefix(self, seq_id: str, src_seq_id: str, n_tokens: int) -> None:
        """Share the first n_tokens (a whole number of pages) of src with an
        EMPTY sequence — copy-on-write prefix sharing for agents with a
        common system prompt. The adopter's page table points at the shared
        pages; its subsequent appends land past the shared region (length
        starts at n_tokens, a page boundary), so the shared pages stay
        read-only. Refcounts keep them alive until the last owner frees."""
        with self._lock:
            src = self._seqs[src_seq_id]
            dst = self._seqs[seq_id]
            if dst.length != 0:
                raise ValueError(f"adopt_prefix: {seq_id} is not empty")
            if n_tokens % self.page_size != 0 or n_tokens <= 0:
                raise ValueError("adopt_prefix: n_tokens must be whole pages")
            n_pg = n_tokens // self.page_size
            if src.length < n_tokens or len(src.pages) < n_pg:
                raise ValueError("adopt_prefix: source prefix too short")
            shared = src.pages[:n_pg]
            for p in shared:
                self._refs[p] = self._refs.get(p, 1) + 1
            # pages already attached at length 0 are admission reservations
            # (reserve()) sized for the FULL prompt; the shared prefix now
            # supplies the first n_pg pages' worth, so release exactly that
            # surplus and keep the rest as the post-prefix tail
            tail = dst.pages
            for _ in range(min(n_pg, len(tail))):
                self._free.append(tail.pop())
            dst.pages = list(shared) + tail
            dst.length = n_tokens
            if self.mirrors:
                slot = self._slot_of[seq_id]
                self.dev_page_table[slot, :len(dst.pages)] = torch.tensor(
                    dst.pages, dtype=torch.int32, device=self.device)
                self.dev_seq_lens[slot] = n_tokens

    def _release_pages(self, pages: List[int]) -> None:
        """Return pages to the pool, honoring shared-page refcounts. Caller
        holds the lock."""
        for p in reversed(pages):
            c = self._refs.get(p)
            if c is None:
                self._free.append(p)       # sole owner — really free
            elif c <= 2:
                del self._refs[p]          # one owner left; unshared again
            else:
                self._refs[p] = c - 1

    def free_seq(self, seq_id: str) -> None:
        with self._lock:
            s = self._seqs.pop(seq_id, None)
            if s:
                self._release_pages(s.pages)
            slot = self._slot_of.pop(seq_id, None)
            if slot is not None:
                self._seq_of_slot.pop(slot, None)
                if self.mirrors:
                    self.dev_seq_lens[slot] = -1
                self._free_slots.append(slot)

    def reset_seq(self, seq_id: str) -> None:
        """Drop a sequence's KV but keep it registered (context truncation)."""
        with self._lock:
            s = self._seqs[seq_id]
            self._release_pages(s.pages)
            s.pages = []
            s.length = 0
            if self.mirrors:
                self.dev_seq_lens[self._slot_of[seq_id]] = 0

    def reserve(self, seq_id: str, n_tokens: int) -> None:
        """Pre-allocate pages covering n_tokens future appends (chunked
        prefill admission: room for the whole prompt+generation is claimed
        up front, so other agents admitted between chunks cannot starve a
        half-prefilled sequence into OutOfPages mid-plan). Raises
        OutOfPages atomically — no pages are taken on failure."""
        with self._lock:
            s = self._seqs[seq_id]
            need_pages = -(-(s.length + n_tokens) // self.page_size)
            if need_pages > self.max_pages_per_seq:
                raise OutOfPages("sequence would exceed max_pages_per_seq")
            short = need_pages - len(s.pages)
            if short <= 0:
                return
            if short > len(self._free):
                raise OutOfPages(f"KV pool exhausted ({self.n_pages} pages)")
            start = len(s.pages)
            taken = self._free[-short:][::-1]  # same order as a pop() loop
            del self._free[-short:]
            s.pages.extend(taken)
            if self.mirrors:
                # one batched mirror write — per-page scalar assigns cost
                # a tiny H2D launch EACH (visible in the admit phase)
                self.dev_page_table[self._slot_of[seq_id],
                                    start:start + short] = torch.tensor(
                    taken, dtype=torch.int32, device=self.device)

    def can_append(self, seq_id: str, n_tokens: int) -> bool:
        with self._lock:
            s = self._seqs[seq_id]
            have = len(s.pages) * self.page_size - s.length
            need_pages = max(0, -(-(n_tokens - have) // self.page_size))
            return need_pages <= len(self._free)

    def can_append_after_reset(self, seq_id: str, n_tokens: int) -> bool:
        """Would n_tokens fit if this sequence's pages were freed first?
        Shared (refcounted) pages don't return to the pool on reset."""
        with self._lock:
            s = self._seqs[seq_id]
            need_pages = -(-n_tokens // self.page_size)
            freeable = sum(1 for p in s.pages if p not in self._refs)
            return need_pages <= len(self._free) + freeable

    def append_slots(self, seq_id: str, n_tokens: int) -> List[int]:
        """Reserve slots for n_tokens new tokens; allocates pages as needed.
        Returns global slot ids (page * page_size + offset)."""
        with self._lock:
            s = self._seqs[seq_id]
            slots = []
            for _ in range(n_tokens):
                if s.length == len(s.pages) * self.page_size:
                    if not self._free:
                        raise OutOfPages(
                            f"KV pool exhausted ({self.n_pages} pages)")
                    s.pages.append(self._free.pop())
                page = s.pages[s.length // self.page_size]
                off = s.length % self.page_size
                slots.append(page * self.page_size + off)
                s.length += 1
            return slots

    def page_table(self, seq_ids: List[str], device=None) -> torch.Tensor:
        """int32 [B, max_pages_in_batch] (padded with 0)."""
        with self._lock:
            rows = [self._seqs[sid].pages for sid in seq_ids]
        width = max((len(r) for r in rows), default=1) or 1
        t = torch.zeros(len(rows), width, dtype=torch.int32)
        for i, r in enumerate(rows):
            if r:
                t[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
        return t.to(device or self.device)

    def seq_lens(self, seq_ids: List[str], device=None) -> torch.Tensor:
        with self._lock:
            lens = [self._seqs[sid].length for sid in seq_ids]
        return torch.tensor(lens, dtype=torch.int32, device=device or self.device)

    # ---------- checkpoint (stop/resume, crash recovery) ----------

    def offload(self, seq_id: str, free: bool = True) -> Optional[KVCheckpoint]:
        """Gather the sequence's pages and stream them to pinned host memory."""
        with self._lock:
            s = self._seqs.get(seq_id)
            if s is None or not s.pages:
                if free and s is not None:
                    self.free_seq(seq_id)
                return None
            pages = list(s.pages)
            length = s.length
            slot = self._slot_of[seq_id]
        n = len(pages)
        state = None
        if self.states is not None:
            state = torch.zeros(self.n_layers, self.layout.state_elems(),
                                dtype=torch.float32)
            for li in range(self.n_layers):
                row = torch.zeros(state.size(1), dtype=torch.float32,
                                  device=self.device)
                self.layout.gather_state(self.states[li], slot, row)
                state[li].copy_(row)
        page_ids = torch.tensor(pages, dtype=torch.int32, device=self.device)
        is_gpu = str(self.device) not in ("cpu",)
        host = torch.empty(self.n_layers, n, self.page_shorts, dtype=self.dtype,
                           pin_memory=is_gpu)
        if is_gpu:
            staging = torch.empty(n, self.page_shorts, dtype=self.dtype,
                                  device=self.device)
            for li in range(self.n_layers):
                self.layout.gather(self.caches[li], staging, page_ids)
                host[li].copy_(staging, non_blocking=True)
            torch.cuda.synchronize()
        else:
            staging = torch.empty(n, self.page_shorts, dtype=self.dtype)
            for li in range(self.n_layers):
                self.layout.gather(self.caches[li], staging, page_ids)
                host[li].copy_(staging)
        if free:
            self.free_seq(seq_id)
        return KVCheckpoint(length=length, n_pages=n, data=host, state=state)

    def restore(self, seq_id: str, ckpt: Optional[KVCheckpoint]) -> None:
        """Upload a checkpoint into freshly allocated pages."""
        with self._lock:
            if seq_id in self._seqs:
                self.free_seq(seq_id)
            s = self.create_seq(seq_id)
            if ckpt is None or ckpt.n_pages == 0:
                return
            if len(self._free) < ckpt.n_pages:
                raise OutOfPages("not enough pages to restore checkpoint")
            s.pages = [self._free.pop() for _ in range(ckpt.n_pages)]
            s.length = ckpt.length
            pages = list(s.pages)
            slot = self._slot_of[seq_id]
        if self.states is not None and ckpt.state is not None:
            for li in range(self.n_layers):
                self.layout.scatter_state(self.states[li], slot,
                                          ckpt.state[li].to(self.device))
        page_ids = torch.tensor(pages, dtype=torch.int32, device=self.device)
        is_gpu = str(self.device) not in ("cpu",)
        for li in range(self.n_layers):
            staging = ckpt.data[li].to(self.device, non_blocking=is_gpu)
            self.layout.scatter(self.caches[li], staging, page_ids)
        self.push_dev(seq_id)
        if is_gpu:
            torch.cuda.synchronize()
