"""Cache manager of models that carry more than keys and values: a page pool per attention layer
(each with its own head count and key / value widths) next to fixed-size recurrent state per
sequence, held in numbered slots.  It stands beside KVCacheManager (core/cache_manager.py), which
serves the Llama-shaped family with one geometry for all layers and whole-prompt allocation; here a
sequence grows by any number of tokens per step (a prompt's portion or one decoded token), its pages
are taken when a step first needs them and its slot when it is admitted, and both go back to their
free lists when it ends.  Nothing is cleared on reuse: a page row is written before a step reads it,
and the kernels take the state of a sequence that has no tokens yet as zero.

`plan()` lays one step out for the kernels (csrc/seq_mix.hip): tokens of all rows back to back with
each token's row, position and predecessor (a sequence's last token is kept on the host between steps,
for embeddings that look at pairs of tokens), per row its first token, length, tokens held before, slot,
and its row of the block table - one pinned staging buffer and one host-to-device copy per step.
"""
import collections
from dataclasses import dataclass
from typing import Dict, List, Sequence as Seq, Tuple

import torch


@dataclass
class RaggedStep:
    tokens: int
    rows: int
    page: int
    ids: torch.Tensor          # int32 [T]
    tok_row: torch.Tensor      # int32 [T]
    tok_pos: torch.Tensor      # int32 [T]
    tok_prev: torch.Tensor     # int32 [T] the token before each token in its sequence, -1 at position 0
    row_start: torch.Tensor    # int32 [B]
    row_len: torch.Tensor
    row_ctx: torch.Tensor
    row_slot: torch.Tensor
    block_table: torch.Tensor  # int32 [B, W]
    max_slot: int              # host copies of what the kernels will index with, for the wrappers' checks
    max_page: int
    # rows of more than SCAN_SEQ_MAX tokens cut into chunks of SCAN_CHUNK for the chunked recurrence
    n_chunks: int = 0
    ch_start: torch.Tensor = None   # int32 [chunks] first token of the chunk (index into the step)
    ch_len: torch.Tensor = None     # int32 [chunks]
    row_ch0: torch.Tensor = None    # int32 [B] the row's first chunk
    row_nch: torch.Tensor = None    # int32 [B] its number of chunks (0: a short row)
    slots: tuple = ()               # host copy of row_slot
    short_tokens: int = -1          # tokens in rows of up to SCAN_SEQ_MAX tokens (the rows outside the chunk table); -1: unknown


from ..kernel.ragged_ops import SCAN_SEQ_MAX  # noqa: E402  rows up to this length are not cut into chunks

SCAN_CHUNK = 64      # csrc/seq_mix.hip kCh


class PoolExhausted(RuntimeError):
    """No page or no state slot is free for `seq_id`; nothing of the step was booked."""

    def __init__(self, seq_id, what):
        super().__init__(f"no free {what} for sequence {seq_id}")
        self.seq_id, self.what = seq_id, what


class HybridCacheManager:
    def __init__(self, n_pages: int, page_size: int, n_slots: int, kv_layers: Dict[int, Tuple[int, int, int]],
                 state_layers: Dict[int, Dict[str, Tuple[int, ...]]], dtype=torch.bfloat16, device="cuda",
                 max_tokens: int = 4096, max_rows: int = 32, max_step_tokens: int = 8192):
        """kv_layers: layer run -> (kv_heads, key width, value width; 0 = no separate values); state_layers: layer run ->
        {name: shape per slot} (fp32).  `max_tokens`: the longest sequence a block-table row
        describes."""
        self.n_pages, self.page_size, self.n_slots = n_pages, page_size, n_slots
        self.dtype, self.device = dtype, device
        self.k_caches, self.v_caches, self.states = {}, {}, {}
        for li, (g, d, dv) in kv_layers.items():
            self.k_caches[li] = torch.zeros(n_pages, page_size, g, d, dtype=dtype, device=device)
            # value width 0: what a token keeps serves as key and value alike (a cached latent)
            self.v_caches[li] = torch.zeros(n_pages, page_size, g, dv, dtype=dtype, device=device) if dv else None
        for li, named in state_layers.items():
            self.states[li] = {name: torch.zeros((n_slots,) + tuple(shape), dtype=torch.float32, device=device)
                               for name, shape in named.items()}
        self._free_pages = collections.deque(range(n_pages))
        self._free_slots = collections.deque(range(n_slots))
        self._pages: Dict[object, List[int]] = {}
        self._slot: Dict[object, int] = {}
        self._len: Dict[object, int] = {}
        self._tail: Dict[object, int] = {}       # the last token of each sequence, as of the last advance()
        self._tail_next: Dict[object, int] = {}  # ... as it will be once the planned step has been advanced
        self.max_seq_pages = (max_tokens + page_size - 1) // page_size
        self.max_rows, self.max_step_tokens = max_rows, max_step_tokens
        self._on_gpu = torch.cuda.is_available() and str(device).startswith("cuda")
        words = 4 * max_step_tokens + max_rows * (6 + self.max_seq_pages) + \
            2 * (max_step_tokens // SCAN_CHUNK + max_rows)
        self._ring = 4 if self._on_gpu else 1
        # a ring of pinned staging buffers (the host may run ahead of the copies), ONE device buffer: the
        # copies and the kernels that read it are ordered on the stream, and a step of a given shape
        # finds its fields at the same addresses every time - what a captured step needs
        self._host = [torch.zeros(words, dtype=torch.int32, pin_memory=self._on_gpu) for _ in range(self._ring)]
        self._dev = torch.zeros(words, dtype=torch.int32, device=device)
        self._events = [None] * self._ring
        self._next = 0

    # ------------------------------------------------------------------ bookkeeping
    def length(self, seq_id) -> int:
        return self._len.get(seq_id, 0)

    def has(self, seq_id) -> bool:
        return seq_id in self._slot

    def admit(self, seq_id) -> int:
        """A state slot for a new sequence."""
        if seq_id in self._slot:
            return self._slot[seq_id]
        if not self._free_slots:
            raise PoolExhausted(seq_id, "state slot")
        self._slot[seq_id] = self._free_slots.popleft()
        self._pages[seq_id], self._len[seq_id] = [], 0
        return self._slot[seq_id]

    def pages_needed(self, seq_id, n_new: int) -> int:
        total = self._len.get(seq_id, 0) + n_new
        return max(0, (total + self.page_size - 1) // self.page_size - len(self._pages.get(seq_id, [])))

    def reserve(self, rows: Seq[Tuple[object, int]]):
        """Slots and pages for one step: rows = [(seq_id, new tokens)].  All or nothing."""
        for sid, n in rows:
            if self._len.get(sid, 0) + n > self.max_seq_pages * self.page_size:
                raise ValueError(f"sequence {sid} would pass the {self.max_seq_pages * self.page_size} positions "
                                 "a block-table row describes")
        new_slots = len({sid for sid, _ in rows if sid not in self._slot})
        if new_slots > len(self._free_slots):
            raise PoolExhausted(next(sid for sid, _ in rows if sid not in self._slot), "state slot")
        need = {sid: self.pages_needed(sid, n) for sid, n in rows}
        if sum(need.values()) > len(self._free_pages):
            raise PoolExhausted(next(sid for sid, k in need.items() if k), "page")
        for sid, n in rows:
            self.admit(sid)
            for _ in range(need[sid]):
                self._pages[sid].append(self._free_pages.popleft())

    def advance(self, rows: Seq[Tuple[object, int]]):
        for sid, n in rows:
            self._len[sid] += n
            if sid in self._tail_next:
                self._tail[sid] = self._tail_next.pop(sid)

    def free(self, seq_id):
        pages = self._pages.pop(seq_id, None)
        if pages:
            self._free_pages.extend(pages)
        slot = self._slot.pop(seq_id, None)
        if slot is not None:
            self._free_slots.append(slot)
        self._len.pop(seq_id, None)
        self._tail.pop(seq_id, None)
        self._tail_next.pop(seq_id, None)

    def reset(self):
        for sid in list(self._slot):
            self.free(sid)

    def get_blocks(self, seq_id):
        return self._pages.get(seq_id, [])

    def slot_of(self, seq_id):
        return self._slot.get(seq_id)

    @property
    def stats(self):
        return {"total": self.n_pages, "free": len(self._free_pages), "used": self.n_pages - len(self._free_pages),
                "slots_free": len(self._free_slots)}

    # ------------------------------------------------------------------ one step
    def plan(self, rows: Seq[Tuple[object, Seq[int]]]) -> RaggedStep:
        """rows = [(seq_id, its next token ids)], already reserved.  Positions continue each sequence."""
        B = len(rows)
        T = sum(len(t) for _, t in rows)
        if B > self.max_rows or T > self.max_step_tokens:
            raise ValueError(f"step of {B} rows / {T} tokens exceeds {self.max_rows} rows / {self.max_step_tokens} tokens")
        i = self._next
        self._next = (i + 1) % self._ring
        if self._events[i] is not None:
            self._events[i].synchronize()
        host = self._host[i].numpy()
        W = self.max_seq_pages
        o_ids, o_row, o_pos, o_prev = 0, T, 2 * T, 3 * T
        o_rows = 4 * T
        o_bt = o_rows + 4 * B
        start = 0
        max_slot = max_page = 0
        host[o_bt:o_bt + B * W] = -1
        for b, (sid, toks) in enumerate(rows):
            n, ctx, slot, pages = len(toks), self._len[sid], self._slot[sid], self._pages[sid]
            assert n > 0 and (ctx + n + self.page_size - 1) // self.page_size <= len(pages)
            host[o_ids + start:o_ids + start + n] = toks
            host[o_row + start:o_row + start + n] = b
            host[o_pos + start:o_pos + start + n] = range(ctx, ctx + n)
            host[o_prev + start] = self._tail[sid] if ctx else -1
            host[o_prev + start + 1:o_prev + start + n] = toks[:-1]
            self._tail_next[sid] = int(toks[-1])
            host[o_rows + b], host[o_rows + B + b] = start, n
            host[o_rows + 2 * B + b], host[o_rows + 3 * B + b] = ctx, slot
            host[o_bt + b * W:o_bt + b * W + len(pages)] = pages
            max_slot, max_page = max(max_slot, slot), max(max_page, max(pages))
            start += n
        # chunk table of the long rows
        o_c0 = o_bt + B * W
        o_nch = o_c0 + B
        chunks = []
        for b, (sid, toks) in enumerate(rows):
            n = len(toks)
            host[o_c0 + b] = len(chunks)
            if n > SCAN_SEQ_MAX:
                first = int(host[o_rows + b])
                for off in range(0, n, SCAN_CHUNK):
                    chunks.append((first + off, min(SCAN_CHUNK, n - off)))
            host[o_nch + b] = len(chunks) - int(host[o_c0 + b])
        NC = len(chunks)
        o_cs = o_nch + B
        o_cl = o_cs + NC
        if NC:
            host[o_cs:o_cs + NC] = [c[0] for c in chunks]
            host[o_cl:o_cl + NC] = [c[1] for c in chunks]
        used = o_cl + NC
        dev = self._dev
        dev[:used].copy_(self._host[i][:used], non_blocking=True)
        if self._on_gpu:
            ev = self._events[i] or torch.cuda.Event()
            ev.record()
            self._events[i] = ev
        return RaggedStep(
            tokens=T, rows=B, page=self.page_size, ids=dev[o_ids:o_ids + T], tok_row=dev[o_row:o_row + T],
            tok_pos=dev[o_pos:o_pos + T], tok_prev=dev[o_prev:o_prev + T], row_start=dev[o_rows:o_rows + B], row_len=dev[o_rows + B:o_rows + 2 * B],
            row_ctx=dev[o_rows + 2 * B:o_rows + 3 * B], row_slot=dev[o_rows + 3 * B:o_rows + 4 * B],
            block_table=dev[o_bt:o_bt + B * W].view(B, W), max_slot=max_slot, max_page=max_page, n_chunks=NC,
            ch_start=dev[o_cs:o_cs + NC], ch_len=dev[o_cl:o_cl + NC], row_ch0=dev[o_c0:o_c0 + B],
            row_nch=dev[o_nch:o_nch + B], slots=tuple(self._slot[sid] for sid, _ in rows),
            short_tokens=sum(len(t) for _, t in rows if len(t) <= SCAN_SEQ_MAX))
