"""Minimal page-table builder for the paged entry points, so that `nsa_prefill` / `nsa_decode` can be driven without
an inference engine around them.

It follows the contract of upstream's nano-vllm engine:
  * raw K/V rows and compressed rows of a sequence live in pages of the same pool, listed in two tables
    (`Sequence.block_table` / `cmp_block_table`, nano-vllm/nanovllm/engine/sequence.py:75-88);
  * a sequence of L tokens owns cdiv(L, page) raw pages and cdiv(cmp_len(L), page) pages of compressed rows,
    cmp_len(L) = max((L - kernel_size) // stride + 1, 0); pages are taken when a length first needs them
    (nano-vllm/nanovllm/engine/block_manager.py:59, 87-92, 111-140) and compressed pages are never shared;
  * a step's tensors are the ones `ModelRunner.prepare_prefill / prepare_decode` build
    (nano-vllm/nanovllm/engine/model_runner.py:185-277): context_lens, block tables padded with -1, the flat pool row
    of every new token (slot_mapping) and of every compressed row the step completes (cmp_slot_mapping);
  * K and V pools of a layer are the two halves of one allocation (model_runner.py:157-171).
Prefix sharing by content hash (block_manager.py:36-84) is an engine policy and is not part of this builder.

Everything here is host-side bookkeeping; the only device work is the upload of the step's int32 tensors."""
from collections import deque

import torch


def cdiv(a, b):
    return (a + b - 1) // b


V_STAGGER_BYTES = 256  # start of a V pool relative to the start of its K pool, modulo 1 KB


def allocate_kv_pools(num_pages, page_size, num_kv_heads, qk_head_dim, v_head_dim=None, num_layers=1,
                      device="cuda", dtype=torch.bfloat16):
    """One allocation holding, per layer, the K pool [pages, page, KH, D] followed by the V pool [pages, page, KH, VD]
    (upstream nano-vllm/nanovllm/engine/model_runner.py:157-171), with the V pool staggered against the K pool (see
    below).  Returns a list of (k_cache, v_cache) views."""
    v_head_dim = qk_head_dim if v_head_dim is None else v_head_dim
    rows = num_pages * page_size * num_kv_heads
    esize = torch.empty(0, dtype=dtype).element_size()
    k_elems, v_elems = rows * qk_head_dim, rows * v_head_dim
    # Stagger: the V pool starts V_STAGGER_BYTES (mod 1 KB) after where the K pool starts.  A decode workgroup streams
    # the K rows and the V rows of ONE kv head; when the two pools start at the same offset inside a 1 KB window
    # (as they do when one pool simply follows the other), both streams of every workgroup fall on the same quarter
    # of the memory channels and the step is 8 % slower (measured on MI355X: 74.3 against 68.5 us for 64 requests).
    layer_elems = k_elems + v_elems + 2 * 1024 // esize
    storage = torch.empty(num_layers * layer_elems + 1024 // esize, device=device, dtype=dtype)
    pools = []
    for layer in range(num_layers):
        k_off = layer * layer_elems
        k_off += ((-(storage.data_ptr() + k_off * esize)) % 1024) // esize          # K pool: 1 KB aligned
        v_off = k_off + k_elems
        v_addr = storage.data_ptr() + v_off * esize
        v_off += ((V_STAGGER_BYTES - v_addr) % 1024) // esize
        k = storage[k_off:k_off + k_elems].view(num_pages, page_size, num_kv_heads, qk_head_dim)
        v = storage[v_off:v_off + v_elems].view(num_pages, page_size, num_kv_heads, v_head_dim)
        pools.append((k, v))
    return pools


class _Seq:
    __slots__ = ("length", "pages", "cmp_pages", "pooled")

    def __init__(self):
        self.length = 0      # tokens whose K/V are (or are being) written to the pool
        self.pages = []      # raw pages
        self.cmp_pages = []  # pages of compressed rows
        self.pooled = 0      # compressed rows already written


class PageTableBuilder:
    """Hands out pages to sequences and builds the index tensors of prefill and decode steps."""

    def __init__(self, num_pages, page_size=256, kernel_size=32, stride=16):
        assert page_size % 64 == 0, "the kernels need a page size that is a multiple of 64"
        assert kernel_size % stride == 0
        self.num_pages, self.page_size = num_pages, page_size
        self.kernel_size, self.stride = kernel_size, stride
        self.free = deque(range(num_pages))
        self.seqs = {}

    # ------------------------------------------------------------------ bookkeeping
    def cmp_len(self, length):
        return max((length - self.kernel_size) // self.stride + 1, 0)

    def pages_needed(self, seq_id, new_tokens):
        """Pages that extending seq_id (or a not yet known sequence) by new_tokens would take."""
        s = self.seqs.get(seq_id)
        have_raw, have_cmp, length = (len(s.pages), len(s.cmp_pages), s.length) if s else (0, 0, 0)
        length += new_tokens
        return (cdiv(length, self.page_size) - have_raw) + (cdiv(self.cmp_len(length), self.page_size) - have_cmp)

    def can_extend(self, seq_id, new_tokens):
        return len(self.free) >= self.pages_needed(seq_id, new_tokens)

    def _take(self):
        if not self.free:
            raise RuntimeError("KV pool exhausted")
        return self.free.popleft()

    def _extend(self, seq_id, new_tokens):
        if not self.can_extend(seq_id, new_tokens):
            raise RuntimeError(f"KV pool exhausted: sequence {seq_id} needs {self.pages_needed(seq_id, new_tokens)} "
                               f"more pages, {len(self.free)} free")
        s = self.seqs.setdefault(seq_id, _Seq())
        s.length += new_tokens
        while len(s.pages) < cdiv(s.length, self.page_size):
            s.pages.append(self._take())
        while len(s.cmp_pages) < cdiv(self.cmp_len(s.length), self.page_size):
            s.cmp_pages.append(self._take())
        return s

    def release(self, seq_id):
        s = self.seqs.pop(seq_id)
        self.free.extend(reversed(s.cmp_pages))
        self.free.extend(reversed(s.pages))

    def length(self, seq_id):
        return self.seqs[seq_id].length

    def slot(self, seq_id, position):
        """Flat pool row of token `position` of the sequence."""
        s = self.seqs[seq_id]
        return s.pages[position // self.page_size] * self.page_size + position % self.page_size

    def cmp_slot(self, seq_id, row):
        """Flat pool row of compressed row `row` of the sequence."""
        s = self.seqs[seq_id]
        return s.cmp_pages[row // self.page_size] * self.page_size + row % self.page_size

    # ------------------------------------------------------------------ step tensors
    @staticmethod
    def _table(rows, width, device):
        t = torch.full((len(rows), max(width, 1)), -1, dtype=torch.int32)
        for i, r in enumerate(rows):
            if r:
                t[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
        return t.to(device)

    def _tables(self, ids, device, raw_width=None, cmp_width=None):
        raw = [self.seqs[i].pages for i in ids]
        cmp_ = [self.seqs[i].cmp_pages for i in ids]
        rw = max(len(r) for r in raw) if raw_width is None else raw_width
        cw = max(len(r) for r in cmp_) if cmp_width is None else cmp_width
        return self._table(raw, rw, device), self._table(cmp_, cw, device)

    def prefill(self, seq_ids, new_lens, device="cuda"):
        """Extends every sequence by its number of new tokens (a whole prompt, or the next chunk of one) and returns
        the tensors of that prefill step as keyword arguments for `nsa_prefill` (all but q, k, v, w and the new
        rows): x_cu_seqlens, y_cu_seqlens, x_maxlen, y_maxlen, context_lens, block_tables, cmp_slot_mapping,
        cmp_block_tables, and slot_mapping (rows of the new tokens, for the cache writer)."""
        x_cu, y_cu, ctx, slots, cmp_slots = [0], [0], [], [], []
        for sid, n in zip(seq_ids, new_lens):
            assert n > 0
            s = self._extend(sid, n)
            start = s.length - n
            x_cu.append(x_cu[-1] + n)
            ctx.append(s.length)
            slots.extend(self.slot(sid, p) for p in range(start, s.length))
            y = self.cmp_len(s.length)
            y_cu.append(y_cu[-1] + y)
            # every compressed row of the sequence is listed; the ones pooled by earlier chunks are marked done
            cmp_slots.extend(-1 if r < s.pooled else self.cmp_slot(sid, r) for r in range(y))
            s.pooled = y
        bt, cbt = self._tables(seq_ids, device)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32).to(device)
        ys = [y_cu[i + 1] - y_cu[i] for i in range(len(seq_ids))]
        return dict(x_cu_seqlens=i32(x_cu), y_cu_seqlens=i32(y_cu), x_maxlen=max(new_lens), y_maxlen=max(ys),
                    context_lens=i32(ctx), block_tables=bt, cmp_slot_mapping=i32(cmp_slots), cmp_block_tables=cbt,
                    slot_mapping=i32(slots))

    def decode(self, seq_ids, device="cuda", pad_to=None, raw_width=None, cmp_width=None):
        """Extends every sequence by one token and returns the tensors of that decode step for `nsa_decode`:
        context_lens, block_tables, cmp_slot_mapping, cmp_block_tables, and slot_mapping (row of the new token).
        pad_to: batch size of a captured graph; the padding rows get context 0 and slot -1, as the graph-variable
        update of upstream's runner fills them (nano-vllm/nanovllm/engine/model_runner.py:287-309);
        raw_width / cmp_width: fixed table widths for such a graph."""
        ctx, slots, cmp_slots = [], [], []
        for sid in seq_ids:
            s = self._extend(sid, 1)
            ctx.append(s.length)
            slots.append(self.slot(sid, s.length - 1))
            y = self.cmp_len(s.length)
            if y > s.pooled:  # the new token completes compressed row y-1
                cmp_slots.append(self.cmp_slot(sid, y - 1))
                s.pooled = y
            else:
                cmp_slots.append(-1)
        bt, cbt = self._tables(seq_ids, device, raw_width, cmp_width)
        pad = 0 if pad_to is None else pad_to - len(seq_ids)
        assert pad >= 0
        if pad:
            fill = lambda t: torch.cat([t, torch.full((pad, t.size(1)), -1, dtype=torch.int32, device=t.device)])
            bt, cbt = fill(bt), fill(cbt)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32).to(device)
        return dict(context_lens=i32(ctx + [0] * pad), block_tables=bt, cmp_slot_mapping=i32(cmp_slots + [-1] * pad),
                    cmp_block_tables=cbt, slot_mapping=i32(slots + [-1] * pad))
