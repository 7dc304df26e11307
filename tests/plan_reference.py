"""A plain planner of a step's index arrays, in NumPy: which sequences run, where each stands,
which tokens it brings, which rows' logits are wanted, the prefill's tiles, the decode attention's
work list, every token's cache page.  The engine in the library plans every step itself
(csrc/engine.hip); the tests hold its arrays to these, and call single kernels with them.

The sequences of a step either all bring their first tokens (a prefill step; lengths may
differ) or each bring one more token (a decode step).  picolm has the two as separate
single-sequence functions (`model_forward_prefill`, `model_forward`, picolm/model.h:538-539);
here they are one step over a batch, and tokens are packed without padding.
"""
from __future__ import annotations

import numpy as np
import torch

from picolm_amd.cache import PAGE_TOKENS, pages_for
from picolm_amd.engine.errors import StepError


def _to_device(host: torch.Tensor, device) -> torch.Tensor:
    """A copy of a small host array on the device that does not make the host wait for the GPU (a
    plain copy from pageable memory waits for everything the stream still has to do, and a prefill
    step asks for such arrays after its first kernels are on their way): through pinned memory,
    which torch keeps until the transfer has run."""
    if torch.device(device).type != "cuda":
        return host.to(device)
    return host.pin_memory().to(device, non_blocking=True)


class StepBatch:
    def __init__(self, slots, pos0, new_tokens, want, vocab_size: int, device):
        """slots[i]: cache slot of sequence i; pos0[i]: tokens it holds; new_tokens[i]: its
        next tokens; want[i]: indices into new_tokens[i] whose logits are asked for."""
        self.n_seq = len(slots)
        if self.n_seq == 0:
            raise StepError("a step needs at least one sequence")
        if not (len(pos0) == len(new_tokens) == len(want) == self.n_seq):
            raise StepError("slots, positions, tokens and wanted rows differ in length")
        if len(set(slots)) != self.n_seq:
            raise StepError("a slot appears twice in one step")
        n_new = [len(t) for t in new_tokens]
        if min(n_new) < 1:
            raise StepError("every sequence of a step brings at least one token")
        self.slots = list(slots)
        self.pos0 = [int(p) for p in pos0]
        self.n_new = n_new
        self.max_new = max(n_new)
        self.T = sum(n_new)
        self.is_decode = self.max_new == 1
        self.max_len = max(p + n for p, n in zip(self.pos0, n_new))

        cu = np.zeros(self.n_seq + 1, dtype=np.int32)
        cu[1:] = np.cumsum(n_new)
        tokens = np.concatenate([np.asarray(t, dtype=np.int64) for t in new_tokens])
        if tokens.min() < 0 or tokens.max() >= vocab_size:
            bad = int(tokens[(tokens < 0) | (tokens >= vocab_size)][0])
            raise StepError(f"token id {bad} is outside the vocabulary of {vocab_size}")
        tok_pos = np.concatenate([np.arange(p, p + n, dtype=np.int32) for p, n in zip(self.pos0, n_new)])
        tok_seq = np.repeat(np.arange(self.n_seq, dtype=np.int32), n_new)
        rows = []
        for i, w in enumerate(want):
            for j in w:
                if not 0 <= j < n_new[i]:
                    raise StepError(f"wanted row {j} of a sequence that brings {n_new[i]} tokens")
                rows.append(int(cu[i]) + int(j))
        self.n_want = len(rows)
        self.want_counts = [len(w) for w in want]
        self.wants_every_row = rows == list(range(self.T))

        parts = {
            "seq_slot": np.asarray(self.slots, dtype=np.int32),
            "seq_pos0": np.asarray(self.pos0, dtype=np.int32),
            "seq_nnew": np.asarray(n_new, dtype=np.int32),
            "cu_seqlens": cu,
            "tok_pos": tok_pos,
            "tok_seq": tok_seq,
            "tokens": tokens.astype(np.int32),
            "want_rows": np.asarray(rows, dtype=np.int32),
        }
        self._host = parts
        self._device = torch.device(device)
        self._upload(parts)
        self._tiles = {}
        self._chunks = {}
        self._write_pages = {}

    def _upload(self, parts) -> None:
        sizes = [max(len(v), 1) for v in parts.values()]
        flat = np.zeros(sum(sizes), dtype=np.int32)
        off = 0
        spans = {}
        for (k, v), n in zip(parts.items(), sizes):
            flat[off:off + len(v)] = v
            spans[k] = (off, n)
            off += n
        dev = _to_device(torch.from_numpy(flat), self._device)
        for k, (o, n) in spans.items():
            setattr(self, k, dev[o:o + n])

    # -- derived launch geometry ----------------------------------------------------------
    def prefill_tiles(self, rows_per_tile: int):
        """(tile_seq, tile_q0, n_tiles) on the device: tiles of `rows_per_tile` new tokens."""
        if rows_per_tile not in self._tiles:
            tiles = []
            for i, n in enumerate(self.n_new):
                for q0 in range(0, n, rows_per_tile):
                    tiles.append((self.pos0[i] + min(q0 + rows_per_tile, n), i, q0))
            tiles.sort()          # by the keys a tile sees: the kernels hand out the longest first
            seqs = [t[1] for t in tiles]
            q0s = [t[2] for t in tiles]
            flat = _to_device(torch.tensor(seqs + q0s, dtype=torch.int32), self._device)
            self._tiles[rows_per_tile] = (flat[:len(seqs)], flat[len(seqs):], len(seqs))
        return self._tiles[rows_per_tile]

    def chunks(self, chunk_tokens: int):
        """The step cut along positions: chunk c holds, of every sequence, its new tokens
        c*chunk_tokens .. (c+1)*chunk_tokens - 1.  Each chunk looks like a step of its own to
        the attention kernels (`rows` lists its token rows)."""
        n_chunks = (self.max_new + chunk_tokens - 1) // chunk_tokens
        cu = self._host["cu_seqlens"]
        for c in range(n_chunks):
            lo = c * chunk_tokens
            seqs = [i for i, n in enumerate(self.n_new) if n > lo]
            yield _Chunk(self, seqs, lo, [min(chunk_tokens, self.n_new[i] - lo) for i in seqs],
                         [int(cu[i]) + lo for i in seqs])

    def write_pages(self, group: int, table_host, ring_pages: int):
        """For every token of the step the physical page of cache group `group` that takes its
        key and value (device int32 [T])."""
        if group not in self._write_pages:
            pages = token_pages(self._host["tok_seq"], self._host["tok_pos"], self.slots, table_host, ring_pages)
            self._write_pages[group] = _to_device(torch.from_numpy(pages), self._device)
        return self._write_pages[group]

    def decode_chunks(self, blocks_per_chunk: int, max_pages_per_chunk: int, window: int, group: int, table_host,
                      ring_pages: int):
        """The decode attention's work list for this step over one cache group's pages:
        (header and entries on the device, number of entries, pages_per_chunk, most chunks of a
        sequence)."""
        key = (blocks_per_chunk, max_pages_per_chunk, window, group)
        if key not in self._chunks:
            ppc = decode_pages_per_chunk(self.pos0, blocks_per_chunk, max_pages_per_chunk)
            entries, most = decode_chunk_list(self.slots, self.pos0, window, ppc, table_host, ring_pages)
            self._chunks[key] = (_to_device(torch.from_numpy(with_header(entries, len(entries))), self._device), len(entries),
                                 ppc, most)
        return self._chunks[key]


def token_pages(tok_seq, tok_pos, slots, table_host, ring_pages: int):
    table = table_host.numpy() if hasattr(table_host, "numpy") else np.asarray(table_host)
    slot = np.asarray(slots, dtype=np.int64)[np.asarray(tok_seq, dtype=np.int64)]
    return table[slot, (np.asarray(tok_pos, dtype=np.int64) // PAGE_TOKENS) % ring_pages].astype(np.int32)


def decode_pages_per_chunk(pos0, blocks_per_chunk: int, max_pages_per_chunk: int = 16, min_blocks: int = 160) -> int:
    """Pages that one workgroup of the decode attention takes: the largest of 4, 8, 16, 32, 64
    within `max_pages_per_chunk` (what the kernel that will run was measured with) that still
    leaves `min_blocks` workgroups for the launch, which is most of the CUs; 4 (a page for each of
    four waves) if none does.  Fewer, larger chunks mean fewer partial results to merge and longer
    streams a wave."""
    pages = [int(p) // PAGE_TOKENS + 1 for p in pos0]
    for ppc in (64, 32, 16, 8):
        if ppc <= max_pages_per_chunk and sum((n + ppc - 1) // ppc for n in pages) * max(1, blocks_per_chunk) >= min_blocks:
            return ppc
    return 4


def with_header(entries, n_live: int):
    """The work list as the kernels read it: a header entry whose first int is the number of
    entries in use, then the entries."""
    out = np.zeros((len(entries) + 1, CHUNK_ENTRY_INTS), dtype=np.int32)
    out[0, 0] = n_live
    out[1:] = entries
    return out


CHUNK_ENTRY_INTS = 8


def decode_chunk_list(slots, pos0, window: int, pages_per_chunk: int, table_host, ring_pages: int):
    """(entries [n][8] int32, most chunks of one sequence): every sequence's visible pages
    (those of its last `window` keys, or all) cut into runs of `pages_per_chunk`.  An entry is
    {sequence, which chunk, position of the new token, slot, physical pages of the chunk's first
    four pages or -1}; the kernels derive each chunk's pages from the same arithmetic.  The
    entries come in no particular order of sequences: every entry says whose it is."""
    pos = np.asarray(pos0, dtype=np.int64)
    slot = np.asarray(slots, dtype=np.int64)
    first = (np.maximum(0, pos - window + 1) if window > 0 else np.zeros_like(pos)) // PAGE_TOKENS
    end = pos // PAGE_TOKENS + 1
    n = (end - first + pages_per_chunk - 1) // pages_per_chunk
    seq = np.repeat(np.arange(len(pos), dtype=np.int64), n)
    idx = np.arange(int(n.sum())) - np.repeat(np.cumsum(n) - n, n)
    # the chunks with the most pages first: workgroups are handed out in the list's order, and
    # the short last chunks of the sequences then fill the gaps at the end
    n_pages = np.minimum(end[seq] - first[seq] - idx * pages_per_chunk, pages_per_chunk)
    order = np.argsort(-n_pages, kind="stable")
    seq, idx = seq[order], idx[order]
    entries = np.empty((len(seq), CHUNK_ENTRY_INTS), dtype=np.int32)
    entries[:, 0] = seq
    entries[:, 1] = idx
    entries[:, 2] = pos[seq]
    entries[:, 3] = slot[seq]
    table = table_host.numpy() if hasattr(table_host, "numpy") else np.asarray(table_host)
    page0 = first[seq] + idx * pages_per_chunk
    for w in range(4):
        page = page0 + w
        inside = (page < end[seq]) & (w < pages_per_chunk)
        phys = table[slot[seq], np.where(inside, page, 0) % ring_pages]
        entries[:, 4 + w] = np.where(inside, phys, -1)
    return entries, int(n.max())


class _Chunk:
    """A slice of a step along positions, with the fields the attention kernels read."""

    def __init__(self, parent: StepBatch, seqs, lo, n_new, first_rows):
        self.n_seq = len(seqs)
        self.n_new = n_new
        self.pos0 = [parent.pos0[i] + lo for i in seqs]
        self.max_new = max(n_new)
        self.is_decode = False
        rows = np.concatenate([np.arange(r, r + n, dtype=np.int32) for r, n in zip(first_rows, n_new)])
        self.n_rows = len(rows)
        self._device = parent._device
        self._tiles = {}
        StepBatch._upload(self, {
            "seq_slot": np.asarray([parent.slots[i] for i in seqs], dtype=np.int32),
            "seq_pos0": np.asarray(self.pos0, dtype=np.int32),
            "seq_nnew": np.asarray(n_new, dtype=np.int32),
            "cu_seqlens": np.asarray(first_rows, dtype=np.int32),
            "rows": rows,
        })

    prefill_tiles = StepBatch.prefill_tiles
