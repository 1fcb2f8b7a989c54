"""From (request, its next tokens) to the flat tensors of one step.

The fields are those of the reference's `build_batch`
(worker/src/inference/qwen2/paged_attn.py:325-357): positions, slots, prefix sums; plus the
request of each token, slots for every cache group, state slots, and the rows whose logits
are wanted. Everything is packed into one int32 host buffer and reaches the device with one
copy. The block tables are not rebuilt: they live on the device (one row per state slot, kept
by the cache manager), and a step brings only the entries that changed since the step before,
so what the host does for a step does not grow with the length of its requests' contexts
(the reference rebuilds a padded table from Python lists every step and names that as a large
share of its step's host time: benchmarks/results/stage4-a100-vs-vllm.md:53).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..kernels.interface import BatchMeta, GroupMeta


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens, and the places among them whose
    logits are wanted (`want`; indexes into `tokens`)."""

    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)


class BatchBuilder:
    STAGING_BUFFERS = 3

    def __init__(self, cache: CacheManager, max_model_len: int, device, vocab_size: int, ops=None) -> None:
        self.cache = cache
        self.device = device
        self.ops = ops
        self.vocab_size = vocab_size
        self.max_model_len = int(max_model_len)
        self.table_width = max(1, -(-self.max_model_len // cache.block_size))
        cache.bind_tables(self.table_width)
        # pinned staging buffers for the step descriptions, used in turn: [host tensor, its numpy view, event of
        # the last copy out of it]. With them the copy to the device does not wait for the work queued before
        # it, so the host can prepare a step while the one before still runs.
        self._staging = [[None, None, None] for _ in range(self.STAGING_BUFFERS)]
        self._next_staging = 0

    def layout(self, T: int, B: int, R: int):
        """Offsets of the fields inside the packed int32 buffer of a step with T tokens, B requests
        and R wanted rows."""
        G = len(self.cache.groups)
        sizes = [T, T, T, B + 1, B, B, R] + [T] * G
        return np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)

    def flush_tables(self) -> None:
        """Bring the device's block tables up to the book-keeping: the entries that changed since the last
        call, as one small copy and one scattered write per group (nothing, if nothing changed)."""
        for g, group in enumerate(self.cache.groups):
            index, value = self.cache.take_changes(g)
            if not index:
                continue
            both = np.asarray([index, value], dtype=np.int32)
            if self.ops is not None:
                dev = self.ops.upload(both)
                self.ops.scatter_int32(group.table, dev[0], dev[1])
            else:
                dev = torch.from_numpy(both).to(group.table.device)
                group.table.view(-1)[dev[0].long()] = dev[1]

    def fill(self, host: np.ndarray, entries: Sequence[StepEntry], pad_requests: int = 0, want_all: bool = False,
             pad_tokens: int = 0, want_last: bool = False):
        """Write the step into `host` (int32, at least layout(...)[-1] long).
        -> (offsets, T, B, R, max_q, max_kv, host_cu_q, host_past)

        Pages for the new tokens must have been reserved. `pad_requests` appends that many
        requests that write to the sink page and the sink slot (for captured steps of
        fixed size): one token each, the first of them `pad_tokens` more (positions 0, 1, ...). `want_all`:
        every row is wanted, whatever the entries say. `want_last`: one row a request, its last (also of
        the padding requests), whatever the entries say."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        if pad_tokens and not pad_requests:
            raise ValueError("padding tokens need a padding request to belong to")
        cache = self.cache
        P = cache.block_size
        G = len(cache.groups)
        B = len(entries) + pad_requests
        T = sum(len(e.tokens) for e in entries) + pad_requests + pad_tokens
        R = T if want_all else (B if want_last else sum(len(e.want) for e in entries))
        if len({e.request_id for e in entries}) != len(entries):
            raise ValueError("a request may appear once in a step")
        offsets = self.layout(T, B, R)
        if host.shape[0] < offsets[-1]:
            raise ValueError("host buffer too small for this step")
        host[:offsets[-1]] = 0
        cut = lambda i: host[offsets[i]:offsets[i + 1]]
        ids, positions, token_request, cu_q, kv_len, slots_state, want_rows = (cut(i) for i in range(7))
        slots = [cut(7 + g) for g in range(G)]
        t0 = 0
        r0 = 0
        max_q = max_kv = 1
        host_past = np.zeros(B, dtype=np.int64)
        for b, entry in enumerate(entries):
            n = len(entry.tokens)
            if n < 1:
                raise ValueError(f"request {entry.request_id!r}: a step entry needs at least one token")
            state = cache.request(entry.request_id)
            past = state.num_cached
            if past + n > self.max_model_len:
                raise ValueError(f"request {entry.request_id!r}: {past + n} tokens exceed the limit of {self.max_model_len}")
            cu_q[b + 1] = t0 + n
            kv_len[b] = past + n
            slots_state[b] = state.slot
            host_past[b] = past
            if n == 1:
                # a decoded token: the same as below without an array per field (most rows of most steps)
                tok = int(entry.tokens[0])
                if tok < 0 or tok >= self.vocab_size:
                    raise ValueError(f"request {entry.request_id!r}: token id outside 0..{self.vocab_size - 1}")
                ids[t0] = tok
                positions[t0] = past
                token_request[t0] = b
                for g in range(G):
                    table = state.tables[g]
                    if len(table) * P <= past:
                        raise ValueError(f"request {entry.request_id!r}: pages were not reserved for this step")
                    page = table[past // P]
                    if page < 0:
                        raise AssertionError("a new token would be written to a page that was given back")
                    slots[g][t0] = page * P + past % P
            else:
                toks = np.asarray(entry.tokens, dtype=np.int64)
                if toks.min() < 0 or toks.max() >= self.vocab_size:
                    raise ValueError(f"request {entry.request_id!r}: token id outside 0..{self.vocab_size - 1}")
                ids[t0:t0 + n] = toks
                pos = np.arange(past, past + n, dtype=np.int64)
                positions[t0:t0 + n] = pos
                token_request[t0:t0 + n] = b
                first_page = past // P
                for g in range(G):
                    if len(state.tables[g]) * P < past + n:
                        raise ValueError(f"request {entry.request_id!r}: pages were not reserved for this step")
                    # the pages of the new positions only: the cost does not grow with what is cached already
                    table = np.asarray(state.tables[g][first_page:(past + n - 1) // P + 1], dtype=np.int64)
                    pages = table[pos // P - first_page]
                    if (pages < 0).any():
                        raise AssertionError("a new token would be written to a page that was given back")
                    slots[g][t0:t0 + n] = pages * P + pos % P
            if want_last:
                want_rows[b] = t0 + n - 1
            elif not want_all:
                for w in entry.want:
                    if not 0 <= int(w) < n:
                        raise ValueError(f"request {entry.request_id!r}: wanted place {w} is outside its {n} tokens")
                    want_rows[r0] = t0 + int(w)
                    r0 += 1
            t0 += n
            max_q = max(max_q, n)
            max_kv = max(max_kv, past + n)
        for b in range(len(entries), B):           # padding requests
            n = 1 + (pad_tokens if b == len(entries) else 0)
            pos = np.arange(n, dtype=np.int64)
            positions[t0:t0 + n] = pos
            token_request[t0:t0 + n] = b
            cu_q[b + 1] = t0 + n
            kv_len[b] = n
            slots_state[b] = cache.sink_slot
            for g, group in enumerate(cache.groups):
                slots[g][t0:t0 + n] = group.sink_page * P + pos % P
            if want_last:
                want_rows[b] = t0 + n - 1
            t0 += n
            max_q = max(max_q, n)
            max_kv = max(max_kv, n)
        if want_all:
            want_rows[:] = np.arange(T)
        return offsets, T, B, R, int(max_q), int(max_kv), cu_q.copy(), host_past

    def meta_of(self, dev: torch.Tensor, offsets, T: int, B: int, R: int, max_q: int, max_kv: int,
                host_cu_q=None, host_past=None, singles_bound=None):
        """Views into the device copy `dev` of a packed buffer -> (ids, BatchMeta, want_rows)."""
        dcut = lambda i: dev[int(offsets[i]):int(offsets[i + 1])]
        meta = BatchMeta(
            num_tokens=T, num_requests=B,
            positions=dcut(1), token_request=dcut(2), cu_q=dcut(3), kv_len=dcut(4), state_slots=dcut(5),
            max_q=max_q, max_kv=max_kv, block_size=self.cache.block_size,
            groups=[GroupMeta(block_table=group.table, slots=dcut(7 + g)) for g, group in enumerate(self.cache.groups)],
            host_cu_q=host_cu_q, host_past=host_past, all_decode=(max_q == 1), table_rows=dcut(5),
            singles_bound=singles_bound,
        )
        return dcut(0), meta, (dcut(6) if R else None)

    def build(self, entries: Sequence[StepEntry]):
        """-> (ids int32 [T], BatchMeta, want_rows int32 [R] or None), on the device, with one copy."""
        T = sum(len(e.tokens) for e in entries)
        R = sum(len(e.want) for e in entries)
        words = int(self.layout(T, len(entries), R)[-1])
        self.flush_tables()
        if torch.device(self.device).type != "cuda":
            host = np.empty(words, dtype=np.int32)
            offsets, T, B, R, max_q, max_kv, cu_q, past = self.fill(host, entries)
            dev = torch.from_numpy(host).to(self.device)
            return self.meta_of(dev, offsets, T, B, R, max_q, max_kv, cu_q, past)
        slot = self._staging[self._next_staging]
        self._next_staging = (self._next_staging + 1) % len(self._staging)
        if slot[2] is not None:
            slot[2].synchronize()                       # the copy made out of this buffer some steps ago is done
        if slot[0] is None or slot[0].numel() < words:
            slot[0] = torch.empty(max(words, 2 * (slot[0].numel() if slot[0] is not None else 0)), dtype=torch.int32,
                                  pin_memory=True)
            slot[1] = slot[0].numpy()
            slot[2] = torch.cuda.Event()
        offsets, T, B, R, max_q, max_kv, cu_q, past = self.fill(slot[1], entries)
        dev = torch.empty(words, dtype=torch.int32, device=self.device)
        dev.copy_(slot[0][:words], non_blocking=True)
        slot[2].record()
        return self.meta_of(dev, offsets, T, B, R, max_q, max_kv, cu_q, past)
