"""Per-step attention metadata for a mixed (decode + chunked-prefill) batch.

Token layout of a step: all decode tokens first (one per decoding sequence),
then the prefill chunks back to back. The decode part can be replayed from a
captured hipGraph (static buffers, fixed split plan); the prefill part is
always eager.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class SeqMeta:
    """Per-sequence description of a step for models whose layers keep per-sequence state or use
    the per-row attention kernels (ops/seqmix.py): the step's tokens are the sequences' runs back
    to back, decodes (one token each) first, then the prefill portions."""
    num_seqs: int
    seq_start: torch.Tensor          # [n + 1] int32: token bounds of each sequence's run
    seq_slot: torch.Tensor           # [n] int32: state slot (engine/state_cache.py)
    seq_init: torch.Tensor           # [n] int32: 1 = the slot holds this sequence's earlier state
    row_seq: torch.Tensor            # [T] int32: token -> sequence (row of ``tables``)
    row_len: torch.Tensor            # [T] int32: keys the token sees (= position + 1)
    tables: torch.Tensor             # [n, W] int32 block tables
    max_len: int = 0                 # longest context of the step
    max_q: int = 0                   # longest run of the step
    q_lens: Optional[list] = None    # host copy of the run lengths
    ctx_lens: Optional[list] = None  # host copy of each sequence's context length after the step
    _items: Optional[dict] = None    # (tokens per item, balance) -> [n, 3] int32 work items (attention_items)
    _chunks: Optional[dict] = None   # chunk length -> (table, number of chunks) (scan_chunks)

    def attention_items(self, tokens_per_item: int, balance: int = 0) -> torch.Tensor:
        """Work items (sequence, first token row, tokens) of the matrix-core attention kernel: every
        run cut into pieces of at most ``tokens_per_item`` tokens. Built once per step and size.

        ``balance`` > 0 (needs ``ctx_lens``): a causal item's work grows with its position in the
        prompt, and the workgroups of a step are all resident at once, dealt to the CUs in order. The
        items are sorted by their number of keys and laid out as a snake over blocks of ``balance``
        items (descending, ascending, descending, ...), so that the workgroups that land on one CU -
        one of every block - sum to about the same number of key tiles."""
        if self._items is None:
            self._items = {}
        key = (tokens_per_item, balance if self.ctx_lens is not None else 0)
        it = self._items.get(key)
        if it is None:
            rows, keys, t0 = [], [], 0
            for s, n in enumerate(self.q_lens):
                for a in range(0, n, tokens_per_item):
                    c = min(tokens_per_item, n - a)
                    rows.append((s, t0 + a, c))
                    if key[1]:
                        keys.append(self.ctx_lens[s] - n + a + c)
                t0 += n
            if key[1] and len(rows) > 1:
                order = sorted(range(len(rows)), key=lambda i: -keys[i])
                snake = []
                for b in range(0, len(order), balance):
                    blk = order[b:b + balance]
                    snake.extend(blk if (b // balance) % 2 == 0 else blk[::-1])
                rows = [rows[i] for i in snake]
            it = torch.tensor(rows, dtype=torch.int32).view(-1, 3)
            if self.tables.is_cuda:
                it = it.pin_memory().to(self.tables.device, non_blocking=True)
            self._items[key] = it
        return it


    def _scan_chunks(self, length: int):
        bounds, first = [0], [0]
        for n in self.q_lens:
            t0 = bounds[-1]
            for a in range(0, n, length):
                bounds.append(t0 + min(n, a + length))
            first.append(len(bounds) - 1)
        nc = len(bounds) - 1
        table = torch.tensor(bounds + list(range(nc)) + [0] * nc + [1] * nc + first, dtype=torch.int32)
        if self.tables.is_cuda:
            table = table.pin_memory().to(self.tables.device, non_blocking=True)
        return table, nc

    def scan_chunks(self, length: int):
        """Every run cut into chunks of at most ``length`` tokens, for recurrences that are linear in their
        state and scan the chunks of a prompt side by side. Returns (table, nc): int32 [chunk bounds
        (nc + 1) | 0 .. nc - 1 | nc zeros | nc ones | first chunk of each sequence (n + 1)] - the bounds,
        scratch slots and "start from zero" / "continue" flags of the chunks as runs of their own, and each
        sequence's range of chunks. Built once per step and length."""
        if self._chunks is None:
            self._chunks = {}
        if length not in self._chunks:
            self._chunks[length] = self._scan_chunks(length)
        return self._chunks[length]


@dataclass
class AttnMeta:
    num_tokens: int
    positions: torch.Tensor          # [T] int64
    slot_mapping: torch.Tensor       # [T] int64 (-1 = do not write)
    # decode part
    num_decode: int = 0
    d_block_tables: Optional[torch.Tensor] = None  # [Bd, W] int32
    d_seq_lens: Optional[torch.Tensor] = None      # [Bd] int32
    d_split: Optional[tuple] = None                # (split_size, nsplit)
    d_workspace: Optional[tuple] = None            # (part_o, part_ml)
    d_max_ctx: int = 0
    d_cascade: Optional[tuple] = None              # shared-prefix decode (ops.cascade_tensors)
    d_split_dev: Optional[torch.Tensor] = None     # [1] int32 keys per split, set per graph replay
    # prefill part
    num_prefill_tokens: int = 0
    p_block_tables: Optional[torch.Tensor] = None  # [Bp, W] int32
    p_q_start: Optional[torch.Tensor] = None       # [Bp] int32 (relative to the prefill part)
    p_q_len: Optional[torch.Tensor] = None
    p_ctx_len: Optional[torch.Tensor] = None
    p_items: Optional[torch.Tensor] = None         # [n, 2] int32
    p_items_per_window: Optional[dict] = None
    # MLA (one attention row per decode sequence / prefill token)
    mla_d_rows: Optional[torch.Tensor] = None      # [Bd] int32 = arange (row -> d_block_tables row)
    mla_split: Optional[tuple] = None              # fixed (split_size, nsplit) under graph capture
    mla_workspace: Optional[tuple] = None
    mla_split_dev: Optional[torch.Tensor] = None   # [1] int32 keys per split, set per graph replay
    p_row_seq: Optional[torch.Tensor] = None       # [Tp] int32 prefill token -> p_block_tables row
    p_row_len: Optional[torch.Tensor] = None       # [Tp] int32 keys visible (= position + 1)
    p_max_ctx: int = 0
    # multimodal: step rows that are image placeholders and their embeddings
    mm_rows: Optional[torch.Tensor] = None         # [n] int64
    mm_embeds: Optional[torch.Tensor] = None       # [n, d_model]
    # hybrid KV cache (engine/hybrid_kv.py): the windowed layers' own slot mapping and
    # block tables (everything else shared), or None
    swa: Optional["AttnMeta"] = None
    # per-sequence runs, state slots and per-row attention lengths (stateful / per-layer stacks)
    seq: Optional[SeqMeta] = None

    @property
    def has_prefill(self) -> bool:
        return self.num_prefill_tokens > 0
