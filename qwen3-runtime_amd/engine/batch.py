"""One step's batch: the entries given, flattened into the arrays the kernels read.

An entry is a request's next tokens: a portion of a prompt, or one decoded
token, it makes no difference. All entries of a step are packed into one batch
(reference: qwen3_runtime/engine/batch.py:45-60 builds the same arrays with
Python loops and lists; here they are numpy arrays packed into one host buffer
so that a step costs one upload).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, Sequence

import numpy as np


@dataclass
class StepEntry:
    """``tokens``: the request's next token ids. ``want``: indices into ``tokens``
    whose logits are asked for (may be empty)."""

    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class PackedStep:
    num_tokens: int
    num_seqs: int
    q_lens: list[int]
    kv_lens: list[int]
    # name -> int32 array; uploaded together, in this order
    arrays: dict[str, np.ndarray] = field(default_factory=dict)
    num_rows: int = 0


def pack_step(entries: Sequence[StepEntry], cache, vocab_size: int, table_width: int | None = None) -> PackedStep:
    """Flatten entries. ``cache`` must already hold the pages of every entry's tokens."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    seen = set()
    q_lens, starts = [], []
    for e in entries:
        if e.request_id in seen:
            raise ValueError(f"request {e.request_id!r} appears twice in one step")
        seen.add(e.request_id)
        n = len(e.tokens)
        if n < 1:
            raise ValueError(f"request {e.request_id!r} brings no tokens")
        for w in e.want:
            if not 0 <= int(w) < n:
                raise ValueError(f"request {e.request_id!r} wants row {w} of {n} tokens")
        q_lens.append(n)
        starts.append(cache.length(e.request_id))
    s = len(entries)
    t = int(sum(q_lens))
    cu_q = np.zeros(s + 1, dtype=np.int32)
    np.cumsum(q_lens, out=cu_q[1:])
    rows: list[int] = []
    row_seq: list[int] = []
    if t == s:  # one token each (decoding): no loops over tokens
        ids = np.asarray([e.tokens[0] for e in entries], dtype=np.int64).astype(np.int32)
        positions = np.asarray(starts, dtype=np.int32)
        seq_of_token = np.arange(s, dtype=np.int32)
        for i, e in enumerate(entries):
            if len(e.want):
                rows.append(i)
                row_seq.append(i)
    else:
        ids = np.empty(t, dtype=np.int32)
        positions = np.empty(t, dtype=np.int32)
        seq_of_token = np.empty(t, dtype=np.int32)
        for i, e in enumerate(entries):
            a, b = int(cu_q[i]), int(cu_q[i + 1])
            ids[a:b] = np.asarray(e.tokens, dtype=np.int64)
            positions[a:b] = np.arange(starts[i], starts[i] + q_lens[i], dtype=np.int32)
            seq_of_token[a:b] = i
            rows.extend(a + int(w) for w in e.want)
            row_seq.extend(i for _ in e.want)
    if ids.min() < 0 or ids.max() >= vocab_size:
        raise ValueError(f"token id outside [0, {vocab_size})")
    kv_lens = [st + n for st, n in zip(starts, q_lens)]
    rids = [e.request_id for e in entries]
    state_slots = np.asarray([cache.slots.slot(r) for r in rids], dtype=np.int32)
    arrays = {
        "ids": ids,
        "positions": positions,
        "seq_of_token": seq_of_token,
        "cu_q": cu_q,
        "kv_lens": np.asarray(kv_lens, dtype=np.int32),
        "state_slots": state_slots,
        "first_span": np.asarray([1 if st == 0 else 0 for st in starts], dtype=np.int32),
        "rows": np.asarray(rows, dtype=np.int32),
        # the state slot of each wanted row's request (the sampler reads its options there)
        "row_slots": state_slots[np.asarray(row_seq, dtype=np.int64)] if rows else np.zeros(0, dtype=np.int32),
    }
    width = table_width if table_width is not None else cache.table_width(rids)
    for gi in range(len(cache.groups)):
        table = np.empty((s, width), dtype=np.int32)
        cache.fill_tables(gi, rids, table)
        arrays[f"table{gi}"] = table
        arrays[f"slots{gi}"] = np.concatenate(
            [cache.token_slots(gi, e.request_id, starts[i], q_lens[i]) for i, e in enumerate(entries)]
        )
    return PackedStep(t, s, q_lens, kv_lens, arrays, num_rows=len(rows))
