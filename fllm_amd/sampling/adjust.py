"""What a request asks to be done to its logits before a token is chosen: penalties on tokens seen before, biases,
and end and stop ids that `min_tokens` still blocks (rust/engine/src/sampling.rs:220-229, :252-274).  The host keeps
the counts and packs them for the kernel; the newest token of a request may still be on the device only."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .params import SamplingParams

ROW_WORDS = 10      # int32 words of a row record: three floats, then seen_off, seen_len, bias_off, bias_len, blocked_off, blocked_len, last_row


class SeenTokens:
    """How often each token occurs among the first `upto` tokens of a request (all of them count; a window is cut out
    of the token list itself).  Kept as arrays that grow by a token a step, so that packing a step's rows copies them
    instead of walking a dictionary."""

    def __init__(self):
        self.ids = np.zeros(64, dtype=np.int32)
        self.counts = np.zeros(64, dtype=np.int32)
        self.size = 0
        self.at: Dict[int, int] = {}
        self.upto = 0

    def catch_up(self, tokens: Sequence[int], known: int) -> None:
        if self.size == 0 and known - self.upto > 32:          # a whole prompt at once
            ids, counts = np.unique(np.asarray(tokens[self.upto:known], dtype=np.int64), return_counts=True)
            ids = np.where((ids >= -(1 << 31)) & (ids < (1 << 31)), ids, -1)
            room = max(64, 1 << int(len(ids)).bit_length())
            self.ids, self.counts = np.zeros(room, dtype=np.int32), np.zeros(room, dtype=np.int32)
            self.ids[:len(ids)], self.counts[:len(ids)] = ids, counts
            self.size = len(ids)
            self.at = {t: i for i, t in enumerate(ids.tolist())}
            self.upto = known
            return
        for t in tokens[self.upto:known]:
            i = self.at.get(t)
            if i is None:
                if self.size == len(self.ids):
                    self.ids = np.concatenate([self.ids, np.zeros_like(self.ids)])
                    self.counts = np.concatenate([self.counts, np.zeros_like(self.counts)])
                i = self.at[t] = self.size
                self.ids[i] = t if -(1 << 31) <= t < (1 << 31) else -1
                self.size += 1
            self.counts[i] += 1
        self.upto = max(self.upto, known)

    def lists(self) -> Tuple[np.ndarray, np.ndarray]:
        return self.ids[:self.size], self.counts[:self.size]


@dataclass
class AdjustRow:
    """One row's share: the distinct tokens seen (within the window) with their counts (a dictionary, or the two
    arrays of `SeenTokens.lists`), ids blocked for now, and where the newest token lies on the device when the host
    does not know it yet."""
    params: SamplingParams
    seen: object
    blocked: Tuple[int, ...] = ()
    last_row: int = -1

    def seen_lists(self) -> Tuple[np.ndarray, np.ndarray]:
        if isinstance(self.seen, dict):
            ids = np.fromiter((t if -(1 << 31) <= t < (1 << 31) else -1 for t in self.seen), dtype=np.int32, count=len(self.seen))
            return ids, np.fromiter(self.seen.values(), dtype=np.int32, count=len(self.seen))
        return self.seen


def row_for(params: SamplingParams, tokens: Sequence[int], prompt_len: int, pending_row: Optional[int], eos: Sequence[int],
            seen: Optional[SeenTokens] = None) -> Optional[AdjustRow]:
    """The adjustment of the next token of a request whose tokens so far are `tokens`; the last of them is a
    placeholder when `pending_row` is given (its value is row `pending_row` of the tokens of the step in flight).
    None when the request asks for nothing.  `seen`: counts kept from step to step (no window)."""
    generated = len(tokens) - prompt_len
    if not params.adjusts_logits(generated):
        return None
    known = len(tokens) - (1 if pending_row is not None else 0)
    counts: object = {}
    last_row = -1
    if params.penalizes:
        n = params.repeat_last_n
        if n < 0 and seen is not None:
            seen.catch_up(tokens, known)
            counts = seen.lists()
        else:
            first = 0 if n < 0 else max(0, len(tokens) - n)
            counts = {}
            for t in tokens[first:known]:
                counts[t] = counts.get(t, 0) + 1
        if pending_row is not None and n != 0:
            last_row = pending_row
    blocked: Tuple[int, ...] = ()
    if generated < params.min_tokens:
        blocked = tuple(dict.fromkeys(list(eos) + list(params.stop_token_ids)))
    return AdjustRow(params, counts, blocked, last_row)


def pack(rows: Sequence[Optional[AdjustRow]]) -> Tuple[torch.Tensor, Tuple[int, int, int]]:
    """The kernel's input for a step's rows (None: a row left alone) as one int32 CPU tensor, and the lengths of its
    three list sections (seen, bias, blocked)."""
    records = np.zeros((len(rows), ROW_WORDS), dtype=np.int32)
    floats = records.view(np.float32)
    seen_ids, seen_counts, bias_ids, bias_values, blocked = [], [], [], [], []
    n_seen = n_bias = n_blocked = 0
    for i, r in enumerate(rows):
        if r is None:
            floats[i, 0] = 1.0
            records[i, 9] = -1
            continue
        p = r.params
        ids, counts = r.seen_lists()
        floats[i, 0:3] = (p.repetition_penalty, p.presence_penalty, p.frequency_penalty)
        records[i, 3:] = (n_seen, len(ids), n_bias, len(p.logit_bias), n_blocked, len(r.blocked), r.last_row)
        seen_ids.append(ids)
        seen_counts.append(counts)
        bias_ids.extend(t if t < (1 << 31) else -1 for t, _ in p.logit_bias)
        bias_values.extend(b for _, b in p.logit_bias)
        blocked.extend(t if -(1 << 31) <= t < (1 << 31) else -1 for t in r.blocked)
        n_seen, n_bias, n_blocked = n_seen + len(ids), n_bias + len(p.logit_bias), n_blocked + len(r.blocked)
    parts = [records.reshape(-1)] + seen_ids + seen_counts + [np.asarray(bias_ids, dtype=np.int32),
                                                              np.asarray(bias_values, dtype=np.float32).view(np.int32),
                                                              np.asarray(blocked, dtype=np.int32)]
    packed = torch.from_numpy(np.concatenate(parts).astype(np.int32, copy=False))
    return packed, (n_seen, n_bias, n_blocked)
