"""What a request asks to be done to its logits before a token is chosen: penalties on tokens seen before, biases,
end and stop ids that `min_tokens` still blocks, an allow list and bad words (rust/engine/src/sampling.rs:220-250, :252-274).  The host keeps
the counts and packs them for the kernel; the newest token of a request may still be on the device only."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .params import SamplingParams

# int32 words of a row record: three floats, then seen_off, seen_len, bias_off, bias_len, blocked_off, blocked_len, last_row,
# allowed_off, allowed_len, pairs_off, pairs_len
ROW_WORDS = 14


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
    arrays of `SeenTokens.lists`), ids blocked for now, the allow list, pairs (a, b) that block b if the newest token
    is a, and where the newest token lies on the device when the host does not know it yet."""
    params: SamplingParams
    seen: object
    blocked: Tuple[int, ...] = ()
    last_row: int = -1
    allowed: Tuple[int, ...] = ()
    pairs: Tuple[Tuple[int, int], ...] = ()

    def seen_lists(self) -> Tuple[np.ndarray, np.ndarray]:
        if isinstance(self.seen, dict):
            ids = np.fromiter((t if -(1 << 31) <= t < (1 << 31) else -1 for t in self.seen), dtype=np.int32, count=len(self.seen))
            return ids, np.fromiter(self.seen.values(), dtype=np.int32, count=len(self.seen))
        return self.seen


def bad_word_blocks(words: Sequence[Sequence[int]], tokens: Sequence[int], known: int) -> Tuple[List[int], List[Tuple[int, int]]]:
    """sampling.rs:241-248: the last token of a word is blocked when the tokens before it stand at the end of the history.
    `tokens[:known]` are final; one more token may follow that only the device knows: then a word whose other tokens
    fit is blocked on the condition that this token is the word's last but one.  Returns (blocked ids, (newest token,
    blocked id) pairs)."""
    blocked: List[int] = []
    pairs: List[Tuple[int, int]] = []
    pending = len(tokens) > known
    for word in words:
        *before, last = word
        if not pending:
            if len(before) <= known and list(tokens[known - len(before):known]) == before:
                blocked.append(last)
        elif not before:
            blocked.append(last)
        else:
            rest = before[:-1]
            if len(rest) <= known and list(tokens[known - len(rest):known]) == rest:
                pairs.append((before[-1], last))
    return blocked, pairs


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
    blocked: List[int] = []
    if generated < params.min_tokens:
        blocked = list(eos) + list(params.stop_token_ids)
    word_blocks, pairs = bad_word_blocks(params.bad_word_ids, tokens, known)
    if pairs:
        last_row = pending_row
    return AdjustRow(params, counts, tuple(dict.fromkeys(blocked + word_blocks)), last_row, params.allowed_token_ids, tuple(pairs))


def pack(rows: Sequence[Optional[AdjustRow]]) -> Tuple[torch.Tensor, Tuple[int, int, int, int, int]]:
    """The kernel's input for a step's rows (None: a row left alone) as one int32 CPU tensor, and the lengths of its
    five list sections (seen, bias, blocked, allowed, pairs)."""
    records = np.zeros((len(rows), ROW_WORDS), dtype=np.int32)
    floats = records.view(np.float32)
    seen_ids, seen_counts, bias_ids, bias_values, blocked, allowed, if_last, then_blocked = [], [], [], [], [], [], [], []
    n_seen = n_bias = n_blocked = n_allowed = n_pairs = 0
    word = lambda t: t if -(1 << 31) <= t < (1 << 31) else -1
    for i, r in enumerate(rows):
        if r is None:
            floats[i, 0] = 1.0
            records[i, 9] = -1
            continue
        p = r.params
        ids, counts = r.seen_lists()
        # a window of no tokens: the penalties see nothing, not even the newest token that `last_row` names for the pairs
        floats[i, 0:3] = (p.repetition_penalty, p.presence_penalty, p.frequency_penalty) if p.repeat_last_n != 0 else (1.0, 0.0, 0.0)
        records[i, 3:] = (n_seen, len(ids), n_bias, len(p.logit_bias), n_blocked, len(r.blocked), r.last_row,
                          n_allowed, len(r.allowed), n_pairs, len(r.pairs))
        seen_ids.append(ids)
        seen_counts.append(counts)
        bias_ids.extend(word(t) for t, _ in p.logit_bias)
        bias_values.extend(b for _, b in p.logit_bias)
        blocked.extend(word(t) for t in r.blocked)
        allowed.extend(min(t, (1 << 31) - 1) for t in sorted(r.allowed))
        if_last.extend(word(a) for a, _ in r.pairs)
        then_blocked.extend(word(b) for _, b in r.pairs)
        n_seen, n_bias, n_blocked = n_seen + len(ids), n_bias + len(p.logit_bias), n_blocked + len(r.blocked)
        n_allowed, n_pairs = n_allowed + len(r.allowed), n_pairs + len(r.pairs)
    parts = [records.reshape(-1)] + seen_ids + seen_counts + [np.asarray(bias_ids, dtype=np.int32),
                                                              np.asarray(bias_values, dtype=np.float32).view(np.int32)]
    parts += [np.asarray(a, dtype=np.int32) for a in (blocked, allowed, if_last, then_blocked)]
    packed = torch.from_numpy(np.concatenate(parts).astype(np.int32, copy=False))
    return packed, (n_seen, n_bias, n_blocked, n_allowed, n_pairs)
