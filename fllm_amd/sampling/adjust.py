"""What a request asks to be done to its logits before a token is chosen: penalties on tokens seen before, biases,
and end and stop ids that `min_tokens` still blocks (rust/engine/src/sampling.rs:220-229, :252-274).  The host keeps
the counts and packs them for the kernel; the newest token of a request may still be on the device only."""
from __future__ import annotations

import struct
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .params import SamplingParams

ROW_WORDS = 10      # int32 words of a row record: three floats, then seen_off, seen_len, bias_off, bias_len, blocked_off, blocked_len, last_row


@dataclass
class SeenTokens:
    """How often each token occurs among the first `upto` tokens of a request (all of them count; a window is cut
    out of the token list itself)."""
    counts: Dict[int, int] = field(default_factory=dict)
    upto: int = 0

    def catch_up(self, tokens: Sequence[int], known: int) -> None:
        for t in tokens[self.upto:known]:
            self.counts[t] = self.counts.get(t, 0) + 1
        self.upto = max(self.upto, known)


@dataclass
class AdjustRow:
    """One row's share: the distinct tokens seen (within the window) with their counts, biases, ids blocked for now, and
    where the newest token lies on the device when the host does not know it yet."""
    params: SamplingParams
    seen: Dict[int, int]
    blocked: Tuple[int, ...] = ()
    last_row: int = -1


def row_for(params: SamplingParams, tokens: Sequence[int], prompt_len: int, pending_row: Optional[int], eos: Sequence[int],
            seen: Optional[SeenTokens] = None) -> Optional[AdjustRow]:
    """The adjustment of the next token of a request whose tokens so far are `tokens`; the last of them is a
    placeholder when `pending_row` is given (its value is row `pending_row` of the tokens of the step in flight).
    None when the request asks for nothing.  `seen`: counts kept from step to step (no window)."""
    generated = len(tokens) - prompt_len
    if not params.adjusts_logits(generated):
        return None
    known = len(tokens) - (1 if pending_row is not None else 0)
    counts: Dict[int, int] = {}
    last_row = -1
    if params.penalizes:
        n = params.repeat_last_n
        if n < 0 and seen is not None:
            seen.catch_up(tokens, known)
            counts = seen.counts
        else:
            first = 0 if n < 0 else max(0, len(tokens) - n)
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
    records, seen_ids, seen_counts, bias_ids, bias_values, blocked = [], [], [], [], [], []
    for r in rows:
        if r is None:
            records.append(struct.pack("<fffiiiiiii", 1.0, 0.0, 0.0, 0, 0, 0, 0, 0, 0, -1))
            continue
        p = r.params
        records.append(struct.pack("<fffiiiiiii", float(p.repetition_penalty), float(p.presence_penalty), float(p.frequency_penalty),
                                   len(seen_ids), len(r.seen), len(bias_ids), len(p.logit_bias), len(blocked), len(r.blocked),
                                   int(r.last_row)))
        seen_ids.extend(r.seen.keys())
        seen_counts.extend(r.seen.values())
        bias_ids.extend(t for t, _ in p.logit_bias)
        bias_values.extend(b for _, b in p.logit_bias)
        blocked.extend(r.blocked)
    clip = lambda ids: [t if -(1 << 31) <= t < (1 << 31) else -1 for t in ids]
    raw = (b"".join(records) + struct.pack(f"<{len(seen_ids)}i", *clip(seen_ids)) + struct.pack(f"<{len(seen_counts)}i", *seen_counts)
           + struct.pack(f"<{len(bias_ids)}i", *clip(bias_ids)) + struct.pack(f"<{len(bias_values)}f", *bias_values)
           + struct.pack(f"<{len(blocked)}i", *clip(blocked)))
    packed = torch.frombuffer(bytearray(raw), dtype=torch.int32).clone()
    return packed, (len(seen_ids), len(bias_ids), len(blocked))
