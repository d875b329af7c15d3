"""Chooses tokens from logits on the device: argmax for greedy rows, the device sampler
otherwise (temperature, top-k, top-p, Gumbel-max draw keyed by seed and draw number)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from .params import SamplingParams


@dataclass
class SampleRequest:
    params: SamplingParams
    seed: int
    draw: int


SMALL_TOP_K = 64     # rows with a top-k up to this are shared by several workgroups (the kernel's own limit)
_RECORD = 32   # bytes of one row record: float temperature, float top_p, int32 top_k, float min_p, uint64 seed, uint64 draw


def pack_rows(rows: Sequence[SampleRequest]) -> torch.Tensor:
    """The row records the sampling kernel reads, as a uint8 CPU tensor [rows, 32]."""
    import struct
    raw = bytearray()
    for r in rows:
        p = r.params
        raw += struct.pack("<ffifQQ", float(p.temperature), float(p.top_p), int(p.top_k), float(p.min_p),
                           int(r.seed) & ((1 << 64) - 1), int(r.draw))
    return torch.frombuffer(raw, dtype=torch.uint8).view(len(rows), _RECORD).clone()


def draws_from_all(p: SamplingParams, vocab: int) -> bool:
    """A temperature and none of top-k, top-p and min-p: the kernel's own test, on the float32 values that the row record
    holds (a temperature or top-p that rounds across its limit must be judged as the kernel judges it)."""
    import struct
    temperature, top_p, min_p = struct.unpack("<fff", struct.pack("<fff", float(p.temperature), float(p.top_p), float(p.min_p)))
    limit = struct.unpack("<f", struct.pack("<f", 1e-5))[0]
    return temperature > limit and not (0 < int(p.top_k) < vocab) and not (0.0 < top_p < 1.0) and not min_p > 0.0


class Sampler:
    def __init__(self, rt):
        self.rt = rt

    def adjust(self, logits: torch.Tensor, rows, last_tokens=None) -> torch.Tensor:
        """Penalties, biases and blocked ids of the rows that ask for any (`rows`: one `AdjustRow` or None a row of
        `logits`), on the logits in place; nothing is launched when no row asks.  `last_tokens`: the device tensor that
        the rows' `last_row` points into."""
        if all(r is None for r in rows):
            return logits
        pointing = [r.last_row for r in rows if r is not None and r.last_row >= 0]
        if pointing and (last_tokens is None or max(pointing) >= last_tokens.numel()):
            raise ValueError(f"rows name their newest token at index {max(pointing)} of `last_tokens`, which "
                             + ("was not given" if last_tokens is None else f"holds {last_tokens.numel()} tokens"))
        from .adjust import pack
        packed, sections = pack(rows)
        if logits.is_cuda:
            packed = packed.pin_memory().to(logits.device, non_blocking=True)
        self.rt.ops.adjust_logits(logits, packed, sections, last_tokens)
        return logits

    def sample(self, logits: torch.Tensor, rows: Sequence[SampleRequest]) -> List[int]:
        """`logits`: float32 [len(rows), vocab] on the device.  Returns one token id per row."""
        return self.read(self.launch(logits, rows))

    @staticmethod
    def start_read(tokens: torch.Tensor):
        """Asks for the tokens of `launch` on the host without waiting: the copy into pinned memory is queued right
        behind the kernels that choose them, and an event marks its end.  What is launched after this call does not
        delay the read.  Returns what `finish_read` takes."""
        if not tokens.is_cuda or tokens.numel() == 0:
            return tokens, None
        host = torch.empty(tokens.shape, dtype=tokens.dtype, pin_memory=True)
        host.copy_(tokens, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return host, done

    @staticmethod
    def finish_read(pending) -> List[int]:
        """The token ids on the host; waits until the copy that `start_read` queued has ended."""
        host, done = pending
        if done is not None:
            done.synchronize()
        return [int(t) for t in host.tolist()]

    @classmethod
    def read(cls, tokens: torch.Tensor) -> List[int]:
        """The token ids of `launch` on the host (waits for the device)."""
        return cls.finish_read(cls.start_read(tokens))

    def start_logprobs(self, logits: torch.Tensor, tokens: torch.Tensor, wanted: Sequence[int], top: int,
                       processed: Sequence[int] = (), seen: Optional[torch.Tensor] = None,
                       requests: Optional[Sequence[SampleRequest]] = None):
        """Asks for the log-probabilities of `tokens[r]` and of the `top` likeliest tokens in the softmax of `logits[r]`
        (as the model gave them: hand in the logits as they were before `adjust`), for the rows r in `wanted`.  The
        rows in `processed` get theirs in the distribution they were drawn from instead (`SamplingParams.
        logprobs_processed`): from `seen`, the logits as the sampler saw them, and `requests`, what `launch` took.
        Nothing waits: the kernels and the copies to the host are queued behind what chose the tokens.  Returns what
        `finish_logprobs` takes."""
        wanted, processed = [int(r) for r in wanted], [int(r) for r in processed]
        if any(not 0 <= r < logits.shape[0] for r in wanted + processed):
            raise ValueError(f"log-probabilities asked for rows {wanted + processed} of {logits.shape[0]}")
        if processed and (seen is None or requests is None or len(requests) != logits.shape[0]):
            raise ValueError("processed log-probabilities need the logits the sampler saw and its requests, one a row")
        top = min(int(top), logits.shape[1])
        rows = torch.tensor(wanted + processed, dtype=torch.int32)
        if logits.is_cuda:
            rows = rows.pin_memory().to(logits.device, non_blocking=True)
        values = torch.empty((len(wanted) + len(processed), 1 + top), dtype=torch.float32, device=logits.device)
        ids = torch.empty((len(wanted) + len(processed), 1 + top), dtype=torch.int32, device=logits.device)
        n = len(wanted)
        if wanted:
            self.rt.ops.logprobs(logits, rows[:n], tokens, top, values[:n], ids[:n])
        if processed:
            params = pack_rows(requests)
            if seen.is_cuda:
                params = params.pin_memory().to(seen.device, non_blocking=True)
            self.rt.ops.logprobs_processed(seen, rows[n:], tokens, params, top, values[n:], ids[n:])
        return wanted + processed, self.start_read(values), self.start_read(ids)

    @staticmethod
    def finish_logprobs(pending) -> dict:
        """{row: (log-probability of the chosen token, [(token id, log-probability), ...] likeliest first)}; waits for
        the copies."""
        wanted, (values, values_done), (ids, ids_done) = pending
        for done in (values_done, ids_done):
            if done is not None:
                done.synchronize()
        values, ids = values.tolist(), ids.tolist()
        return {r: (values[w][0], [(int(i), v) for i, v in zip(ids[w][1:], values[w][1:]) if i >= 0])
                for w, r in enumerate(wanted)}

    def launch(self, logits: torch.Tensor, rows: Sequence[SampleRequest]) -> torch.Tensor:
        """Starts the choice of one token per row and returns the int32 device tensor that will
        hold them; nothing waits for the device."""
        count = logits.shape[0]
        if count != len(rows):
            raise ValueError(f"{count} rows of logits for {len(rows)} requests")
        out = torch.empty(count, dtype=torch.int32, device=logits.device)
        if count == 0:
            return out
        if all(r.params.greedy for r in rows):
            self.rt.ops.argmax(logits, out)
        else:
            params = pack_rows(rows)
            if logits.is_cuda:      # from pinned memory, so that the copy does not wait for the device
                params = params.pin_memory().to(logits.device, non_blocking=True)
            work = torch.empty_like(logits)
            vocab = logits.shape[1]
            from_all = [draws_from_all(r.params, vocab) for r in rows]
            kinds = 1 if all(from_all) else (3 if any(from_all) else 2)
            if any(0 < int(r.params.top_k) <= SMALL_TOP_K and not r.params.greedy for r in rows):
                kinds |= 4          # rows with a small top-k: several workgroups a row
            self.rt.ops.sample(logits, work, params, out, kinds)
        return out
