"""Plain PyTorch versions of every kernel of the library, one function per kernel, with the
kernels' own signatures.  They compute in float64 on whatever device the tensors are on and
round once to the output type.

Two uses: the GPU tests compare each HIP kernel with its function here, and the CPU tests hand
a `ReferenceOps` to the engine in place of the kernel library, so that the step function, the
cache and the scheduler can be exercised without a GPU.  The product never imports this file.
"""
import math

import numpy as np
import torch

import plain_llama


class ReferenceOps:
    def embed(self, ids, table, out, scale=1.0):
        out.copy_((table[ids.long()].double() * scale).to(out.dtype))
        return out

    def rmsnorm(self, x, weight, eps, out, rows=None):
        src = x if rows is None else x[rows.long()]
        src = src.double()
        inv = 1.0 / torch.sqrt((src * src).sum(-1, keepdim=True) / src.shape[-1] + eps)
        out.copy_((src * (inv * weight.double())).to(out.dtype))
        return out

    def linear(self, x, w, out, bias=None, accumulate=False):
        y = x.double() @ w.double().T
        if bias is not None:
            y = y + bias.double()
        if accumulate:
            out.add_(y.to(out.dtype))
        else:
            out.copy_(y.to(out.dtype))
        return out

    # fused forms of decode steps: the same formulas, composed
    def fused_decode_supported(self, rows, width):
        return 1 <= rows <= 16 and width % 8 == 0

    def _normed(self, x, norm_weight, eps):
        x = x.double()
        return x * (torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * norm_weight.double())

    def norm_linear(self, x, norm_weight, eps, w, out, bias=None):
        y = self._normed(x, norm_weight, eps) @ w.double().T
        out.copy_((y if bias is None else y + bias.double()).to(out.dtype))
        return out

    def gate_up_swiglu(self, x, w_gate_up, out, bias=None):
        y = x.double() @ w_gate_up.double().T
        if bias is not None:
            y = y + bias.double()
        inter = y.shape[1] // 2
        g, u = y[:, :inter], y[:, inter:]
        out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
        return out

    def norm_gate_up_swiglu(self, x, norm_weight, eps, w_gate_up, out, bias=None):
        y = self._normed(x, norm_weight, eps) @ w_gate_up.double().T
        if bias is not None:
            y = y + bias.double()
        inter = y.shape[1] // 2
        g, u = y[:, :inter], y[:, inter:]
        out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
        return out

    def norm_qkv_rope_store(self, x, norm_weight, eps, w_qkv, q_out, row_pos, row_seg, tables, cos, sin, k_pages, v_pages,
                            heads, kv_heads, head_dim, rope_dims, page_size, bias=None):
        y = self._normed(x, norm_weight, eps) @ w_qkv.double().T
        if bias is not None:
            y = y + bias.double()
        qkv = y.clone()                 # rotated in float64, rounded once when stored
        kp = None if k_pages is None else k_pages.double()
        vp = None if v_pages is None else v_pages.double()
        self.rope_kv_store(qkv, row_pos, row_seg, tables, cos, sin, kp, vp, heads, kv_heads, head_dim, rope_dims, 1, page_size)
        q_out.copy_(qkv[:, : heads * head_dim].to(q_out.dtype))
        if k_pages is not None:
            k_pages.copy_(kp.to(k_pages.dtype))
            v_pages.copy_(vp.to(v_pages.dtype))
        return q_out

    def add_rmsnorm(self, x, branch, weight, eps, out):
        x.add_(branch.to(x.dtype))
        return self.rmsnorm(x, weight, eps, out)

    def add_residual(self, residual, branch):
        residual.add_(branch.to(residual.dtype))
        return residual

    def swiglu(self, gate_up, out):
        inter = gate_up.shape[1] // 2
        g, u = gate_up[:, :inter].double(), gate_up[:, inter:].double()
        out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
        return out

    def rope_kv_store(self, qkv, row_pos, row_seg, tables, cos, sin, k_pages, v_pages, heads, kv_heads, head_dim,
                      rope_dims, pairing, page_size):
        rows = qkv.shape[0]
        half = rope_dims // 2
        view = qkv.view(rows, heads + 2 * kv_heads, head_dim)
        for r in range(rows):
            seg = int(row_seg[r])
            if seg < 0:
                continue
            pos = int(row_pos[r])
            c, s = cos[pos].double(), sin[pos].double()
            if pairing == 0:
                ia, ib = torch.arange(half), torch.arange(half) + half
            else:
                ia, ib = torch.arange(half) * 2, torch.arange(half) * 2 + 1
            ia, ib = ia.to(qkv.device), ib.to(qkv.device)
            for h in range(heads + kv_heads):
                a, b = view[r, h, ia].double(), view[r, h, ib].double()
                view[r, h, ia] = (a * c - b * s).to(qkv.dtype)
                view[r, h, ib] = (b * c + a * s).to(qkv.dtype)
            if k_pages is None:
                continue
            page = int(tables[seg, pos // page_size])
            off = pos % page_size
            # keys lie chunk by chunk in a page: [page][kv_head][head_dim / 8][token][8]
            k_pages[page, :, :, off, :] = view[r, heads:heads + kv_heads, :].reshape(kv_heads, head_dim // 8, 8)
            v_pages[page, :, :, off] = view[r, heads + kv_heads:, :]

    def attention_workspace_bytes(self, rows, heads, kv_heads, head_dim, max_context):
        return 0

    def attention(self, q, k_pages, v_pages, tables, row_pos, row_seg, seg_start, out, heads, kv_heads, head_dim, page_size, scale,
                  window, max_context, uniform_rows=0, workspace=None, single_from=None, head_slopes=None):
        rows = q.shape[0]
        group = heads // kv_heads
        for r in range(rows):
            seg = int(row_seg[r])
            if seg < 0:
                out[r] = 0
                continue
            pos = int(row_pos[r])
            n = pos + 1
            lo = max(0, n - window) if window else 0
            keys = torch.arange(lo, n, device=q.device)
            pages = tables[seg, (keys // page_size).long()].long()
            offs = (keys % page_size).long()
            k = k_pages[pages, :, :, offs, :].double().reshape(len(keys), kv_heads, head_dim)     # [n, kv_heads, d]
            v = v_pages[pages, :, :, offs].double()          # [n, kv_heads, d]
            qr = q[r].double().view(heads, head_dim)
            for h in range(heads):
                s = (k[:, h // group, :] @ qr[h]) * scale
                if head_slopes is not None:
                    s = s + float(head_slopes[h]) * (keys - pos).double()
                p = torch.softmax(s, dim=0)
                out[r, h * head_dim:(h + 1) * head_dim] = (p @ v[:, h // group, :]).to(out.dtype)
        return out

    def carry_ids(self, ids, source, previous):
        for r in range(ids.numel()):
            if int(source[r]) >= 0:
                ids[r] = previous[int(source[r])]
        return ids

    def argmax(self, logits, out):
        for r in range(logits.shape[0]):
            row = logits[r].float().cpu().numpy()
            row = np.where(np.isfinite(row), row, -np.inf)
            out[r] = 0 if not np.isfinite(row).any() else plain_llama.greedy(row)
        return out

    def adjust_logits(self, logits, packed, sections, last_tokens=None):
        """The packed lists of `Ops.adjust_logits`, taken apart here and applied with the plain functions."""
        rows, vocab = logits.shape
        seen, bias, blocked, allowed, pairs = (int(n) for n in sections)
        words = packed.cpu().numpy().astype(np.int32)
        at = rows * 14
        lists = []
        for count in (seen, seen, bias, bias, blocked, allowed, pairs, pairs):
            lists.append(words[at:at + count])
            at += count
        seen_ids, seen_counts, bias_ids, bias_values, blocked_ids, allowed_ids, if_last, then_blocked = lists
        bias_values = bias_values.view(np.float32)
        for r in range(rows):
            rec = words[r * 14:(r + 1) * 14]
            rep, pres, freq = (float(v) for v in rec[:3].view(np.float32))
            (seen_off, seen_len, bias_off, bias_len, blocked_off, blocked_len, last_row, allowed_off, allowed_len,
             pairs_off, pairs_len) = (int(v) for v in rec[3:])
            history = []
            for t, n in zip(seen_ids[seen_off:seen_off + seen_len], seen_counts[seen_off:seen_off + seen_len]):
                history += [int(t)] * int(n)
            last = int(last_tokens[last_row]) if last_row >= 0 else -1
            if last_row >= 0:
                history.append(last)
            row = plain_llama.apply_penalties(logits[r].float().cpu().numpy(), history, rep, pres, freq, -1,
                                              list(zip(bias_ids[bias_off:bias_off + bias_len].tolist(),
                                                       bias_values[bias_off:bias_off + bias_len].tolist())))
            row[[int(t) for t in blocked_ids[blocked_off:blocked_off + blocked_len] if 0 <= t < vocab]] = -np.inf
            for a, b in zip(if_last[pairs_off:pairs_off + pairs_len], then_blocked[pairs_off:pairs_off + pairs_len]):
                if int(a) == last and 0 <= b < vocab:
                    row[int(b)] = -np.inf
            if allowed_len:
                row = plain_llama.apply_generation_controls(row, 0, 0, (), (), allowed_ids[allowed_off:allowed_off + allowed_len].tolist())
            logits[r] = torch.from_numpy(row).to(logits.dtype)
        return logits

    def logprobs(self, logits, wanted_rows, tokens, top, values, ids):
        for w, r in enumerate(int(r) for r in wanted_rows):
            got = plain_llama.raw_logprobs(logits[r].float().cpu().numpy(), int(tokens[r]), top)
            ids[w, 0] = int(tokens[r])
            if got is None:
                values[w] = float("nan")
                ids[w, 1:] = torch.tensor([-1] * top, dtype=ids.dtype)
                continue
            values[w, 0] = got[0]
            for k in range(top):
                ids[w, 1 + k] = got[1][k][0] if k < len(got[1]) else -1
                values[w, 1 + k] = got[1][k][1] if k < len(got[1]) else float("nan")

    def logprobs_processed(self, logits, wanted_rows, tokens, params, top, values, ids):
        rec = np.frombuffer(params.cpu().numpy().tobytes(), dtype=np.dtype([("temperature", "<f4"), ("top_p", "<f4"), ("top_k", "<i4"),
                                                                            ("min_p", "<f4"), ("seed", "<u8"), ("draw", "<u8")]))
        for w, r in enumerate(int(r) for r in wanted_rows):
            p = rec[r]
            got = plain_llama.processed_logprobs(logits[r].float().cpu().numpy(), int(tokens[r]), top, float(p["temperature"]),
                                                 int(p["top_k"]), float(p["top_p"]), float(p["min_p"]))
            ids[w, 0] = int(tokens[r])
            if got is None:
                values[w] = float("nan")
                ids[w, 1:] = torch.tensor([-1] * top, dtype=ids.dtype)
                continue
            values[w, 0] = got[0]
            for k in range(top):
                ids[w, 1 + k] = got[1][k][0] if k < len(got[1]) else -1
                values[w, 1 + k] = got[1][k][1] if k < len(got[1]) else float("nan")

    def sample(self, logits, work, params, out, kinds=3):
        raw = params.cpu().numpy().tobytes()
        rec = np.frombuffer(raw, dtype=np.dtype([("temperature", "<f4"), ("top_p", "<f4"), ("top_k", "<i4"),
                                                 ("min_p", "<f4"), ("seed", "<u8"), ("draw", "<u8")]))
        for r in range(logits.shape[0]):
            p = rec[r]
            out[r] = plain_llama.device_sample(logits[r].float().cpu().numpy(), float(p["temperature"]), int(p["top_k"]),
                                               float(p["top_p"]), int(p["seed"]), int(p["draw"]), float(p["min_p"]))
        return out
