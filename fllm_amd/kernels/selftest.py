"""`selftest-gpu`: every kernel on random data on the device against PyTorch computing the same
formula in float64, in the manner of the reference's op self-test
(rust/engine/src/backend/selftest.rs:1-47, groups :74-102).  Prints one line per check."""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional

import torch

GROUPS = ["embedding", "norm", "linear", "fused", "activation", "rope_kv", "attention", "sampling"]


def _err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double() - want.double()).abs().max() / max(1e-30, float(want.double().abs().max())))


def _embedding(ops, dev, report):
    for dtype in (torch.float32, torch.bfloat16):
        table = torch.randn(515, 160, device=dev).to(dtype)
        ids = torch.randint(0, 515, (13,), device=dev, dtype=torch.int32)
        got = ops.embed(ids, table, torch.empty(13, 160, device=dev))
        report(f"embed {dtype}", _err(got, table[ids.long()].float()), 0.0)


def _norm(ops, dev, report):
    x = torch.randn(13, 4104, device=dev) * 3
    w = 1 + 0.1 * torch.randn(4104, device=dev)
    want = x.double() * (torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * w.double())
    report("rmsnorm f32", _err(ops.rmsnorm(x, w, 1e-5, torch.empty_like(x)), want), 4e-6)
    report("rmsnorm bf16", _err(ops.rmsnorm(x, w, 1e-5, torch.empty_like(x, dtype=torch.bfloat16)), want), 2 ** -8)


def _linear(ops, dev, report):
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-5)):
        for M, N, K in ((1, 4096, 4096), (5, 520, 264), (8, 6144, 4096), (8, 4096, 14336), (64, 1000, 4096), (200, 384, 1024),
                        (13, 100, 72)):
            x = torch.randn(M, K, device=dev).to(dtype)
            w = (torch.randn(N, K, device=dev) / math.sqrt(K)).to(dtype)
            want = x.double() @ w.double().T
            got = ops.linear(x, w, torch.empty(M, N, device=dev, dtype=torch.float32))
            report(f"linear {dtype} {M}x{N}x{K}", _err(got, want), tol)


def _fused(ops, dev, report):
    """The decode forms: RMSNorm folded into the product, SwiGLU in its epilogue."""
    for M, N, K in ((1, 4096, 4096), (8, 6144, 4096), (16, 520, 264), (9, 96, 14336)):
        x = torch.randn(M, K, device=dev) * (1 + 4 * torch.rand(M, 1, device=dev))
        nw = 1 + 0.1 * torch.randn(K, device=dev)
        w = (torch.randn(N, K, device=dev) / math.sqrt(K)).to(torch.bfloat16)
        normed = x.double() * (torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * nw.double())
        got = ops.norm_linear(x, nw, 1e-5, w, torch.empty(M, N, device=dev, dtype=torch.bfloat16))
        report(f"norm_linear {M}x{N}x{K}", _err(got, normed @ w.double().T), 2 ** -6)
    for M, inter, K in ((1, 14336, 4096), (8, 432, 160), (13, 1000, 4096)):
        x = torch.randn(M, K, device=dev) * 2
        nw = 1 + 0.1 * torch.randn(K, device=dev)
        w = (torch.randn(2 * inter, K, device=dev) / math.sqrt(K)).to(torch.bfloat16)
        normed = x.double() * (torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * nw.double())
        gu = normed @ w.double().T
        g, u = gu[:, :inter], gu[:, inter:]
        got = ops.norm_gate_up_swiglu(x, nw, 1e-5, w, torch.empty(M, inter, device=dev, dtype=torch.bfloat16))
        report(f"norm_gate_up_swiglu {M}x{inter}x{K}", _err(got, g * torch.sigmoid(g) * u), 2 ** -6)


def _activation(ops, dev, report):
    gu = torch.randn(13, 2 * 432, device=dev) * 3
    g, u = gu[:, :432].double(), gu[:, 432:].double()
    report("swiglu f32", _err(ops.swiglu(gu, torch.empty(13, 432, device=dev)), g * torch.sigmoid(g) * u), 4e-6)


def _paged(dev, dtype, segs, kv_heads, head_dim, page_size):
    ctx = max(p + n for p, n in segs)
    pages_each = -(-ctx // page_size)
    num_pages = len(segs) * pages_each + 1
    tables = torch.randperm(num_pages, device=dev)[: len(segs) * pages_each].to(torch.int32).view(len(segs), pages_each)
    k = torch.randn(num_pages, kv_heads, head_dim // 8, page_size, 8, device=dev).to(dtype)      # keys chunk by chunk in a page
    v = torch.randn(num_pages, kv_heads, head_dim, page_size, device=dev).to(dtype)
    row_pos = torch.tensor([p + i for p, n in segs for i in range(n)], dtype=torch.int32, device=dev)
    row_seg = torch.tensor([s for s, (_, n) in enumerate(segs) for _ in range(n)], dtype=torch.int32, device=dev)
    starts = [0]
    for _, n in segs:
        starts.append(starts[-1] + n)
    return tables, k, v, row_pos, row_seg, torch.tensor(starts, dtype=torch.int32, device=dev), ctx


def _rope_kv(ops, dev, report):
    heads, kv_heads, d, ps = 8, 2, 64, 16
    segs = [(0, 5), (37, 1), (15, 3)]
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 2 ** -8)):
        tables, k, v, row_pos, row_seg, _, ctx = _paged(dev, dtype, segs, kv_heads, d, ps)
        angle = torch.rand(64, d // 2, device=dev, dtype=torch.float64) * 6.28
        cos, sin = angle.cos().float(), angle.sin().float()
        qkv = torch.randn(row_pos.numel(), (heads + 2 * kv_heads) * d, device=dev).to(dtype)
        view = qkv.double().view(-1, heads + 2 * kv_heads, d)
        c, s = cos[row_pos.long()].double()[:, None, :], sin[row_pos.long()].double()[:, None, :]
        a, b = view[:, : heads + kv_heads, : d // 2], view[:, : heads + kv_heads, d // 2:]
        rotated = torch.cat([a * c - b * s, b * c + a * s], dim=-1)
        ops.rope_kv_store(qkv, row_pos, row_seg, tables, cos, sin, k, v, heads, kv_heads, d, d, 0, ps)
        report(f"rope q {dtype}", _err(qkv.view(-1, heads + 2 * kv_heads, d)[:, :heads], rotated[:, :heads]), tol)
        pages = tables[row_seg.long(), (row_pos // ps).long()].long()
        offs = (row_pos % ps).long()
        report(f"rope k pages {dtype}", _err(k[pages, :, :, offs, :].reshape(len(pages), kv_heads, d), rotated[:, heads:]), tol)
        report(f"v pages {dtype}", _err(v[pages, :, :, offs], view[:, heads + kv_heads:]), 0.0)


def _attention(ops, dev, report):
    heads, kv_heads, d, ps = 8, 2, 64, 16
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        for segs, window in (([(700, 1), (31, 1), (128, 1)], None), ([(100, 17), (0, 70)], None), ([(300, 40)], 64)):
            tables, k, v, row_pos, row_seg, seg_start, ctx = _paged(dev, dtype, segs, kv_heads, d, ps)
            rows = row_pos.numel()
            q = torch.randn(rows, heads * d, device=dev).to(dtype)
            want = torch.empty(rows, heads, d, dtype=torch.float64, device=dev)
            for r in range(rows):
                pos, seg = int(row_pos[r]), int(row_seg[r])
                lo = max(0, pos + 1 - window) if window else 0
                keys = torch.arange(lo, pos + 1, device=dev)
                pg, off = tables[seg, (keys // ps).long()].long(), (keys % ps).long()
                kk = k[pg, :, :, off, :].double().reshape(len(keys), kv_heads, d).repeat_interleave(heads // kv_heads, 1)      # [n, heads, d]
                vv = v[pg, :, :, off].double().repeat_interleave(heads // kv_heads, 1)
                sc = torch.einsum("hd,nhd->hn", q[r].double().view(heads, d), kk) * d ** -0.5
                want[r] = torch.einsum("hn,nhd->hd", torch.softmax(sc, -1), vv)
            uniform = int(all(n == 1 for _, n in segs))
            nbytes = ops.attention_workspace_bytes(rows, heads, kv_heads, d, ctx)
            ws = torch.empty(max(1, nbytes), dtype=torch.uint8, device=dev)
            got = ops.attention(q, k, v, tables, row_pos, row_seg, seg_start, torch.empty(rows, heads * d, dtype=dtype, device=dev),
                                heads, kv_heads, d, ps, d ** -0.5, window, ctx, uniform_rows=uniform, workspace=ws)
            report(f"attention {dtype} {segs} window={window}", _err(got, want.view(rows, -1)), tol)


def _sampling(ops, dev, report):
    logits = torch.randn(5, 1000, device=dev)
    logits[0, 7] = logits[0, 900] = 60.0
    got = ops.argmax(logits, torch.empty(5, dtype=torch.int32, device=dev))
    ok = int(got[0]) == 7 and all(int(got[r]) == int(logits[r].argmax()) for r in range(1, 5))
    report("argmax first maximum", 0.0 if ok else 1.0, 0.0)


_CHECKS: Dict[str, Callable] = {"embedding": _embedding, "norm": _norm, "linear": _linear, "fused": _fused, "activation": _activation,
                                "rope_kv": _rope_kv, "attention": _attention, "sampling": _sampling}


def run(only: Optional[List[str]] = None, device: str = "cuda:0") -> int:
    from . import Ops
    ops = Ops()
    torch.manual_seed(0)
    failed = 0

    def report(name: str, err: float, tol: float) -> None:
        nonlocal failed
        ok = err <= tol
        failed += 0 if ok else 1
        print(f"{'ok  ' if ok else 'FAIL'} {name}: relative error {err:.3e} (limit {tol:.1e})", flush=True)

    for group in only or GROUPS:
        if group not in _CHECKS:
            print(f"unknown group {group!r}; groups: {', '.join(GROUPS)}")
            return 2
        print(f"[{group}]", flush=True)
        _CHECKS[group](ops, device, report)
    print("selftest: all checks passed" if not failed else f"selftest: {failed} checks FAILED")
    return 1 if failed else 0
