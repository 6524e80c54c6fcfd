"""Helpers to call one part alone on the GPU: a runtime, a step context built
by hand (not by the engine), and a paged cache with scattered pages."""

import torch

from kllm_amd.parts import PagedCacheView, Runtime, StepContext

DEV = "cuda"


def runtime(dtype):
    return Runtime(device=torch.device(DEV), dtype=dtype)


def context(rt, spans, page_size=16, tables=None, token_ids=None, want_rows=None):
    """spans: list of (start position, length)."""
    n = sum(l for _, l in spans)
    S = len(spans)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    starts = [0]
    for _, l in spans:
        starts.append(starts[-1] + l)
    if tables is None:
        tables, nxt = [], 0
        for p0, l in spans:
            cnt = -(-(p0 + l) // page_size)
            tables.append(list(range(nxt, nxt + cnt)))
            nxt += cnt
    maxp = max(len(t) for t in tables)
    bt = i32([t + [-1] * (maxp - len(t)) for t in tables])
    return StepContext(
        n=n, n_spans=S,
        token_ids=i32(token_ids if token_ids is not None else [0] * n),
        positions=i32([p0 + i for p0, l in spans for i in range(l)]),
        span_of_token=i32([s for s, (_, l) in enumerate(spans) for _ in range(l)]),
        span_start=i32(starts), span_pos=i32([p0 for p0, _ in spans]), slots=i32(list(range(S))),
        logit_rows=i32(want_rows) if want_rows else None,
        h_span_start=starts, h_span_pos=[p0 for p0, _ in spans], h_span_len=[l for _, l in spans],
        block_tables=[bt], runtime=rt, max_span_len=max(l for _, l in spans),
        all_decode=all(l == 1 for _, l in spans))


def empty_cache(num_pages, kv_heads, head_dim, page_size, dtype):
    return torch.full((num_pages, 2, kv_heads, page_size * head_dim), float("nan"), dtype=dtype, device=DEV)


def view(cache, ctx, page_size=16, write=True):
    return PagedCacheView(cache, ctx.block_tables[0], page_size, write)
