"""Attention over a context of more than 32,768 keys, at the sizes at which long contexts are
served: pages of 16 tokens scattered over a pool of more than 40,000 pages (page numbers past
2**15, byte offsets past 2**31 in fp32), the key range of a single token in 1, 8 and 64 cuts,
and a query run of 2,048 tokens at the end of the sequence in items of one and of two row tiles,
paired and alone.  Every result is compared with ``plain.causal_attention`` on the CPU, computed
in float64 over one block of queries at a time.

Random scores over 32,768 keys average the values to nearly nothing, and a page read from the
wrong place would move the result by less than a tolerance.  So the queries are made peaked
(scores with a spread of about three, so that a few dozen keys carry the weight, other ones for
every query), and some queries are pointed at one key (the first, one in the middle, the last
before the run, the query's own) whose value the output must then equal.
(The cases of the reference's tests/test_paged_attention.py:59-74, scaled up.)"""

from __future__ import annotations

import math
import random

import pytest
import torch

from tests.plain import llama as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"
N = 32_800            # keys of the sequence: 2,050 pages of 16
POOL = 40_960         # pages in the pool
BS = 16
H, KV = 8, 2
RUN = 2048            # the query run at the end of the sequence


def ops():
    from kvforge_amd.kernels import ops as o
    return o


class LongCache:
    """One sequence of ``N`` keys in pages drawn at random from the whole pool (junk in every
    other page), built on the device page by page; keys and values of the sequence stay on the
    CPU in 32-bit, as the cache holds them (rounded to ``dtype``)."""

    def __init__(self, d: int, dtype: torch.dtype, seed: int) -> None:
        g = torch.Generator().manual_seed(seed)
        self.d, self.dtype = d, dtype
        self.keys = torch.randn(N, KV, d, generator=g).to(dtype).float()
        self.values = torch.randn(N, KV, d, generator=g).to(dtype).float()
        pages = random.Random(seed).sample(range(POOL), -(-N // BS))
        assert max(pages) >= 2 ** 15 and min(pages) < 2 ** 12
        self.table = torch.full((1, -(-N // BS) + 3), -1, dtype=torch.int32)
        self.table[0, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        dg = torch.Generator(device=DEV).manual_seed(seed)
        self.k = torch.randn(POOL, KV, BS, d, generator=dg, device=DEV, dtype=torch.float32).to(dtype)
        self.v = torch.randn(POOL, KV, d, BS, generator=dg, device=DEV, dtype=torch.float32).to(dtype)
        pad = len(pages) * BS - N
        kk = torch.cat([self.keys, torch.randn(pad, KV, d, generator=g)]).to(dtype)
        vv = torch.cat([self.values, torch.randn(pad, KV, d, generator=g)]).to(dtype)
        idx = torch.tensor(pages, device=DEV)
        self.k[idx] = kk.view(len(pages), BS, KV, d).permute(0, 2, 1, 3).to(DEV)
        self.v[idx] = vv.view(len(pages), BS, KV, d).permute(0, 2, 3, 1).to(DEV)
        self.table_dev = self.table.to(DEV)


_caches: dict = {}


def cache_for(d: int, dtype: torch.dtype) -> LongCache:
    """One cache per (head size, type) at a time: they are hundreds of megabytes each."""
    key = (d, dtype)
    if key not in _caches:
        _caches.clear()
        torch.cuda.empty_cache()
        _caches[key] = LongCache(d, dtype, seed=d)
    return _caches[key]


def peaked_queries(cache: LongCache, positions: list[int], pointed: dict[int, int], seed: int) -> torch.Tensor:
    """``[len(positions), H, d]``: random directions, long enough that the scores over the
    context spread by about three; row ``r`` in ``pointed`` looks at key ``pointed[r]`` alone
    (score 40 there, as in the far-key test of the short contexts)."""
    d = cache.d
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(len(positions), H, d, generator=g)
    q = q / q.norm(dim=-1, keepdim=True) * 3.0 * math.sqrt(d)
    for r, key_pos in pointed.items():
        assert key_pos <= positions[r]
        for h in range(H):
            key = cache.keys[key_pos, h // (H // KV)]
            q[r, h] = key * 40.0 / key.norm() ** 2 * math.sqrt(d)
    return q.to(cache.dtype)


def reference(cache: LongCache, q: torch.Tensor, first_pos: int, block: int = 128) -> torch.Tensor:
    """Queries at consecutive positions from ``first_pos`` on, in float64, a block at a time."""
    k64, v64 = cache.keys.double(), cache.values.double()
    scale = 1 / math.sqrt(cache.d)
    out = []
    for lo in range(0, q.shape[0], block):
        hi = min(q.shape[0], lo + block)
        last = first_pos + hi
        out.append(plain.causal_attention(q[lo:hi].double(), k64[:last], v64[:last], scale, first_pos + lo))
    return torch.cat(out).float()


def tolerance(dtype):
    # 32-bit: tens of thousands of terms, summed in other orders, with exponents of scores up to
    # 40 whose own rounding (2**-24 relative, so 2e-6 absolute) the weights inherit
    return dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("d", [128, 64])
def test_one_token_over_32k_keys_in_1_8_and_64_cuts(d, dtype):
    cache = cache_for(d, dtype)
    scale = 1 / math.sqrt(d)
    # contexts that end inside a page, at a page's edge and at the sequence's end, with queries
    # pointed at the first key, one in the middle, the last one, and at nothing in particular
    cases = [(N, 0), (N, 16_383), (N, N - 1), (N, None), (32_768, 32_767), (32_768, 0), (32_777, 17_000),
             (32_777, None)]
    for ctx, far in cases:
        pos = ctx - 1
        q = peaked_queries(cache, [pos], {} if far is None else {0: far}, seed=ctx + (far or 7))
        want = reference(cache, q.float(), pos).reshape(1, H * d)
        if far is not None:
            for h in range(H):
                assert (want.reshape(H, d)[h] - cache.values[far, h // (H // KV)]).abs().max() < 1e-3
        buf = torch.zeros(1, (H + 2 * KV) * d, dtype=dtype)
        buf[:, :H * d] = q.reshape(1, -1)
        for splits in (1, 8, 64):
            ws = (torch.full((H * splits * d,), float("nan"), device=DEV),
                  torch.full((H * splits * 2,), float("nan"), device=DEV)) if splits > 1 else None
            out = torch.zeros(1, H * d, dtype=dtype, device=DEV)
            ops().attn_decode(buf.to(DEV), cache.k, cache.v, cache.table_dev, None, 1,
                              torch.arange(2, dtype=torch.int32, device=DEV),
                              torch.tensor([ctx], dtype=torch.int32, device=DEV), out, H, KV, d, scale,
                              0, splits, ws, token_is_seq=True)
            torch.testing.assert_close(out.float().cpu(), want, **tolerance(dtype),
                                       msg=lambda m: f"ctx {ctx}, far {far}, {splits} cuts: {m}")


def work_rows(rows_total: int, per_item: int, paired: bool) -> torch.Tensor:
    n = -(-rows_total // per_item)
    if paired:
        rows = [(0, i, n - 1 - i if n - 1 - i > i else -1) for i in range((n + 1) // 2)]
    else:
        rows = [(0, i, -1) for i in reversed(range(n))]
    return torch.tensor(rows, dtype=torch.int32).reshape(-1, 3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("d", [128, 64])
def test_a_run_of_2048_queries_at_the_end_of_32k_keys(d, dtype):
    cache = cache_for(d, dtype)
    scale = 1 / math.sqrt(d)
    first = N - RUN
    positions = list(range(first, N))
    # rows pointed at: the first key, a key deep in the middle, the last key before the run, the
    # query's own key (first, a middle and the last row of the run), a key inside the run
    pointed = {0: 0, 1: 16_383, 2: first - 1, 3: first + 3, 700: 16_384, 1023: first + 1023,
               1024: 16_000, 2015: 32_767, 2046: first + 5, 2047: N - 1}
    q = peaked_queries(cache, positions, pointed, seed=d)
    want = reference(cache, q.float(), first)
    for r, key_pos in pointed.items():
        for h in range(H):
            assert (want[r, h] - cache.values[key_pos, h // (H // KV)]).abs().max() < 1e-3
    want = want.reshape(RUN, H * d)
    buf = torch.zeros(RUN, (H + 2 * KV) * d, dtype=dtype)
    buf[:, :H * d] = q.reshape(RUN, -1)
    buf = buf.to(DEV)
    cu = torch.tensor([0, RUN], dtype=torch.int32, device=DEV)
    ctx = torch.tensor([N], dtype=torch.int32, device=DEV)
    sizes = sorted({ops().prefill_rows_per_item(dtype, d, BS, tiles) for tiles in (1, 2)})
    assert sizes == ([64, 128] if dtype == torch.bfloat16 else [64])
    for per_item in sizes:
        for paired in (True, False):
            out = torch.zeros(RUN, H * d, dtype=dtype, device=DEV)
            ops().attn_prefill(buf, cache.k, cache.v, cache.table_dev, cu, ctx,
                               work_rows(RUN * (H // KV), per_item, paired).to(DEV), out, H, KV, d, scale, 0,
                               rows_per_item=per_item)
            torch.testing.assert_close(out.float().cpu(), want, **tolerance(dtype),
                                       msg=lambda m: f"items of {per_item} rows, paired {paired}: {m}")
