"""Each HIP kernel alone against a plain fp32 torch reference, at sizes other than the engine's
(odd widths, head sizes that are no power of two, group sizes 1/3/4/6, scattered pages)."""

from __future__ import annotations

import math
import random

import pytest
import torch

from tests.plain import llama as plain
from tests.plain import sampling as plain_sampling

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def ops():
    from kvforge_amd.kernels import ops as o
    return o


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(dtype):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(37, 48, generator=g).to(dtype)
    ids = torch.tensor([0, 36, 5, 5, 99, -1, 17], dtype=torch.int32)
    out = torch.full((7, 48), 7.0, device=DEV)
    ops().embed(ids.to(DEV), table.to(DEV), out)
    want = torch.zeros(7, 48)
    for i, t in enumerate(ids.tolist()):
        if 0 <= t < 37:
            want[i] = table[t].float()
    assert torch.equal(out.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [96, 100, 2048, 5000])
@pytest.mark.parametrize("add32", [False, True])
def test_rmsnorm_with_owed_sum(dtype, h, add32):
    """norm(x + add): without rows the sum is left in x; with rows x stays as it was.  The sum
    owed is in the output's type (a library product, half of a product cut in K) or in fp32."""
    g = torch.Generator().manual_seed(h + 1)
    x = torch.randn(7, h, generator=g) * 2
    add = torch.randn(7, h, generator=g).to(torch.float32 if add32 else dtype)
    w = (1 + 0.1 * torch.randn(h, generator=g)).to(dtype)
    total = x + add.float()
    xd = x.to(DEV)
    out = torch.empty(7, h, dtype=dtype, device=DEV)
    ops().rmsnorm(xd, w.to(DEV), 1e-5, out, None, add.to(DEV))
    torch.testing.assert_close(out.float().cpu(), plain.rms_norm(total, w.float(), 1e-5), **tol(dtype))
    torch.testing.assert_close(xd.cpu(), total, atol=1e-6, rtol=1e-6)
    rows = torch.tensor([6, 2, 2], dtype=torch.int32)
    xd = x.to(DEV)
    out = torch.empty(3, h, dtype=dtype, device=DEV)
    ops().rmsnorm(xd, None, 1e-5, out, rows.to(DEV), add.to(DEV))
    want = plain.rms_norm(total[rows.long()], torch.ones(h), 1e-5)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
    assert torch.equal(xd.cpu(), x)
    # the sum alone
    xd = x.to(DEV)
    ops().add_rows(xd, add.to(DEV))
    torch.testing.assert_close(xd.cpu(), total, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [96, 100, 2048, 3000, 5000])
@pytest.mark.parametrize("w32", [False, True])
def test_rmsnorm(dtype, h, w32):
    g = torch.Generator().manual_seed(h)
    x = torch.randn(9, h, generator=g) * 3
    w = (1 + 0.1 * torch.randn(h, generator=g))
    w = w if w32 else w.to(dtype)
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    out = torch.empty(4, h, dtype=dtype, device=DEV)
    ops().rmsnorm(x.to(DEV), w.to(DEV), 1e-5, out, rows.to(DEV))
    want = plain.rms_norm(x[rows.long()], w.float(), 1e-5)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
    # against the library routine
    lib = torch.nn.functional.rms_norm(x[rows.long()], (h,), w.float(), 1e-5)
    torch.testing.assert_close(out.float().cpu(), lib, **tol(dtype))
    out2 = torch.empty(9, h, dtype=dtype, device=DEV)
    ops().rmsnorm(x.to(DEV), w.to(DEV), 1e-6, out2)
    torch.testing.assert_close(out2.float().cpu(), plain.rms_norm(x, w.float(), 1e-6), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    g = torch.Generator().manual_seed(1)
    gu = (torch.randn(5, 2 * 176, generator=g) * 2).to(dtype)
    out = torch.empty(5, 176, dtype=dtype, device=DEV)
    ops().silu_mul(gu.to(DEV), out)
    want = torch.nn.functional.silu(gu[:, :176].float()) * gu[:, 176:].float()
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
    ops().silu_mul(gu.to(DEV), out, paired=True)       # gate at 2i, up at 2i + 1
    want = torch.nn.functional.silu(gu[:, 0::2].float()) * gu[:, 1::2].float()
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("ta", DTYPES)
@pytest.mark.parametrize("tw", DTYPES)
@pytest.mark.parametrize("mnk", [(1, 384, 96), (5, 37, 50), (70, 130, 96), (33, 256, 176),
                                 (130, 70, 257)])
def test_gemm_generic(ta, tw, mnk):
    m, n, k = mnk
    g = torch.Generator().manual_seed(m * n + k)
    a = torch.randn(m, k, generator=g).to(ta)
    w = (torch.randn(n, k, generator=g) * 0.1).to(tw)
    want = a.double() @ w.double().T
    # bf16 x bf16 with many rows goes to the library, whose product is rounded to bf16
    library = ops().is_library_product(a.to(DEV), w.to(DEV))
    assert library == (ta == tw == torch.bfloat16 and k % 8 == 0 and m > ops().SKINNY_MAX_M)
    t32 = tol(torch.bfloat16) if library else dict(atol=2e-5, rtol=2e-5)
    for out_dtype in DTYPES:
        out = torch.empty(m, n, dtype=out_dtype, device=DEV)
        ops().gemm(a.to(DEV), w.to(DEV), out)
        t = tol(out_dtype) if out_dtype == torch.bfloat16 else t32
        torch.testing.assert_close(out.double().cpu(), want, **t)
    res = torch.randn(m, n, generator=g)
    acc = res.clone().to(DEV)
    ops().gemm(a.to(DEV), w.to(DEV), acc, accumulate=True)
    torch.testing.assert_close(acc.double().cpu(), res.double() + want, **t32)
    # a view with a wider row stride
    wide = torch.zeros(m, k + 24, dtype=ta)
    wide[:, :k] = a
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    ops().gemm(wide.to(DEV)[:, :k], w.to(DEV), out)
    torch.testing.assert_close(out.double().cpu(), want, **t32)


@pytest.mark.parametrize("m", [1, 5, 16, 17, 33, 64, 100, 128, 200, 300])
@pytest.mark.parametrize("n,k", [(16, 40), (37, 96), (384, 176), (2048, 2048), (200, 8192), (3072, 64)])
def test_gemm_bf16_mfma(m, n, k):
    """bf16 x bf16 on the matrix cores: fp32 store, bf16 store and fp32 accumulate, with tails in
    M, N and K."""
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    want = a.double() @ w.double().T
    # the hand-written kernel keeps fp32 sums; the library's product is rounded to bf16 before
    # it is widened or added
    own = not ops().is_library_product(a.to(DEV), w.to(DEV))
    assert own == (m <= 16 or (m <= ops().SKINNY_MAX_M and k < 2 * n))
    t32 = dict(atol=1e-4, rtol=1e-4) if own else dict(atol=2e-2, rtol=2e-2)
    out = torch.empty(m, n, device=DEV)
    ops().gemm(a.to(DEV), w.to(DEV), out)
    torch.testing.assert_close(out.double().cpu(), want, **t32)
    outb = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops().gemm(a.to(DEV), w.to(DEV), outb)
    torch.testing.assert_close(outb.double().cpu(), want, atol=2e-2, rtol=2e-2)
    res = torch.randn(m, n, generator=g)
    acc = res.clone().to(DEV)
    ops().gemm(a.to(DEV), w.to(DEV), acc, accumulate=True)
    torch.testing.assert_close(acc.double().cpu(), res.double() + want, **t32)
    # a strided view of a wider buffer as left operand
    wide = torch.zeros(m, k + 16, dtype=torch.bfloat16)
    wide[:, 8:k + 8] = a
    out2 = torch.empty(m, n, device=DEV)
    ops().gemm(wide.to(DEV)[:, 8:k + 8], w.to(DEV), out2)
    torch.testing.assert_close(out2.double().cpu(), want, **t32)


@pytest.mark.parametrize("m", [20, 32, 50, 64])
@pytest.mark.parametrize("n,k", [(16400, 256), (5120, 96), (4104, 512), (40000, 64)])
def test_gemm_bf16_rows_in_two_to_four_tiles_over_many_columns(m, n, k, monkeypatch):
    """17 to 64 rows over weights with so many columns that a wave takes two or four groups of
    16 of them (the choice follows the columns and the chip): every store, with columns that end
    inside a group."""
    monkeypatch.setattr(ops(), "SKINNY_MAX_M", 64)
    monkeypatch.setattr(ops(), "is_library_product", lambda a, w: False)
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    plain_w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16).to(DEV)
    want = a.double().cpu() @ plain_w.double().cpu().T
    res = torch.randn(m, n, generator=g)
    for w in (plain_w, ops().StreamedWeight(plain_w)):
        out, acc = torch.empty(m, n, device=DEV), res.clone().to(DEV)
        outb = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        gate = torch.empty(m, n // 2, dtype=torch.bfloat16, device=DEV)
        ops().gemm(a, w, out)
        ops().gemm(a, w, outb)
        ops().gemm(a, w, acc, accumulate=True)
        ops().gemm_fused(a, w, gate, silu_pairs=True)
        torch.testing.assert_close(out.double().cpu(), want, atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(outb.double().cpu(), want, atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(acc.double().cpu(), res.double() + want, atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(gate.double().cpu(), torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2],
                                   atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("m", [33, 64, 100, 257])
@pytest.mark.parametrize("n,k", [(37, 96), (384, 176), (2048, 2048), (200, 8192), (3072, 64)])
def test_gemm_of_many_rows_through_the_library_entry_point(m, n, k):
    """Many bf16 rows go to hipBLASLt through the engine's own entry point: fp32 sums stored as
    fp32 (plain or added to what is there) or rounded once to bf16, strided operands, tails in
    every size."""
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16).to(DEV)
    want = a.double() @ w.double().cpu().T
    wide = torch.zeros(m, k + 16, dtype=torch.bfloat16)
    wide[:, 8:k + 8] = a
    av = wide.to(DEV)[:, 8:k + 8]
    assert ops().is_library_product(av, w)
    out = torch.full((m, n + 4), 9.0, device=DEV)
    ops()._library_product(av, w, out[:, :n], False, m, n, k, av.stride(0), out.stride(0))
    torch.testing.assert_close(out[:, :n].double().cpu(), want, atol=1e-4, rtol=1e-4)
    assert bool((out[:, n:] == 9.0).all())                      # nothing written past the columns
    res = torch.randn(m, n, generator=g)
    acc = res.clone().to(DEV)
    ops().gemm(av, w, acc, accumulate=True)
    torch.testing.assert_close(acc.double().cpu(), res.double() + want, atol=1e-4, rtol=1e-4)
    outb = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops().gemm(av, w, outb)
    torch.testing.assert_close(outb.double().cpu(), want, atol=2e-2, rtol=2e-2)
    # a sum still owed to the stream is added by the engine's own kernel on the way
    owed = torch.randn(m, n, generator=g).to(torch.bfloat16)
    acc = res.clone().to(DEV)
    ops().gemm(av, w, acc, accumulate=True, owed=owed.to(DEV))
    torch.testing.assert_close(acc.double().cpu(), res.double() + owed.double() + want, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("m", [1, 3, 8, 16])
@pytest.mark.parametrize("n,k", [(1000, 256), (128256, 128), (8200, 2048), (37, 64)])
@pytest.mark.parametrize("tiled", [True, False])
def test_gemm_pick_is_head_argmax_advance_and_embedding(m, n, k, tiled):
    """The greedy tail of a decode step in one kernel against its parts done plainly: the
    normalised rows times the head's matrix, the largest logit's column per row, the sequences'
    next inputs moved on (padding sequences left alone), the ring row of the step, the step
    counter, and the tokens' embedding rows as the next residual stream.  Twice in a row over
    the same scratch."""
    g = torch.Generator().manual_seed(m * 7 + k)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    embed = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
    sw = ops().StreamedWeight(w.to(DEV)) if tiled else w.to(DEV)
    work = ops().pick_workspace(16, n, DEV)
    ring = torch.full((4, 20), -1, dtype=torch.int32, device=DEV)
    counter = torch.zeros(1, dtype=torch.int32, device=DEV)
    ctx = torch.tensor([5 + i if i % 4 != 3 else 0 for i in range(m)], dtype=torch.int32)  # some padding
    for call in range(2):
        x = torch.randn(m, k + 8, generator=g).to(torch.bfloat16)[:, :k]      # a row stride wider than K
        logits = x.double() @ w.double().T
        residual = torch.full((m, k), 3.0, device=DEV)
        tokens = torch.full((m,), -5, dtype=torch.int32, device=DEV)
        token_ids = torch.full((m,), 7, dtype=torch.int32, device=DEV)
        positions = torch.arange(10, 10 + m, dtype=torch.int32, device=DEV)
        ctx_dev = ctx.clone().to(DEV)
        wide = torch.zeros(m, k + 8, dtype=torch.bfloat16, device=DEV)
        wide[:, :k] = x.to(DEV)
        ops().gemm_pick(wide[:, :k], sw, residual, tokens, token_ids, positions, ctx_dev, ring, counter,
                        embed, work)
        got = tokens.cpu()
        top2 = logits.topk(2, dim=-1).values
        for r in range(m):
            if float(top2[r, 0] - top2[r, 1]) > 1e-4:          # fp32 sums of bf16 products: near exact
                assert int(got[r]) == int(logits[r].argmax()), (call, r)
            assert float(logits[r].max() - logits[r, int(got[r])]) <= 1e-4
        live = ctx > 0
        assert torch.equal(token_ids.cpu()[live], got[live]) and (token_ids.cpu()[~live] == 7).all()
        assert torch.equal(positions.cpu(), torch.arange(10, 10 + m, dtype=torch.int32) + live.int())
        assert torch.equal(ctx_dev.cpu(), ctx + live.int())
        assert int(counter) == call + 1 and torch.equal(ring[call, :m].cpu(), got)
        assert (ring[call + 1:] == -1).all() and int(work[2].abs().sum()) == 0
        assert torch.equal(residual.cpu(), embed.float().cpu()[got.long()])


def test_gemm_pick_takes_the_lowest_of_equal_columns():
    """Rows of zeros give equal logits everywhere: column 0 wins in every row, through every
    workgroup's partial result and the last one's merge."""
    n, k, m = 50000, 64, 8
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(DEV)
    sw = ops().StreamedWeight(w)
    a = torch.zeros(m, k, dtype=torch.bfloat16, device=DEV)
    a[3, 5] = 1.0                                    # one row with a real best column
    tokens = torch.full((m,), -1, dtype=torch.int32, device=DEV)
    i32 = lambda v: torch.full((m,), v, dtype=torch.int32, device=DEV)
    ops().gemm_pick(a, sw, torch.zeros(m, k, device=DEV), tokens, i32(0), i32(0), i32(1),
                    torch.zeros(2, m, dtype=torch.int32, device=DEV),
                    torch.zeros(1, dtype=torch.int32, device=DEV), w, ops().pick_workspace(16, n, DEV))
    want = [0] * m
    want[3] = int(w[:, 5].float().argmax())
    assert tokens.tolist() == want


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n,k", [(352, 96), (40, 2048), (100, 40), (2048, 136), (16, 32)])
def test_gemm_over_tiled_weights_gives_the_same_bits(m, n, k):
    """A weight kept in tiles of 16 x 32 (what the parts stream for few rows) gives bit for bit
    what the row-major matrix gives, in every form of the product: tails in N and K are zero
    padding inside the tiles; beyond the kernel's rows the row-major copy goes to the library."""
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    x = (torch.randn(m, k, generator=g) * 2).to(DEV)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16).to(DEV)
    sw = ops().StreamedWeight(w)
    assert tuple(sw.tiles.shape) == (-(-n // 16), -(-k // 32), 64, 8) and sw.shape == w.shape
    # tile (1, 0) or (0, 0), position 16*c + r: row 16g + r, columns 8c..8c+7
    gi = 1 if n > 16 else 0
    r, c = min(3, n - 16 * gi - 1), 2 if k >= 24 else 0
    assert torch.equal(sw.tiles[gi, 0, 16 * c + r], w[16 * gi + r, 8 * c:8 * c + 8])
    for dt in (torch.float32, torch.bfloat16):
        o1, o2 = torch.empty(m, n, dtype=dt, device=DEV), torch.empty(m, n, dtype=dt, device=DEV)
        ops().gemm(a, w, o1)
        ops().gemm(a, sw, o2)
        assert torch.equal(o1, o2)
    res = torch.randn(m, n, generator=g).to(DEV)
    r1, r2 = res.clone(), res.clone()
    ops().gemm(a, w, r1, accumulate=True)
    ops().gemm(a, sw, r2, accumulate=True)
    assert torch.equal(r1, r2)
    if n % 4 == 0:
        g1 = torch.empty(m, n // 2, dtype=torch.bfloat16, device=DEV)
        g2 = torch.empty_like(g1)
        ops().gemm_fused(x, w, g1, rms_eps=1e-5, silu_pairs=True)
        ops().gemm_fused(x, sw, g2, rms_eps=1e-5, silu_pairs=True)
        assert torch.equal(g1, g2)
    # many rows: the library reads the row-major copy
    big = torch.randn(40, k, generator=g).to(torch.bfloat16).to(DEV)
    o1, o2 = torch.empty(40, n, device=DEV), torch.empty(40, n, device=DEV)
    ops().gemm(big, w, o1)
    ops().gemm(big, sw, o2)
    assert torch.equal(o1, o2)


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("n,k", [(2048, 8192), (100, 4096), (1040, 4104)])
@pytest.mark.parametrize("tiled", [False, True])
def test_gemm_cut_in_two_halves_of_k(m, n, k, tiled):
    """out += a @ w.T with the second half of K left in half_out (bf16: rounded once, as a stored
    product is), and a sum owed to out (bf16 too) added on the way: out + half_out is the whole
    sum; every value is an fp32 sum in a fixed order, so a second call gives the same bits."""
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16).to(DEV)
    w = ops().StreamedWeight(w) if tiled else w
    res = torch.randn(m, n, generator=g)
    owed = torch.randn(m, n, generator=g).to(torch.bfloat16)
    assert ops().k_halves_pay(a.to(DEV), w)
    cut = (-(-k // 32) + 1) // 2 * 32                    # the first half takes the odd k-step
    first = a[:, :cut].double() @ ops().plain_of(w).cpu()[:, :cut].double().T
    second = a[:, cut:].double() @ ops().plain_of(w).cpu()[:, cut:].double().T
    outs = []
    for _ in range(2):
        out, half = res.clone().to(DEV), torch.full((m, n), 7.0, device=DEV, dtype=torch.bfloat16)
        ops().gemm(a.to(DEV), w, out, accumulate=True, owed=owed.to(DEV), half_out=half)
        torch.testing.assert_close(out.double().cpu(), res.double() + owed.double() + first, atol=1e-4, rtol=1e-4)
        # the half is the 32-bit sum rounded to bfloat16 once: within half a unit of its last place
        torch.testing.assert_close(half.double().cpu(), second, atol=1e-4, rtol=2.0 ** -8)
        outs.append((out, half))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    # the sum owed alone, without the cut
    out = res.clone().to(DEV)
    ops().gemm(a.to(DEV), w, out, accumulate=True, owed=owed.to(DEV))
    torch.testing.assert_close(out.double().cpu(), res.double() + owed.double() + first + second,
                               atol=1e-4, rtol=1e-4)
    with pytest.raises(ops().KernelError):
        ops().gemm(a.to(DEV), w, torch.empty(m, n, device=DEV), half_out=torch.empty(m, n, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(ops().KernelError):               # a shallow weight is not cut
        ops().gemm(a.to(DEV)[:, :64].contiguous(), ops().plain_of(w)[:, :64].contiguous(), res.clone().to(DEV),
                   accumulate=True, half_out=torch.empty(m, n, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(ops().KernelError):               # sums that ride along are bfloat16
        ops().gemm(a.to(DEV), w, res.clone().to(DEV), accumulate=True, owed=owed.float().to(DEV))


@pytest.mark.parametrize("m", [1, 8, 16, 20, 33, 50, 64])
@pytest.mark.parametrize("n,k", [(352, 96), (512, 2048), (48, 40)])
def test_gemm_fused_norm_and_gate(m, n, k):
    """The MFMA kernel with the RMS norm folded into its left operand (fp32 rows, factor
    rsqrt(mean(x^2) + eps) per row) and with the SwiGLU gate folded into its store."""
    g = torch.Generator().manual_seed(m * 7 + n + k)
    x = torch.randn(m, k, generator=g) * 3
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    eps = 1e-5
    xn = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    want = xn.double() @ w.double().T
    out = torch.empty(m, n, device=DEV)
    gate = torch.empty(m, n // 2, dtype=torch.bfloat16, device=DEV)
    if m <= ops().FUSED_NORM_MAX_M:
        ops().gemm_fused(x.to(DEV), w.to(DEV), out, rms_eps=eps)
        torch.testing.assert_close(out.double().cpu(), want, atol=2e-2, rtol=2e-2)   # rows are rounded to bf16
        res = torch.randn(m, n, generator=g)
        acc = res.clone().to(DEV)
        ops().gemm_fused(x.to(DEV), w.to(DEV), acc, rms_eps=eps, accumulate=True)
        torch.testing.assert_close(acc.double().cpu(), res.double() + want, atol=2e-2, rtol=2e-2)
        ops().gemm_fused(x.to(DEV), w.to(DEV), gate, rms_eps=eps, silu_pairs=True)
        want_gate = torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2]
        torch.testing.assert_close(gate.double().cpu(), want_gate, atol=2e-2, rtol=3e-2)
    else:
        assert not ops().bf16_kernel_takes(x.to(DEV), w.to(DEV), rms=True)
        with pytest.raises(ops().KernelError):
            ops().gemm_fused(x.to(DEV), w.to(DEV), out, rms_eps=eps)
    xb = xn.to(torch.bfloat16)
    if m <= ops().FUSED_EPILOGUE_MAX_M:
        ops().gemm_fused(xb.to(DEV), w.to(DEV), gate, silu_pairs=True)
        wantb = xb.double() @ w.double().T
        torch.testing.assert_close(gate.double().cpu(),
                                   torch.nn.functional.silu(wantb[:, 0::2]) * wantb[:, 1::2],
                                   atol=1e-2, rtol=1e-2)


# the norm rides in the projection only for one tile of rows
@pytest.mark.parametrize("m,rms", [(m, r) for m in (1, 9, 16, 23, 40, 64) for r in (False, True) if m <= 16 or not r])
@pytest.mark.parametrize("H,KV,d,rot,bs", [(4, 2, 16, 16, 4), (3, 1, 32, 32, 8), (2, 2, 48, 32, 16),
                                            (32, 8, 64, 64, 16), (40, 8, 128, 128, 16)])
def test_gemm_qkv_rope_equals_the_three_steps(m, H, KV, d, rot, bs, rms):
    """The fused projection + rotary + cache write against projection (MFMA kernel), then the
    rotary/cache-write kernel: same q, same pages."""
    k = 96
    g = torch.Generator().manual_seed(m + d)
    x = torch.randn(m, k, generator=g)
    w = (torch.randn((H + 2 * KV) * d, k, generator=g) / 6).to(torch.bfloat16).to(DEV)
    positions = torch.randint(0, min(60, 12 * bs), (m,), generator=g, dtype=torch.int32)
    positions[0] = 5
    seq_of = torch.randint(0, 3, (m,), generator=g, dtype=torch.int32)
    seq_of[0] = 0
    nb = 40
    table = torch.randperm(nb, generator=g)[:3 * 10].reshape(3, 10).to(torch.int32)
    table[1, 2] = -1                                   # a page that was given back
    inv_freq = plain.rope_inv_freq(rot, 10000.0)
    cos_full, sin_full = plain.rope_cos_sin(torch.arange(64), inv_freq)
    cos_t, sin_t = cos_full[:, : rot // 2].contiguous().to(DEV), sin_full[:, : rot // 2].contiguous().to(DEV)
    eps = 1e-5
    assert not rms or m <= ops().FUSED_NORM_MAX_M
    if rms:
        a = x.to(DEV)
        normed = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
        ops().rmsnorm(a, None, eps, normed)
        ref_in = normed
    else:
        a = x.to(torch.bfloat16).to(DEV)
        ref_in = a
    qkv = torch.empty(m, (H + 2 * KV) * d, dtype=torch.bfloat16, device=DEV)
    ops().gemm(ref_in, w, qkv)
    kp_ref = torch.zeros(nb, KV, bs, d, dtype=torch.bfloat16, device=DEV)
    vp_ref = torch.zeros(nb, KV, d, bs, dtype=torch.bfloat16, device=DEV)
    ops().rope_kvwrite(qkv, positions.to(DEV), seq_of.to(DEV), cos_t, sin_t, table.to(DEV), kp_ref,
                       vp_ref, H, KV, d)
    kp, vp = torch.zeros_like(kp_ref), torch.zeros_like(vp_ref)
    q = torch.empty(m, H * d, dtype=torch.bfloat16, device=DEV)
    ops().gemm_qkv_rope(a, w, q, positions.to(DEV), seq_of.to(DEV), cos_t, sin_t, table.to(DEV), kp,
                        vp, H, KV, d, rms_eps=eps if rms else None)
    # the same over the weight in tiles: the same bits
    kp_t, vp_t, q_t = torch.zeros_like(kp_ref), torch.zeros_like(vp_ref), torch.empty_like(q)
    ops().gemm_qkv_rope(a, ops().StreamedWeight(w), q_t, positions.to(DEV), seq_of.to(DEV), cos_t, sin_t,
                        table.to(DEV), kp_t, vp_t, H, KV, d, rms_eps=eps if rms else None)
    assert torch.equal(q_t, q)
    # the fused kernel rotates fp32 accumulators, the reference rounds the projection to bf16
    # first; with fp32 rows the rounding of the normalised input differs as well
    t = dict(atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(q.float().cpu(), qkv[:, :H * d].float().cpu(), **t)
    # two tokens of one sequence at one position write the same slot: compare slots hit once
    slots = {}
    for i in range(m):
        slots.setdefault((int(seq_of[i]), int(positions[i])), []).append(i)
    once = torch.zeros(nb, bs, dtype=torch.bool)
    for (sq, pos), toks in slots.items():
        page = int(table[sq, pos // bs]) if pos // bs < table.shape[1] else -1   # beyond the table: skipped
        if len(toks) == 1 and page >= 0:
            once[page, pos % bs] = True
    sel = once[:, None, :, None].expand(nb, KV, bs, d)
    torch.testing.assert_close(kp.float().cpu()[sel], kp_ref.float().cpu()[sel], **t)
    sel_v = once[:, None, None, :].expand(nb, KV, d, bs)
    torch.testing.assert_close(vp.float().cpu()[sel_v], vp_ref.float().cpu()[sel_v], **t)
    assert once.any()
    untouched = (kp_ref.float().cpu().abs().sum((1, 3)) == 0)
    assert (kp.float().cpu().abs().sum((1, 3))[untouched] == 0).all()
    if rms:
        # a sum still owed to the rows rides in the loads: the same bits as rows summed before,
        # and the rows themselves stay as they were
        a1, a2 = torch.randn(m, k, generator=g), torch.randn(m, k, generator=g).to(torch.bfloat16)
        got = []
        for rows, owed in (((a1 + a2.float()).to(DEV), None), (a1.to(DEV), a2.to(DEV))):
            kp2, vp2, q2 = torch.zeros_like(kp_ref), torch.zeros_like(vp_ref), torch.empty_like(q)
            ops().gemm_qkv_rope(rows, w, q2, positions.to(DEV), seq_of.to(DEV), cos_t, sin_t, table.to(DEV),
                                kp2, vp2, H, KV, d, rms_eps=eps, a_owed=owed)
            got.append((q2, kp2.cpu()[sel], vp2.cpu()[sel_v]))
            assert torch.equal(rows.cpu(), a1 if owed is not None else a1 + a2.float())
        assert all(torch.equal(x1, x2) for x1, x2 in zip(*got))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 4), (3, 1, 40, 8), (32, 8, 64, 16)])
@pytest.mark.parametrize("m", [1, 7, 48])
def test_cache_write_without_rotation(dtype, H, KV, d, bs, m):
    """Without rotary tables q and k stay as they are and only the cache is written, at any
    position the block table covers: there is no table whose length could bound it.  Both the
    kernel of its own and, in bf16, the projection that carries the write."""
    g = torch.Generator().manual_seed(m + d)
    width = (H + 2 * KV) * d
    table = torch.randperm(300, generator=g)[:2 * 140].reshape(2, 140).to(torch.int32)
    positions = (torch.randperm(140 * bs, generator=g)[:m]).to(torch.int32)        # far beyond any prompt here
    seq_of = torch.randint(0, 2, (m,), generator=g, dtype=torch.int32)
    args = (positions.to(DEV), seq_of.to(DEV), None, None, table.to(DEV))

    def expect(qkv):
        kp = torch.zeros(300, KV, bs, d, dtype=dtype)
        vp = torch.zeros(300, KV, d, bs, dtype=dtype)
        for i in range(m):
            page, off = int(table[seq_of[i], positions[i] // bs]), int(positions[i]) % bs
            kp[page, :, off] = qkv[i, H * d:(H + KV) * d].view(KV, d)
            vp[page, :, :, off] = qkv[i, (H + KV) * d:].view(KV, d)
        return kp, vp

    qkv = torch.randn(m, width, generator=g).to(dtype)
    on_dev = qkv.to(DEV)
    kp = torch.zeros(300, KV, bs, d, dtype=dtype, device=DEV)
    vp = torch.zeros(300, KV, d, bs, dtype=dtype, device=DEV)
    ops().rope_kvwrite(on_dev, *args, kp, vp, H, KV, d)
    want_k, want_v = expect(qkv)
    assert torch.equal(on_dev.cpu(), qkv) and torch.equal(kp.cpu(), want_k) and torch.equal(vp.cpu(), want_v)
    if dtype == torch.bfloat16 and d % 4 == 0:
        k = 96
        a = torch.randn(m, k, generator=g).to(dtype).to(DEV)
        w = (torch.randn(width, k, generator=g) / 6).to(dtype).to(DEV)
        proj = torch.empty(m, width, dtype=dtype, device=DEV)
        ops().gemm(a, w, proj)
        kp2, vp2, q2 = torch.zeros_like(kp), torch.zeros_like(vp), torch.empty(m, H * d, dtype=dtype, device=DEV)
        ops().gemm_qkv_rope(a, w, q2, *args, kp2, vp2, H, KV, d)
        want_k, want_v = expect(proj.cpu())
        # the same kernel computes both up to SKINNY_MAX_M rows: the same bits; beyond, the plain
        # product is the library's, with another order of sums
        t = dict(atol=0, rtol=0) if m <= ops().SKINNY_MAX_M else dict(atol=2e-2, rtol=2e-2)
        for got, want in ((q2, proj[:, :H * d]), (kp2, want_k), (vp2, want_v)):
            torch.testing.assert_close(got.float().cpu(), want.float().cpu(), **t)


@pytest.mark.parametrize("m", [5, 40])
def test_gemm_rows_off_a_16_byte_boundary_take_the_plain_kernel(m):
    """Rows that start two bytes past a 16-byte boundary cannot be read 16 bytes at a time: neither
    the matrix-core kernel nor the library takes them, the fused forms refuse them, and the plain
    kernel gives the product."""
    g = torch.Generator().manual_seed(m)
    wide = torch.randn(m, 104, generator=g).to(torch.bfloat16).to(DEV)
    a = wide[:, 1:97]
    w = (torch.randn(48, 96, generator=g) / 10).to(torch.bfloat16).to(DEV)
    assert a.data_ptr() % 16 == 2 and a.stride(0) % 8 == 0
    assert not ops().bf16_kernel_takes(a, w) and not ops().is_library_product(a, w)
    out = torch.empty(m, 48, device=DEV)
    ops().gemm(a, w, out)
    torch.testing.assert_close(out.double().cpu(), a.double().cpu() @ w.double().cpu().T, atol=2e-5, rtol=2e-5)
    with pytest.raises(ops().KernelError):
        ops().gemm_fused(a, w, torch.empty(m, 24, dtype=torch.bfloat16, device=DEV), silu_pairs=True)


def test_gemm_bf16_rows_do_not_depend_on_neighbours():
    g = torch.Generator().manual_seed(9)
    a = torch.randn(16, 2048, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(512, 2048, generator=g) / 45).to(torch.bfloat16).to(DEV)
    full = torch.empty(16, 512, device=DEV)
    ops().gemm(a, w, full)
    one = torch.empty(1, 512, device=DEV)
    ops().gemm(a[7:8], w, one)
    assert torch.equal(one[0], full[7])


def test_gemm_rows_do_not_depend_on_batch():
    """fp32 products are summed in a fixed order: a row alone has the bits of the row in any
    batch that the same kernel takes (up to 32 rows: the weight-streaming one, whatever the
    number of rows per workgroup; more: the tiled one), and the two kernels agree to rounding."""
    g = torch.Generator().manual_seed(3)
    a = torch.randn(77, 176, generator=g).to(DEV)
    w = torch.randn(300, 176, generator=g).to(DEV)

    def product(rows):
        out = torch.empty(rows.shape[0], 300, device=DEV)
        ops().gemm(rows, w, out)
        return out

    full = product(a)
    alone = product(a[40:41])
    for lo, hi in ((40, 42), (38, 42), (35, 43), (30, 46), (20, 52)):     # 2, 4, 8, 16, 32 rows
        assert torch.equal(product(a[lo:hi])[40 - lo], alone[0]), (lo, hi)
    assert torch.equal(product(a[8:77])[32], full[40])                      # 69 rows and 77
    torch.testing.assert_close(alone[0], full[40], atol=2e-5, rtol=1e-5)
    want = a.double() @ w.double().T
    torch.testing.assert_close(full.double(), want, atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(alone[0].double(), want[40], atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("m", [1, 3, 8, 13, 32])
@pytest.mark.parametrize("tw", DTYPES)
def test_gemm_generic_few_rows_over_long_and_uneven_k(m, tw):
    """The weight-streaming fp32 kernel: K beyond one staged chunk and not a multiple of the 256
    elements a wave reads at a time, N that ends inside a workgroup's columns, accumulation
    into the stream, and a row stride wider than K."""
    g = torch.Generator().manual_seed(m)
    n, k = 70, 2348
    a = torch.randn(m, k + 8, generator=g).to(DEV)[:, :k]
    w = (torch.randn(n, k, generator=g) * 0.05).to(tw).to(DEV)
    want = a.double() @ w.double().T
    out = torch.full((m, n), 7.0, device=DEV)
    ops().gemm(a, w, out)
    torch.testing.assert_close(out.double(), want, atol=3e-5, rtol=1e-5)
    acc = torch.ones(m, n, device=DEV)
    ops().gemm(a, w, acc, accumulate=True)
    torch.testing.assert_close(acc.double(), want + 1.0, atol=3e-5, rtol=1e-5)


# bf16 x bf16 with many rows is the library's or the bf16 kernel's product: not among the pairs
@pytest.mark.parametrize("ta,tw", [(a, w) for a in DTYPES for w in DTYPES if torch.float32 in (a, w)])
@pytest.mark.parametrize("mnk", [(33, 130, 96), (200, 70, 260), (129, 257, 2052), (300, 1000, 64),
                                 (128, 128, 32), (260, 4100, 36)])
def test_gemm_generic_many_rows_on_the_matrix_cores(ta, tw, mnk):
    """More than 32 rows with rows of K that start on 16 bytes go to v_mfma_f32_32x32x2_f32:
    32-bit multiply and add, so 32-bit operands that bfloat16 cannot hold give a 64-bit product's
    result to 32-bit rounding; tails in M, N and K, tiles of 128 and of 64 columns, both ways of
    storing and adding into the stream.  A row's result does not depend on the rows around it, and
    the kernel of the vector ALUs, kept for this comparison, agrees to rounding."""
    m, n, k = mnk
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(ta).to(DEV)
    w = (torch.randn(n, k, generator=g) * 0.1).to(tw).to(DEV)
    if ta == torch.float32:
        assert not torch.equal(a.bfloat16().float(), a)
    want = a.double() @ w.double().T
    out = torch.full((m, n), 7.0, device=DEV)
    ops().gemm(a, w, out)
    torch.testing.assert_close(out.double(), want, atol=2e-5, rtol=1e-5)
    before = ops().gemm_generic_vector_alus_only(True)
    try:
        fma = torch.full((m, n), 7.0, device=DEV)
        ops().gemm(a, w, fma)
    finally:
        ops().gemm_generic_vector_alus_only(before)
    torch.testing.assert_close(fma.double(), want, atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(out, fma, atol=2e-5, rtol=1e-5)
    if k > 64:
        assert not torch.equal(out, fma)        # another order of summation: it is the other kernel
    acc = torch.ones(m, n, device=DEV)
    ops().gemm(a, w, acc, accumulate=True)
    torch.testing.assert_close(acc.double(), want + 1.0, atol=2e-5, rtol=1e-5)
    half = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops().gemm(a, w, half)
    torch.testing.assert_close(half.double(), want, atol=2e-2, rtol=2e-2)
    # the same rows among fewer: the same bits
    lo = 0 if m < 80 else m // 3
    hi = min(m, lo + 40)
    part = torch.empty(hi - lo, n, device=DEV)
    ops().gemm(a[lo:hi], w, part)
    assert torch.equal(part, out[lo:hi])
    # a view with a wider row stride
    wide = torch.zeros(m, k + 24, dtype=ta, device=DEV)
    wide[:, :k] = a
    again = torch.empty(m, n, device=DEV)
    ops().gemm(wide[:, :k], w, again)
    assert torch.equal(again, out)


@pytest.mark.parametrize("m", [1, 4, 8, 16, 32])
@pytest.mark.parametrize("n,k", [(6150, 516), (16390, 260)])
@pytest.mark.parametrize("tw", DTYPES)
def test_gemm_generic_few_rows_over_wide_weights(m, n, k, tw):
    """The weight-streaming fp32 kernel changes its shape with the width of W: two columns per
    wave from 6,144 columns on, four from 16,384 (the widths of gate/up and of the vocabulary).
    32-bit weights that bfloat16 cannot hold, N that ends inside a wave's columns, against a
    64-bit product; and the sums are the same whichever shape took them (a column of the wide
    product equals the column computed over a narrow slice of W)."""
    g = torch.Generator().manual_seed(n + m)
    a = torch.randn(m, k, generator=g).to(DEV)
    w = (torch.randn(n, k, generator=g) * 0.05).to(tw).to(DEV)
    if tw == torch.float32:
        assert not torch.equal(w.bfloat16().float(), w)
    want = a.double() @ w.double().T
    out = torch.full((m, n), 7.0, device=DEV)
    ops().gemm(a, w, out)
    torch.testing.assert_close(out.double(), want, atol=2e-5, rtol=1e-5)
    acc = torch.ones(m, n, device=DEV)
    ops().gemm(a, w, acc, accumulate=True)
    torch.testing.assert_close(acc.double(), want + 1.0, atol=2e-5, rtol=1e-5)
    narrow = torch.empty(m, 100, device=DEV)
    ops().gemm(a, w[n - 100:].contiguous(), narrow)
    assert torch.equal(narrow, out[:, n - 100:])


class Paged:
    """Scatters contiguous per-sequence K/V into shuffled pages: K ``[nb, KV, bs, d]``, V
    transposed ``[nb, KV, d, bs]``."""

    def __init__(self, seq_lens, KV, d, bs, dtype, seed=0, spare=7, shape_keys=None):
        rng = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        need = sum(-(-n // bs) for n in seq_lens)
        self.nb = need + spare
        ids = list(range(self.nb))
        rng.shuffle(ids)
        self.k = torch.randn(self.nb, KV, bs, d, generator=g).to(dtype)  # junk everywhere
        self.v = torch.randn(self.nb, KV, d, bs, generator=g).to(dtype)
        width = max(-(-n // bs) for n in seq_lens) + 2
        self.table = torch.full((len(seq_lens), width), -1, dtype=torch.int32)
        self.keys, self.values = [], []
        for s, n in enumerate(seq_lens):
            kk = torch.randn(n, KV, d, generator=g)
            if shape_keys is not None:
                kk = shape_keys(kk)
            kk = kk.to(dtype)
            vv = torch.randn(n, KV, d, generator=g).to(dtype)
            for b in range(-(-n // bs)):
                page = ids.pop()
                self.table[s, b] = page
                seg = slice(b * bs, min(n, (b + 1) * bs))
                cnt = seg.stop - seg.start
                self.k[page, :, :cnt] = kk[seg].transpose(0, 1)
                self.v[page, :, :, :cnt] = vv[seg].permute(1, 2, 0)
            self.keys.append(kk)
            self.values.append(vv)


def attn_reference(paged, q, seq_lens, q_lens, scale, window):
    outs, off = [], 0
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        outs.append(plain.causal_attention(q[off:off + ql].float(), paged.keys[s].float(),
                                           paged.values[s].float(), scale, n - ql, window))
        off += ql
    return torch.cat(outs)


def prefill_work(q_lens, G, dtype=torch.float32, d=16, bs=4, row_tiles=1):
    """Rows (sequence, item, item or -1): an early item paired with a late one, as the engine
    does; the odd one out of three is left alone."""
    rows = ops().prefill_rows_per_item(dtype, d, bs, row_tiles)
    work = []
    for s, ql in enumerate(q_lens):
        n = -(-ql * G // rows)
        for t in range((n + 1) // 2):
            work.append((s, t, n - 1 - t if n - 1 - t > t else -1))
    return torch.tensor(work, dtype=torch.int32).reshape(-1, 3)


# the (context, query) cases of the reference's tests/test_paged_attention.py:60-66 and more
ATTN_CASES = [
    ([9, 16], [9, 16]),
    ([12, 30, 5], [4, 7, 5]),
    ([17, 3, 25], [2, 3, 5]),
    ([200, 131], [67, 131]),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seq_lens,q_lens", ATTN_CASES)
@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 4), (3, 1, 32, 8), (6, 1, 48, 16),
                                        (4, 4, 80, 16), (8, 2, 128, 16), (2, 1, 256, 32),
                                        (32, 8, 64, 16), (20, 1, 16, 8)])
@pytest.mark.parametrize("window", [0, 11])
def test_attn_prefill(dtype, seq_lens, q_lens, H, KV, d, bs, window):
    """Items of one row tile per wave and, where the kernel has them, of two."""
    paged = Paged(seq_lens, KV, d, bs, dtype, seed=len(seq_lens) + d)
    g = torch.Generator().manual_seed(d)
    n = sum(q_lens)
    # q lives inside a wider qkv-like buffer
    buf = torch.randn(n, (H + 2 * KV) * d, generator=g).to(dtype)
    q = buf[:, :H * d].reshape(n, H, d)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    ctx = torch.tensor(seq_lens, dtype=torch.int32)
    out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
    scale = 1 / math.sqrt(d)
    want = attn_reference(paged, q, seq_lens, q_lens, scale, window or None).reshape(n, H * d)
    sizes = sorted({ops().prefill_rows_per_item(dtype, d, bs, tiles) for tiles in (1, 2)})
    assert sizes == ([64, 128] if dtype == torch.bfloat16 and bs % 8 == 0 and d <= 128 else
                     [64])          # the 32-bit kernel's items: four waves of 16 rows
    for row_tiles, per_item in enumerate(sizes, 1):
        out.zero_()
        ops().attn_prefill(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV),
                           cu.to(DEV), ctx.to(DEV), prefill_work(q_lens, H // KV, dtype, d, bs, row_tiles).to(DEV),
                           out, H, KV, d, scale, window, rows_per_item=per_item)
        torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


def test_prefill_kernel_says_how_many_workgroups_a_compute_unit_holds():
    """What the planner of query runs weighs rows per item against: asked of the runtime for the
    kernel that would run, at least one, never more with two row tiles than with one; sizes the
    matrix-core kernel does not take answer through the 32-bit kernel's constant."""
    o = ops()
    for d in (16, 64, 80, 128, 192, 256):
        one = o.prefill_blocks_per_cu(torch.bfloat16, d, 16, 1)
        two = o.prefill_blocks_per_cu(torch.bfloat16, d, 16, 2)
        assert 1 <= two <= one <= 8, (d, one, two)
    assert o.prefill_blocks_per_cu(torch.float32, 64, 16, 1) >= 1
    assert o.prefill_blocks_per_cu(torch.bfloat16, 64, 4, 1) >= 1    # pages of 4: the 32-bit kernel's way


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 4), (3, 1, 32, 8), (6, 1, 48, 16),
                                        (4, 4, 80, 16), (32, 8, 64, 16), (8, 2, 128, 16),
                                        (12, 1, 112, 16), (2, 1, 256, 32), (20, 1, 16, 8),
                                        (4, 2, 32, 6)])
@pytest.mark.parametrize("splits", [1, 3, 7])
@pytest.mark.parametrize("window", [0, 11])
def test_attn_decode(dtype, H, KV, d, bs, splits, window):
    seq_lens = [7, 13, 1, 20, 300, 64]  # tests/test_paged_attention.py:61 of the reference + long
    q_lens = [1] * len(seq_lens)
    paged = Paged(seq_lens, KV, d, bs, dtype, seed=d + H)
    g = torch.Generator().manual_seed(d)
    n = len(seq_lens)
    buf = torch.randn(n, (H + 2 * KV) * d, generator=g).to(dtype)
    q = buf[:, :H * d].reshape(n, H, d)
    cu = torch.arange(n + 1, dtype=torch.int32)
    ctx = torch.tensor(seq_lens, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    want = attn_reference(paged, q, seq_lens, q_lens, scale, window or None).reshape(n, H * d)
    ws = (torch.empty(n * H * splits * d, device=DEV), torch.empty(n * H * splits * 2, device=DEV),
          torch.zeros(n * H, dtype=torch.int32, device=DEV))
    out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
    ops().attn_decode(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), None, n,
                      cu.to(DEV), ctx.to(DEV), out, H, KV, d, scale, window, splits, ws)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
    # the caller may vouch that token i is sequence i's: the same bits without the lookup
    same = torch.zeros_like(out)
    ops().attn_decode(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), None, n,
                      cu.to(DEV), ctx.to(DEV), same, H, KV, d, scale, window, splits, ws,
                      token_is_seq=True)
    assert torch.equal(same, out)
    # a subset of the sequences, named by seq_ids; the others stay untouched
    ids = torch.tensor([4, 1], dtype=torch.int32)
    out2 = torch.full((n, H * d), 5.0, dtype=dtype, device=DEV)
    ops().attn_decode(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV),
                      ids.to(DEV), 2, cu.to(DEV), ctx.to(DEV), out2, H, KV, d, scale, window,
                      splits, ws)
    got = out2.float().cpu()
    torch.testing.assert_close(got[[4, 1]], want[[4, 1]], **tol(dtype))
    assert (got[[0, 2, 3, 5]] == 5.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", [1, 4])
def test_attn_decode_clears_the_rows_of_empty_sequences(dtype, splits):
    """A captured batch is padded with sequences that hold nothing.  With the key range in cuts
    their rows have no partial results; the merge must not read the workspace for them (it holds
    whatever an earlier step left, NaNs here) and gives them zeros.  With the key range whole
    their rows get zeros as well, not what an earlier step left in the output."""
    H, KV, d, bs = 8, 2, 64, 16
    seq_lens = [70, 1, 600]
    paged = Paged(seq_lens, KV, d, bs, dtype, seed=3)
    table = torch.cat([paged.table, torch.full((2, paged.table.shape[1]), -1, dtype=torch.int32)])
    n = 5
    g = torch.Generator().manual_seed(4)
    buf = torch.randn(n, (H + 2 * KV) * d, generator=g).to(dtype)
    ctx = torch.tensor(seq_lens + [0, 0], dtype=torch.int32)
    cu = torch.arange(n + 1, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    want = attn_reference(paged, buf[:3, :H * d].reshape(3, H, d), seq_lens, [1, 1, 1], scale, None)
    ws = (torch.full((n * H * splits * d,), float("nan"), device=DEV),
          torch.full((n * H * splits * 2,), float("nan"), device=DEV))
    out = torch.full((n, H * d), 7.0, dtype=dtype, device=DEV)
    ops().attn_decode(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), table.to(DEV), None, n, cu.to(DEV),
                      ctx.to(DEV), out, H, KV, d, scale, 0, splits, ws if splits > 1 else None,
                      token_is_seq=True)
    torch.testing.assert_close(out[:3].float().cpu(), want.reshape(3, H * d), **tol(dtype))
    assert bool((out[3:] == 0).all())


def attn_reference_with_slopes(paged, q, seq_lens, q_lens, scale, window, slopes):
    """Whole-sequence attention in which the score of key ``j`` for the query at position ``p``
    of head ``h`` is ``scale * q.k + slopes[h] * (j - p)``; written out row by row."""
    outs, off = [], 0
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        k, v = paged.keys[s].double(), paged.values[s].double()
        G = q.shape[1] // k.shape[1]
        out = torch.zeros(ql, q.shape[1], q.shape[2], dtype=torch.float64)
        for i in range(ql):
            p = n - ql + i
            first = max(0, p - window + 1) if window else 0
            j = torch.arange(first, p + 1)
            for h in range(q.shape[1]):
                sc = (k[first:p + 1, h // G] @ q[off + i, h].double()) * scale + float(slopes[h]) * (j - p).double()
                out[i, h] = torch.softmax(sc, 0) @ v[first:p + 1, h // G]
        outs.append(out)
        off += ql
    return torch.cat(outs).float()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 4), (3, 1, 32, 8), (6, 1, 48, 16), (8, 2, 128, 16),
                                        (32, 8, 64, 16), (20, 1, 16, 8), (4, 2, 32, 6)])
@pytest.mark.parametrize("window", [0, 11])
def test_attn_with_a_bias_by_distance(dtype, H, KV, d, bs, window):
    """Slopes of both signs and of different size per head, for query runs and for single tokens
    with the key range whole and in cuts.  A slope of the wrong sign, or one taken from another
    head, moves the weight to the other end of the context."""
    slopes = torch.tensor([(-1) ** h * 0.04 * (1 + h % 5) for h in range(H)], dtype=torch.float32)
    scale = 1 / math.sqrt(d)
    g = torch.Generator().manual_seed(d + H)
    # query runs
    seq_lens, q_lens = [12, 30, 5, 200], [4, 7, 5, 67]
    paged = Paged(seq_lens, KV, d, bs, dtype, seed=d)
    n = sum(q_lens)
    buf = torch.randn(n, (H + 2 * KV) * d, generator=g).to(dtype)
    q = buf[:, :H * d].reshape(n, H, d)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    ctx = torch.tensor(seq_lens, dtype=torch.int32)
    out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
    dev = (buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV))
    ops().attn_prefill(*dev, cu.to(DEV), ctx.to(DEV), prefill_work(q_lens, H // KV, dtype, d, bs).to(DEV),
                       out, H, KV, d, scale, window, slopes=slopes.to(DEV))
    want = attn_reference_with_slopes(paged, q.float(), seq_lens, q_lens, scale, window, slopes).reshape(n, H * d)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
    plain_out = attn_reference(paged, q, seq_lens, q_lens, scale, window or None).reshape(n, H * d)
    assert (want - plain_out).abs().max() > 0.1          # the bias is no detail here
    # single tokens
    seq_lens = [7, 13, 1, 20, 300, 64]
    paged = Paged(seq_lens, KV, d, bs, dtype, seed=d + 1)
    n = len(seq_lens)
    buf = torch.randn(n, (H + 2 * KV) * d, generator=g).to(dtype)
    q = buf[:, :H * d].reshape(n, H, d)
    cu = torch.arange(n + 1, dtype=torch.int32)
    ctx = torch.tensor(seq_lens, dtype=torch.int32)
    want = attn_reference_with_slopes(paged, q.float(), seq_lens, [1] * n, scale, window, slopes).reshape(n, H * d)
    dev = (buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV))
    for splits in (1, 3):
        ws = (torch.empty(n * H * splits * d, device=DEV), torch.empty(n * H * splits * 2, device=DEV))
        out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
        ops().attn_decode(*dev, None, n, cu.to(DEV), ctx.to(DEV), out, H, KV, d, scale, window, splits, ws,
                          slopes=slopes.to(DEV))
        torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


def test_attn_slopes_are_checked():
    H, KV, d, bs = 4, 2, 16, 4
    paged = Paged([9], KV, d, bs, torch.float32)
    buf = torch.randn(1, (H + 2 * KV) * d).to(DEV)
    args = (buf, paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), None, 1,
            torch.arange(2, dtype=torch.int32, device=DEV), torch.tensor([9], dtype=torch.int32, device=DEV),
            torch.zeros(1, H * d, device=DEV), H, KV, d, 0.25)
    for bad in (torch.zeros(H - 1, device=DEV), torch.zeros(H, dtype=torch.bfloat16, device=DEV), torch.zeros(H)):
        with pytest.raises(Exception, match="slopes"):
            ops().attn_decode(*args, slopes=bad)


@pytest.mark.parametrize("slope", [0.12, 0.3, -0.2])
def test_attn_scores_that_keep_rising_or_falling(slope):
    """Scores that grow (or shrink) steadily with the key's position, by less and by more per key
    block than the headroom within which the matrix-core kernel leaves its softmax reference
    alone: a reference raised too late, too early or without rescaling the sums shows here."""
    H, KV, d, bs, n = 8, 2, 64, 16, 600
    b16 = torch.bfloat16
    u = torch.zeros(d)
    u[3] = 1.0

    def ramp(kk):  # key j gets j * slope * sqrt(d) along u: its score with q = u grows by slope
        return 0.3 * kk + (torch.arange(kk.shape[0]).float() * slope * math.sqrt(d))[:, None, None] * u

    paged = Paged([n], KV, d, bs, b16, seed=5, shape_keys=ramp)
    g = torch.Generator().manual_seed(9)
    q = (0.2 * torch.randn(n, H, d, generator=g) + u).to(b16)
    scale = 1 / math.sqrt(d)
    want = plain.causal_attention(q.float(), paged.keys[0].float(), paged.values[0].float(), scale, 0)
    want = want.reshape(n, H * d)
    cu = torch.tensor([0, n], dtype=torch.int32)
    ctx = torch.tensor([n], dtype=torch.int32)
    out = torch.zeros(n, H * d, dtype=b16, device=DEV)
    ops().attn_prefill(q.reshape(n, H * d).to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV),
                       cu.to(DEV), ctx.to(DEV), prefill_work([n], H // KV, b16, d, bs).to(DEV), out,
                       H, KV, d, scale, 0)
    torch.testing.assert_close(out.float().cpu(), want, atol=2e-2, rtol=2e-2)
    # the last token alone, through the decode kernel, whole and in cuts
    cu1 = torch.tensor([0, 1], dtype=torch.int32)
    for splits in (1, 3):
        ws = (torch.empty(H * splits * d, device=DEV), torch.empty(H * splits * 2, device=DEV))
        one = torch.zeros(1, H * d, dtype=b16, device=DEV)
        ops().attn_decode(q[n - 1:].reshape(1, H * d).to(DEV), paged.k.to(DEV), paged.v.to(DEV),
                          paged.table.to(DEV), None, 1, cu1.to(DEV), ctx.to(DEV), one, H, KV, d, scale,
                          0, splits, ws)
        torch.testing.assert_close(one.float().cpu(), want[n - 1:], atol=2e-2, rtol=2e-2)


def test_attn_far_key_stands_out():
    """One key among hundreds carries the weight: q and that key are scaled so that its score
    dominates; a kernel that drops or misplaces a page shows at once."""
    H, KV, d, bs = 4, 2, 64, 16
    for far in (0, 15, 16, 255, 256, 511, 599):
        seq_lens = [600]
        paged = Paged(seq_lens, KV, d, bs, torch.float32, seed=far)
        g = torch.Generator().manual_seed(far)
        q = torch.randn(1, H, d, generator=g)
        for kvh in range(KV):
            key = paged.keys[0][far, kvh]
            for gi in range(H // KV):
                q[0, kvh * (H // KV) + gi] = key * 40.0 / key.norm() ** 2 * math.sqrt(d)
        buf = torch.zeros(1, (H + 2 * KV) * d)
        buf[:, :H * d] = q.reshape(1, -1)
        cu = torch.tensor([0, 1], dtype=torch.int32)
        ctx = torch.tensor(seq_lens, dtype=torch.int32)
        want = attn_reference(paged, q, seq_lens, [1], 1 / math.sqrt(d), None).reshape(1, H * d)
        # the far key's value dominates
        assert (want.reshape(H, d)[0] - paged.values[0][far, 0]).abs().max() < 0.05
        for splits in (1, 4):
            ws = (torch.empty(H * splits * d, device=DEV), torch.empty(H * splits * 2, device=DEV),
                  torch.zeros(H, dtype=torch.int32, device=DEV))
            out = torch.zeros(1, H * d, device=DEV)
            ops().attn_decode(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV),
                              None, 1, cu.to(DEV), ctx.to(DEV), out, H, KV, d, 1 / math.sqrt(d), 0,
                              splits, ws)
            torch.testing.assert_close(out.cpu(), want, atol=2e-5, rtol=2e-5)
            # the same through the matrix-core kernel (operands rounded to bf16)
            b16 = torch.bfloat16
            outb = torch.zeros(1, H * d, dtype=b16, device=DEV)
            ops().attn_decode(buf.to(b16).to(DEV), paged.k.to(b16).to(DEV), paged.v.to(b16).to(DEV),
                              paged.table.to(DEV), None, 1, cu.to(DEV), ctx.to(DEV), outb, H, KV, d,
                              1 / math.sqrt(d), 0, splits, ws)
            wantb = plain.causal_attention(q.to(b16).float(), paged.keys[0].to(b16).float(),
                                           paged.values[0].to(b16).float(), 1 / math.sqrt(d), 599)
            torch.testing.assert_close(outb.float().cpu(), wantb.reshape(1, H * d), atol=2e-2, rtol=2e-2)
            assert (outb.float().cpu().reshape(H, d)[0] - paged.values[0][far, 0]).abs().max() < 0.1
        out = torch.zeros(1, H * d, device=DEV)
        ops().attn_prefill(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV),
                           cu.to(DEV), ctx.to(DEV), prefill_work([1], H // KV, torch.float32, d, bs).to(DEV), out,
                           H, KV, d, 1 / math.sqrt(d), 0)
        torch.testing.assert_close(out.cpu(), want, atol=2e-5, rtol=2e-5)


# (sequence, first position, tokens) of each portion in the flat batch.  The kernel takes the
# batch in tiles of 16 tokens and writes V by whole runs where a tile lies in one page: the cases
# hold tiles that do (pages of 16 from position 0 or 16, pages of 32 from position 8), tiles that
# straddle pages or sequences, a short last tile, and a page that was given back.
ROPE_BATCHES = {
    "mixed": [(0, 2, 5), (1, 0, 19)],              # the first sequence already holds two tokens
    "aligned": [(1, 0, 37)],
    "offset": [(0, 8, 16), (1, 16, 20)],
    "late_start": [(0, 0, 3), (1, 3, 34)],
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch", sorted(ROPE_BATCHES))
@pytest.mark.parametrize("H,KV,d,rot,bs", [(4, 2, 16, 16, 4), (3, 1, 32, 32, 8), (2, 2, 48, 32, 16),
                                            (5, 2, 20, 12, 16), (2, 1, 64, 64, 32), (8, 8, 128, 128, 16)])
def test_rope_kvwrite(dtype, batch, H, KV, d, rot, bs):
    g = torch.Generator().manual_seed(d)
    portions = ROPE_BATCHES[batch]
    n = sum(c for _, _, c in portions)
    qkv = torch.randn(n, (H + 2 * KV) * d, generator=g).to(dtype)
    positions = torch.tensor([p0 + i for _, p0, c in portions for i in range(c)], dtype=torch.int32)
    seq_of = torch.tensor([sq for sq, _, c in portions for _ in range(c)], dtype=torch.int32)
    nb = 24
    width = -(-40 // bs) + 1
    table = torch.randperm(nb, generator=g)[:2 * width].reshape(2, width).to(torch.int32)
    table[0, -(-24 // bs):] = -1                   # the first sequence has no pages past 24 tokens
    if batch == "mixed":
        table[1, 0] = -1                           # a page that was given back
    table = table.contiguous()
    inv_freq = plain.rope_inv_freq(rot, 10000.0)
    cos_full, sin_full = plain.rope_cos_sin(torch.arange(40), inv_freq)
    cos_t, sin_t = cos_full[:, : rot // 2].contiguous(), sin_full[:, : rot // 2].contiguous()
    kp = torch.zeros(nb, KV, bs, d, dtype=dtype, device=DEV)
    vp = torch.zeros(nb, KV, d, bs, dtype=dtype, device=DEV)
    dev_qkv = qkv.to(DEV).clone()
    ops().rope_kvwrite(dev_qkv, positions.to(DEV), seq_of.to(DEV), cos_t.to(DEV), sin_t.to(DEV),
                       table.to(DEV), kp, vp, H, KV, d)
    cos, sin = plain.rope_cos_sin(positions, inv_freq)
    qf = qkv[:, :H * d].float().reshape(n, H, d)
    kf = qkv[:, H * d:(H + KV) * d].float().reshape(n, KV, d)
    vf = qkv[:, (H + KV) * d:].float().reshape(n, KV, d)

    # the kernel pairs neighbouring elements: element 2i / 2i+1 of its layout is what the plain
    # half-split formula calls element i / i + rot/2
    perm = torch.arange(d)
    for i in range(rot // 2):
        perm[2 * i], perm[2 * i + 1] = i, i + rot // 2
    inv = torch.argsort(perm)

    def rot_part(x):
        half_split = x[..., inv]
        r = plain.apply_rope(half_split[..., :rot], cos, sin)
        return torch.cat([r, half_split[..., rot:]], -1)[..., perm]

    want_q, want_k = rot_part(qf), rot_part(kf)
    got_q = dev_qkv[:, :H * d].float().cpu().reshape(n, H, d)
    torch.testing.assert_close(got_q, want_q, **tol(dtype))
    kp, vp = kp.float().cpu(), vp.float().cpu()
    for t in range(n):
        s, p = int(seq_of[t]), int(positions[t])
        page, off = int(table[s, p // bs]), p % bs
        if page < 0:
            continue
        torch.testing.assert_close(kp[page, :, off], want_k[t], **tol(dtype))
        torch.testing.assert_close(vp[page, :, :, off], vf[t], **tol(dtype))
    # nothing else was written
    written = torch.zeros(nb, bs, dtype=torch.bool)
    for t in range(n):
        s, p = int(seq_of[t]), int(positions[t])
        if int(table[s, p // bs]) >= 0:
            written[int(table[s, p // bs]), p % bs] = True
    assert (kp.abs().sum((1, 3))[~written] == 0).all()
    assert (vp.abs().sum((1, 2))[~written] == 0).all()


def test_sample_greedy_and_filters():
    # src/tokenvault tests/test_continuous_batching.py:160-169: logits [4,3,2,1,0]
    logits = torch.tensor([[4.0, 3.0, 2.0, 1.0, 0.0]] * 4, device=DEV)
    temp = torch.tensor([0.0, 1.0, 1.0, 1.0], device=DEV)
    top_k = torch.tensor([0, 2, 0, 1], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([1.0, 1.0, 0.5, 1.0], device=DEV)
    toks = torch.empty(4, dtype=torch.int32, device=DEV)
    for u in (0.0, 0.3, 0.72, 0.74, 0.999):
        uu = torch.full((4,), u, device=DEV)
        ops().sample(logits, temp, top_k, top_p, uu, toks)
        got = toks.tolist()
        assert got[0] == 0
        p2 = plain_sampling.processed_probs(logits[1].cpu(), 1.0, top_k=2)
        assert got[1] == plain_sampling.draw(p2, u) and got[1] in (0, 1)
        assert got[2] == 0          # top_p = 0.5 keeps only the first (mass 0.64)
        assert got[3] == 0


@pytest.mark.parametrize("V", [384, 5000, 128256])
def test_sample_matches_plain(V):
    g = torch.Generator().manual_seed(V)
    rows = 12
    logits = torch.randn(rows, V, generator=g) * 3
    temps = [0.0, 0.8, 1.0, 0.5, 1.3, 0.8, 0.8, 1.0, 0.7, 2.0, 0.0, 1.0]
    ks = [0, 0, 50, 0, 7, 20, 0, 1, 0, 0, 5, 300]
    ps = [1.0, 1.0, 1.0, 0.9, 0.8, 1.0, 0.3, 1.0, 0.95, 1.0, 0.5, 0.6]
    us = [plain_sampling.uniform(V, r, 3) for r in range(rows)]
    toks = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops().sample(logits.to(DEV), torch.tensor(temps, device=DEV),
                 torch.tensor(ks, dtype=torch.int32, device=DEV), torch.tensor(ps, device=DEV),
                 torch.tensor(us, device=DEV), toks)
    got = toks.tolist()
    for r in range(rows):
        probs = plain_sampling.processed_probs(logits[r], temps[r], ks[r], ps[r])
        if temps[r] == 0.0:
            assert got[r] == int(logits[r].argmax())
            continue
        assert probs[got[r]] > 0, f"row {r}: token {got[r]} was filtered out"
        # equal to the plain draw unless u falls within rounding of an interval's edge
        assert plain_sampling.draw_margin(probs, us[r], got[r]) < 1e-5, f"row {r}"


@pytest.mark.parametrize("rows", [1, 8, 37])
@pytest.mark.parametrize("V", [4100, 50001, 128256])
def test_sample_greedy_rows_read_in_chunks(rows, V):
    """Greedy rows cut over several workgroups give the token of one workgroup per row: the
    largest logit, the lowest index among equal ones (put into different chunks here), also on a
    second call that finds the tickets of the first; sampled rows beside them are untouched by
    the cut."""
    g = torch.Generator().manual_seed(rows * V)
    wide = torch.randn(rows, V + 3, generator=g)
    logits = wide[:, :V]                           # an odd vocabulary leaves rows unaligned
    top = float(logits.max()) + 1.0
    for r in range(rows):
        where = torch.randint(0, V, (3,), generator=g)
        logits[r, where] = top + r                 # the same maximum at up to three places
    temps = torch.tensor([0.9 if r % 5 == 3 else 0.0 for r in range(rows)])
    us = torch.tensor([plain_sampling.uniform(1, r, 0) for r in range(rows)])
    dev_logits = wide.to(DEV)[:, :V]
    one = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops().sample(dev_logits, temps.to(DEV), None, None, us.to(DEV), one)
    work = torch.zeros(ops().sample_work_size(rows), dtype=torch.int32, device=DEV)
    for _ in range(2):
        cut = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        ops().sample(dev_logits, temps.to(DEV), None, None, us.to(DEV), cut, work=work)
        assert torch.equal(cut, one)
        assert int(work[:rows].abs().sum()) == 0
    for r in range(rows):
        if temps[r] == 0.0:
            assert int(one[r]) == int((logits[r] == logits[r].max()).nonzero()[0])
    with pytest.raises(ops().KernelError):
        ops().sample(dev_logits, temps.to(DEV), None, None, us.to(DEV), one, work=work[:rows])


def test_sample_frequencies_follow_softmax():
    logits = torch.tensor([1.0, 0.0, -1.0, 2.0, 0.5])
    n = 4000
    us = torch.tensor([plain_sampling.uniform(7, 0, i) for i in range(n)])
    toks = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample(logits.repeat(n, 1).to(DEV), torch.full((n,), 0.8, device=DEV), None, None,
                 us.to(DEV), toks)
    freq = torch.bincount(toks.cpu().long(), minlength=5).double() / n
    want = torch.softmax(logits.double() / 0.8, -1)
    assert (freq - want).abs().max() < 0.03
