"""Python faces of the HIP kernels.  Each function checks on the host that shapes, dtypes,
devices and strides are what its kernel and launch grid assume, then launches on torch's
current stream (so launches made while a torch HIP-graph capture is active are captured).

There is no fallback: every function here runs a hand-written gfx950 kernel, or (``gemm`` for
bf16 with many rows, as the reference's engine does for its products) the library's matrix
product through ``csrc/gemm_library.hip``, or raises.  No torch operator computes anything
here.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

import torch

from kvforge_amd.kernels import library

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32


class KernelError(RuntimeError):
    pass


def _tcode(dtype: torch.dtype) -> int:
    if dtype == F32:
        return 0
    if dtype == BF16:
        return 1
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}")


def _suffix(dtype: torch.dtype) -> str:
    return "f32" if _tcode(dtype) == 0 else "bf16"


# the raw handle of torch's current stream, without a Stream object built for every launch
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(t: torch.Tensor, name: str, dtype=None, shape=None, contiguous=True) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name} must be a tensor on the GPU")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None:
        have = t.shape
        bad = len(have) != len(shape)
        if not bad:
            for want, got in zip(shape, have):   # a plain loop: this runs for every operand of every launch
                if want is not None and want != got:
                    bad = True
                    break
        if bad:
            raise KernelError(f"{name} must have shape {list(shape)}, got {list(have)}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


def _overlap(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Whether the memory spanned by two tensors' storage views intersects."""
    def span(t):
        if t.numel() == 0:
            return t.data_ptr(), t.data_ptr()
        last = sum((n - 1) * st for n, st in zip(t.shape, t.stride()))
        return t.data_ptr(), t.data_ptr() + (last + 1) * t.element_size()
    (a0, a1), (b0, b1) = span(a), span(b)
    return a0 < b1 and b0 < a1


def _ok(code: int, what: str) -> None:
    if code != 0:
        raise KernelError(f"{what} failed with HIP error {code}")


_fn_cache: dict[tuple[str, str], object] = {}


def _fn(module: str, name: str, argtypes: list):
    key = (module, name)
    f = _fn_cache.get(key)
    if f is None:
        lib = library.load(module)
        try:
            f = getattr(lib, name)
        except AttributeError:
            raise KernelError(f"kernel module {module!r} has no entry point {name!r}") from None
        f.argtypes = argtypes
        f.restype = c_int
        _fn_cache[key] = f
    return f


# ------------------------------------------------------------------------------ embedding
def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> None:
    """``out[n] = table[ids[n]]`` widened to fp32 (the residual stream)."""
    n = ids.shape[0]
    _check(ids, "ids", I32, (n,))
    _check(table, "table", None, (None, None))
    vocab, h = table.shape
    _check(out, "out", F32, (n, h))
    f = _fn("elementwise", f"kvf_embed_{_suffix(table.dtype)}",
            [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p])
    _ok(f(ids.data_ptr(), table.data_ptr(), out.data_ptr(), n, h, vocab, _stream()), "embed")


# ------------------------------------------------------------------------------ RMS norm
def rmsnorm(x: torch.Tensor, weight: torch.Tensor | None, eps: float, out: torch.Tensor,
            rows: torch.Tensor | None = None, add: torch.Tensor | None = None) -> None:
    """``out[m] = y * rsqrt(mean(y^2) + eps) * weight`` with ``y = x[rows[m] or m]`` in fp32
    (``weight=None``: no weight, for a norm whose weight is folded into the next matrix).
    ``add`` (``[rows of x, h]``, dtype of ``out`` or fp32) is a sum still owed to ``x``: the norm
    is taken of ``x + add``, and without ``rows`` the sum is written back to ``x`` as well."""
    _check(x, "x", F32, (None, None))
    xr, h = x.shape
    m = out.shape[0]
    _check(out, "out", None, (m, h))
    if weight is not None:
        _check(weight, "weight", None, (h,))
        if weight.dtype not in (F32, out.dtype):
            raise KernelError(f"norm weight must be float32 or {out.dtype}, got {weight.dtype}")
    if rows is not None:
        _check(rows, "rows", I32, (m,))
    elif m > xr:
        raise KernelError("rmsnorm: more output rows than input rows")
    if add is not None:
        _check(add, "add", None, (xr, h))
        if add.dtype not in (F32, out.dtype):
            raise KernelError(f"rmsnorm: add must be float32 or {out.dtype}, got {add.dtype}")
    f = _fn("elementwise", f"kvf_rmsnorm_{_suffix(out.dtype)}",
            [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_int, c_int,
             c_int, c_void_p])
    _ok(f(x.data_ptr(), rows.data_ptr() if rows is not None else None,
          add.data_ptr() if add is not None else None,
          1 if add is not None and add.dtype == F32 else 0,
          weight.data_ptr() if weight is not None else None,
          1 if weight is not None and weight.dtype == F32 else 0, float(eps), out.data_ptr(),
          m, h, xr, _stream()), "rmsnorm")


def add_rows(x: torch.Tensor, delta: torch.Tensor) -> None:
    """``x += delta`` for the fp32 residual stream ``x`` and a product ``delta`` of equal shape."""
    _check(x, "x", F32, (None, None))
    _check(delta, "delta", None, tuple(x.shape))
    f = _fn("elementwise", f"kvf_add_rows_{_suffix(delta.dtype)}", [c_void_p, c_void_p, c_int, c_int, c_void_p])
    _ok(f(x.data_ptr(), delta.data_ptr(), x.shape[0], x.shape[1], _stream()), "add_rows")


# ------------------------------------------------------------------------------ SwiGLU gate
def silu_mul(gate_up: torch.Tensor, out: torch.Tensor, paired: bool = False) -> None:
    """``out[:, i] = silu(gate_i) * up_i`` where the input row holds gate at ``i`` and up at
    ``I + i``, or, with ``paired``, gate at ``2i`` and up at ``2i + 1``."""
    m, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("silu_mul: input width must be even")
    _check(gate_up, "gate_up", None, (m, two_i))
    _check(out, "out", gate_up.dtype, (m, two_i // 2))
    f = _fn("elementwise", f"kvf_silu_mul_{_suffix(out.dtype)}",
            [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p])
    _ok(f(gate_up.data_ptr(), out.data_ptr(), m, two_i // 2, 1 if paired else 0, _stream()),
        "silu_mul")


# ------------------------------------------------------------------------------ rotary + cache
NO_TABLE_LEN = 2**31 - 1


def _rotary_tables(cos, sin, d: int, who: str):
    """(cos pointer, sin pointer, rotary width, positions the tables cover).  Without tables
    (both ``None``) nothing is rotated, the width is 0 and every position is covered."""
    if cos is None and sin is None:
        return None, None, 0, NO_TABLE_LEN
    _check(cos, "cos", F32, (None, None))
    _check(sin, "sin", F32, tuple(cos.shape))
    table_len, half = cos.shape
    if 2 * half > d or half <= 0:
        raise KernelError(f"{who}: rotary width {2 * half} does not fit head_dim {d}")
    return cos.data_ptr(), sin.data_ptr(), 2 * half, table_len


def rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor,
                 cos: torch.Tensor | None, sin: torch.Tensor | None, block_table: torch.Tensor,
                 k_pages: torch.Tensor, v_pages: torch.Tensor, num_heads: int, num_kv_heads: int,
                 head_dim: int, write_kv: bool = True) -> None:
    """Rotate q (in place) and k by the cos/sin rows of each token's position; write rotated k
    and v into the pages named by the token's sequence row of ``block_table``.  Rotary pairs
    are neighbouring elements ``(2i, 2i + 1)`` of a head; without tables (``None``) q and k stay
    as they are and only the cache is written.  ``k_pages``:
    ``[num_blocks, KV, block_size, d]``; ``v_pages`` transposed: ``[num_blocks, KV, d, block_size]``."""
    n = qkv.shape[0]
    H, KV, d = num_heads, num_kv_heads, head_dim
    _check(qkv, "qkv", None, (n, (H + 2 * KV) * d))
    _check(positions, "positions", I32, (None,))
    _check(seq_of_token, "seq_of_token", I32, (None,))
    if positions.shape[0] < n or seq_of_token.shape[0] < n:
        raise KernelError("rope_kvwrite: positions / seq_of_token shorter than the batch")
    cos_p, sin_p, rot, table_len = _rotary_tables(cos, sin, d, "rope_kvwrite")
    _check(block_table, "block_table", I32, (None, None))
    n_seqs, stride = block_table.shape
    _check(k_pages, "k_pages", qkv.dtype, (None, KV, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", qkv.dtype, (nb, KV, d, bs))
    f = _fn("elementwise", f"kvf_rope_kvwrite_{_suffix(qkv.dtype)}",
            [c_void_p] * 8 + [c_int] * 11 + [c_void_p])
    _ok(f(qkv.data_ptr(), positions.data_ptr(), seq_of_token.data_ptr(), cos_p,
          sin_p, block_table.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
          n, H, KV, d, rot, table_len, bs, stride, nb, 1 if write_kv else 0, n_seqs, _stream()),
        "rope_kvwrite")


# ------------------------------------------------------------------------------ matrix products
# Rows of the left operand up to which the weight-streaming MFMA kernel is used for bf16.  Over
# tiled weights it measured faster than the library's product up to 32 rows on the shapes of a
# 1B-parameter decoder (and it folds rotary, cache write, SwiGLU gate and residual sum into its
# store); with more rows the library wins, and the reference's engine uses a library product
# there as well.
SKINNY_MAX_M = 32
FUSED_NORM_MAX_M = 16
FUSED_EPILOGUE_MAX_M = 64
_GEMM_BF16_ARGS = ([c_void_p, c_int, c_void_p, c_int, c_void_p] + [c_int] * 6
                   + [c_float, c_void_p, c_void_p, c_void_p])
# A product that is added to a narrow fp32 stream (few output columns, long K) has too few
# workgroups to pull on the weights with all of the chip: with groups of 16 columns for at most
# half the compute units and from this K on it is cut into two halves of K
# (``k_halves_pay``).  The half that is left owed costs its consumers a second fp32 operand, so
# wider streams lose more there than the product gains (measured at 3072 columns: 7% of the step).
K_HALVES_MIN_K = 4096
_compute_units: dict[int, int] = {}


def compute_units(device) -> int:
    """Compute units of the device, asked of the device once."""
    index = torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    if index not in _compute_units:
        _compute_units[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _compute_units[index]


class StreamedWeight:
    """A bf16 weight matrix ``[N, K]`` kept twice: ``plain`` as the checkpoint has it (what the
    library product and the fp32 kernels read) and ``tiles``, ``[ceil(N/16), ceil(K/32), 64, 8]``,
    where tile ``(g, s)`` holds rows ``16g..16g+15``, columns ``32s..32s+31`` in the order the
    matrix-core instruction takes them (position ``16*c + r`` holds row ``r``, columns
    ``8c..8c+7``), zero-padded.  The weight-streaming kernel then loads 1 KB of consecutive bytes
    per operand fragment instead of 64 bytes from each of 16 rows, which is what lets it reach
    the memory's bandwidth.  Costs the matrix's size in memory a second time."""

    def __init__(self, plain: torch.Tensor) -> None:
        if plain.dim() != 2 or plain.dtype != BF16 or not plain.is_contiguous():
            raise KernelError("a streamed weight is a contiguous bf16 matrix")
        n, k = plain.shape
        n_pad, k_pad = -(-n // 16) * 16, -(-k // 32) * 32
        padded = plain
        if (n_pad, k_pad) != (n, k):
            padded = torch.zeros(n_pad, k_pad, dtype=BF16, device=plain.device)
            padded[:n, :k] = plain
        self.plain = plain
        self.tiles = (padded.view(n_pad // 16, 16, k_pad // 32, 4, 8).permute(0, 2, 3, 1, 4)
                      .contiguous().view(n_pad // 16, k_pad // 32, 64, 8))
        self.shape, self.dtype, self.device = plain.shape, plain.dtype, plain.device

    def dim(self) -> int:
        return 2


TILE_WEIGHTS = True  # parts keep the matrices they stream for few rows in tiles as well


def streamed(w: torch.Tensor):
    """``w`` ready for ``gemm`` and its fused forms: bf16 matrices on the GPU also in tiles."""
    if (TILE_WEIGHTS and w is not None and w.dtype == BF16 and w.is_cuda and w.dim() == 2
            and w.is_contiguous()):
        return StreamedWeight(w)
    return w


def plain_of(w) -> torch.Tensor:
    return w.plain if isinstance(w, StreamedWeight) else w


def copies_of(w) -> list[torch.Tensor]:
    """Every tensor that holds ``w``: the matrix itself, and its tiles if it is streamed."""
    if isinstance(w, StreamedWeight):
        return [w.plain, w.tiles]
    return [] if w is None else [w]


def _w_args(w) -> tuple[int, int]:
    """(pointer, tiled flag) of a weight for the weight-streaming kernel."""
    if isinstance(w, StreamedWeight):
        return w.tiles.data_ptr(), 1
    return w.data_ptr(), 0


def _gemm_operands(a, w, out, n_out):
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
        raise KernelError("gemm takes 2-D tensors")
    m, k = a.shape
    n, k2 = w.shape
    if k != k2 or tuple(out.shape) != (m, n_out(n)):
        raise KernelError(f"gemm shapes do not agree: a {list(a.shape)}, w {list(w.shape)}, "
                          f"out {list(out.shape)}")
    _check(a, "a", None, None, contiguous=False)
    _check(plain_of(w), "w")
    _check(out, "out", None, None, contiguous=False)
    if a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows of a and out must be dense")
    lda = a.stride(0) if m > 1 else k
    ldc = out.stride(0) if m > 1 else out.shape[1]
    return m, n, k, lda, ldc


def _rows_aligned(a: torch.Tensor, k: int, lda: int) -> bool:
    """Rows that the matrix-core kernels (and the library) read 16 bytes at a time: eight
    elements per step of K, every row and the first one at a multiple of 16 bytes."""
    return k % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0


def bf16_kernel_takes(a: torch.Tensor, w: torch.Tensor, rms: bool = False,
                      fused_epilogue: bool = False) -> bool:
    """Whether the MFMA weight-streaming kernel takes these operands: bf16 weights, bf16 rows
    (or, with ``rms``, fp32 rows), 16-byte aligned rows, at most ``SKINNY_MAX_M`` of them.
    Folding the norm in pays only while every workgroup converts one tile of rows
    (``FUSED_NORM_MAX_M``); beyond that a norm kernel of its own is cheaper.  Where the kernel's
    epilogue stands for a kernel of its own after the library's product (``fused_epilogue``:
    rotary and cache write, the SwiGLU gate) it pays up to ``FUSED_EPILOGUE_MAX_M`` rows."""
    m, k = a.shape
    lda = a.stride(0) if m > 1 else k
    limit = FUSED_NORM_MAX_M if rms else (FUSED_EPILOGUE_MAX_M if fused_epilogue else SKINNY_MAX_M)
    return (w.dtype == BF16 and a.dtype == (F32 if rms else BF16) and _rows_aligned(a, k, lda)
            and m <= limit)


def is_library_product(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm(a, w, ...)`` hands the product to the library: bf16 with more rows than the
    weight-streaming kernel takes; or more than one tile of rows over a deep and narrow weight
    (K >= 2 N), where that kernel has few workgroups and each re-reads every row of ``a`` along
    a long K (measured at [2048, 8192] and 32 rows: 19 us against the library's 15)."""
    m, k = a.shape
    n = w.shape[0]
    lda = a.stride(0) if m > 1 else k
    return (a.dtype == BF16 and w.dtype == BF16 and _rows_aligned(a, k, lda)
            and (m > SKINNY_MAX_M or (m > 16 and k >= 2 * n)))


def k_halves_pay(a: torch.Tensor, w) -> bool:
    """Whether ``gemm(a, w, out, accumulate=True, half_out=...)`` is worth asking for: one tile of
    bf16 rows over a deep weight with few columns (the down projection of a small model)."""
    m, k = a.shape
    return (not is_library_product(a, w) and a.dtype == BF16 and plain_of(w).dtype == BF16
            and k % 8 == 0 and m <= 16 and k >= K_HALVES_MIN_K
            and -(-w.shape[0] // 16) <= compute_units(a.device) // 2)


# The library's product is called through an entry point of our own: torch.mm costs 17 us of
# host time a call, which is what bounds a step that is launched kernel by kernel (a portion of a
# prompt) at a few hundred rows.
LIBRARY_WORKSPACE_BYTES = 76 << 20
_library_ready: dict[int, bool] = {}
_LIBRARY_ARGS = [c_void_p, c_void_p, c_void_p] + [c_int] * 7 + [c_void_p]


def library_ready(device) -> None:
    """Set the library product up on ``device`` (its workspace is allocated here, once): to be
    called outside any stream capture, which ``gemm`` does by itself on its first library
    product."""
    dev = torch.device(device).index
    if dev is None:
        dev = torch.cuda.current_device()
    if _library_ready.get(dev):
        return
    if torch.cuda.is_current_stream_capturing():
        raise KernelError("the library product has to be set up before a stream is captured: "
                          "run the step once (or call ops.library_ready) outside the capture")
    init = _fn("gemm_library", "kvf_gemm_library_init", [c_long])
    with torch.cuda.device(dev):
        _ok(init(LIBRARY_WORKSPACE_BYTES), "gemm_library_init")
    _library_ready[dev] = True


def _library_product(a, w, out, accumulate, m, n, k, lda, ldc) -> None:
    """``out = a @ w.T`` (or ``+=``, in fp32) by hipBLASLt, with fp32 sums stored as ``out`` has
    them.  Raises where the library names no algorithm for the shape."""
    if out.dtype not in (F32, BF16) or (accumulate and out.dtype != F32):
        raise KernelError(f"library product: output must be float32 or bfloat16, got {out.dtype}")
    library_ready(a.device)
    f = _fn("gemm_library", "kvf_gemm_library_bf16", _LIBRARY_ARGS)
    code = f(a.data_ptr(), w.data_ptr(), out.data_ptr(), 1 if out.dtype == F32 else 0,
             1 if accumulate else 0, m, n, k, lda, ldc, _stream())
    if code == -1:
        raise KernelError(f"the library has no bf16 product for {m} x {n} x {k} "
                          f"(row strides {lda} / {ldc})")
    _ok(code, "gemm_library")


def gemm(a: torch.Tensor, w, out: torch.Tensor, accumulate: bool = False,
         owed: torch.Tensor | None = None, half_out: torch.Tensor | None = None) -> None:
    """``out = a @ w.T`` (``accumulate``: ``out += a @ w.T`` with ``out`` fp32).

    ``a: [M, K]`` (row stride may exceed K), ``w: [N, K]`` contiguous or a ``StreamedWeight``,
    ``out: [M, N]``.
    bf16 x bf16 runs on MFMA with fp32 accumulation; any operand in fp32 runs the fp32
    vector-ALU kernel (true 32-bit multiply and accumulate).
    With ``accumulate``: ``owed`` (bf16, shape and row stride of ``out``) is a sum still owed to
    ``out`` and is added on the way; ``half_out`` (bf16, likewise, only where ``k_halves_pay``)
    receives the product over the second half of K *instead of* ``out``, which the caller then
    owes to ``out``: twice the workgroups pull on ``w``."""
    m, n, k, lda, ldc = _gemm_operands(a, w, out, lambda n: n)
    if accumulate and out.dtype != F32:
        raise KernelError("gemm: accumulation needs an fp32 output")
    for t, name in ((owed, "owed"), (half_out, "half_out")):
        if t is None:
            continue
        if not accumulate:
            raise KernelError(f"gemm: {name} goes with accumulate")
        _check(t, name, BF16, (m, n), contiguous=False)
        if t.stride(1) != 1 or (m > 1 and t.stride(0) != ldc):
            raise KernelError(f"gemm: {name} must have the row stride of out")
    if half_out is not None and not k_halves_pay(a, w):
        raise KernelError("gemm: half_out only where k_halves_pay(a, w)")
    if half_out is not None:
        # the workgroups of one half of K read owed and out while those of the other write half_out
        for t, name in ((owed, "owed"), (out, "out")):
            if t is not None and _overlap(t, half_out):
                raise KernelError(f"gemm: half_out must not share memory with {name}")
    if m == 0:
        return
    out_kind = 2 if accumulate else (0 if out.dtype == F32 else 1)
    if not accumulate:
        _tcode(out.dtype)
    if a.dtype == BF16 and w.dtype == BF16 and _rows_aligned(a, k, lda):
        if not is_library_product(a, w):
            f = _fn("gemm_bf16", "kvf_gemm_bf16", _GEMM_BF16_ARGS)
            wp, tiled = _w_args(w)
            _ok(f(a.data_ptr(), 0, wp, tiled, out.data_ptr(), out_kind, m, n, k, lda, ldc, 0.0,
                  owed.data_ptr() if owed is not None else None,
                  half_out.data_ptr() if half_out is not None else None, _stream()), "gemm_bf16")
            return
        if owed is not None:
            add_rows(out, owed)
        _library_product(a, plain_of(w), out, accumulate, m, n, k, lda, ldc)
        return
    if owed is not None:
        add_rows(out, owed)
    w = plain_of(w)
    f = _fn("gemm_generic", "kvf_gemm_generic",
            [c_void_p, c_int, c_void_p, c_int, c_void_p] + [c_int] * 6 + [c_void_p])
    _ok(f(a.data_ptr(), _tcode(a.dtype), w.data_ptr(), _tcode(w.dtype), out.data_ptr(), out_kind,
          m, n, k, lda, ldc, _stream()), "gemm_generic")


def gemm_generic_vector_alus_only(on: bool) -> bool:
    """For tests: keep 32-bit products of many rows on the vector ALUs (the kernel of 64 x 64
    tiles that the matrix-core kernel replaced) or let them go to the matrix cores again.
    Returns the setting before."""
    f = _fn("gemm_generic", "kvf_gemm_generic_vector_alus_only", [c_int])
    return bool(f(1 if on else 0))


def gemm_fused(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rms_eps: float | None = None,
               silu_pairs: bool = False, accumulate: bool = False) -> None:
    """The MFMA weight-streaming product with work folded in at both ends.

    ``rms_eps``: ``a`` is the fp32 residual stream and each row is scaled by
    ``rsqrt(mean(a^2) + eps)`` (the norm's weight is already folded into ``w``).
    ``silu_pairs``: columns are (gate, up) pairs and ``out[:, j] = silu(c[2j]) * c[2j+1]``,
    ``out: [M, N/2]`` bf16.  Callers check ``bf16_kernel_takes`` first."""
    rms = rms_eps is not None
    m, n, k, lda, ldc = _gemm_operands(a, w, out, (lambda n: n // 2) if silu_pairs else (lambda n: n))
    if not bf16_kernel_takes(a, w, rms, silu_pairs):
        raise KernelError("gemm_fused: operands do not fit the MFMA kernel")
    if silu_pairs:
        if n % 4 or out.dtype != BF16 or accumulate:
            raise KernelError("gemm_fused: SwiGLU pairs need N in steps of 4 and a bf16 output")
        epi = 3
    elif accumulate:
        if out.dtype != F32:
            raise KernelError("gemm_fused: accumulation needs an fp32 output")
        epi = 2
    else:
        epi = 0 if out.dtype == F32 else 1
        _tcode(out.dtype)
    if m == 0:
        return
    f = _fn("gemm_bf16", "kvf_gemm_bf16", _GEMM_BF16_ARGS)
    wp, tiled = _w_args(w)
    _ok(f(a.data_ptr(), 1 if rms else 0, wp, tiled, out.data_ptr(), epi, m, n, k, lda, ldc,
          float(rms_eps or 0.0), None, None, _stream()), "gemm_bf16")


def gemm_qkv_rope(a: torch.Tensor, w: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                  seq_of_token: torch.Tensor, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  block_table: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int, write_kv: bool = True,
                  rms_eps: float | None = None, a_owed: torch.Tensor | None = None) -> None:
    """Fused q/k/v projection: ``a @ w.T`` with rotary applied to q and k (neighbouring columns
    are pairs), rotated q stored to ``q_out [M, H*d]`` and rotated k and v written into the
    pages; without tables (``None``) nothing is rotated.  ``rms_eps`` as in ``gemm_fused``.  ``a_owed`` (with ``rms_eps``; bf16, shape and
    strides, counted in elements, of ``a``): a sum still owed to ``a``; the projection is taken of ``a + a_owed``, and
    ``a`` itself is left as it is."""
    H, KV, d = num_heads, num_kv_heads, head_dim
    rms = rms_eps is not None
    m, k = a.shape
    _check(a, "a", None, (m, k), contiguous=False)
    _check(plain_of(w), "w", BF16, ((H + 2 * KV) * d, k))
    if not bf16_kernel_takes(a, w, rms, True) or a.stride(1) != 1:
        raise KernelError("gemm_qkv_rope: operands do not fit the MFMA kernel")
    if a_owed is not None:
        if not rms or m > FUSED_NORM_MAX_M:
            raise KernelError("gemm_qkv_rope: a_owed goes with rms_eps (fp32 rows, one tile of them)")
        _check(a_owed, "a_owed", BF16, (m, k), contiguous=False)
        if a_owed.stride() != a.stride():
            raise KernelError("gemm_qkv_rope: a_owed must have the strides of a")
    _check(q_out, "q_out", BF16, (m, H * d))
    _check(positions, "positions", I32, (None,))
    _check(seq_of_token, "seq_of_token", I32, (None,))
    if positions.shape[0] < m or seq_of_token.shape[0] < m:
        raise KernelError("gemm_qkv_rope: positions / seq_of_token shorter than the batch")
    cos_p, sin_p, rot, table_len = _rotary_tables(cos, sin, d, "gemm_qkv_rope")
    if d % 4:
        raise KernelError(f"gemm_qkv_rope: head_dim {d} not supported")
    _check(block_table, "block_table", I32, (None, None))
    _check(k_pages, "k_pages", BF16, (None, KV, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", BF16, (nb, KV, d, bs))
    if m == 0:
        return
    f = _fn("gemm_bf16", "kvf_gemm_bf16_qkv_rope",
            [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_float]
            + [c_void_p] * 8 + [c_int] * 10 + [c_void_p])
    wp, tiled = _w_args(w)
    _ok(f(a.data_ptr(), 1 if rms else 0, wp, tiled, q_out.data_ptr(), m, k,
          a.stride(0) if m > 1 else k, q_out.stride(0) if m > 1 else H * d, float(rms_eps or 0.0),
          a_owed.data_ptr() if a_owed is not None else None, positions.data_ptr(), seq_of_token.data_ptr(), cos_p, sin_p,
          block_table.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), H, KV, d, rot,
          table_len, bs, block_table.shape[1], nb, 1 if write_kv else 0, block_table.shape[0],
          _stream()), "gemm_qkv_rope")


def pick_workspace(rows: int, n: int, device) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Scratch of ``gemm_pick`` for ``rows`` rows over ``n`` columns: the workgroups' best values
    and columns, and the ticket (one int, zero between launches)."""
    pick_groups = _fn("gemm_bf16", "kvf_gemm_bf16_pick_groups", [c_int, c_int])
    # few rows take fewer columns per workgroup, hence more workgroups: room for any count up to rows
    groups = max(int(pick_groups(m, int(n))) for m in range(1, int(rows) + 1))
    tickets = int(_fn("gemm_bf16", "kvf_gemm_bf16_pick_ticket_ints", [])())
    return (torch.empty(16 * groups + 16 * 64, dtype=F32, device=device),
            torch.empty(16 * groups + 16 * 64, dtype=I32, device=device),
            torch.zeros(tickets, dtype=I32, device=device))


def gemm_pick(a: torch.Tensor, w, residual: torch.Tensor, tokens: torch.Tensor,
              token_ids: torch.Tensor, positions: torch.Tensor, ctx_lens: torch.Tensor,
              ring: torch.Tensor, run_counter: torch.Tensor, embed: torch.Tensor, work: tuple) -> None:
    """The output head of a decode step with everything after it folded in: ``a`` (the
    normalised rows, bf16, at most 16, one per sequence) is multiplied by ``w``, the largest
    logit of every row is picked without the logits being stored (lowest column among equal
    ones), and the picked token becomes its sequence's next input exactly as ``decode_advance``
    does it; the tokens' rows of ``embed`` are then written into ``residual`` (fp32, a row per
    sequence) as the next step's residual stream.  ``work``: from ``pick_workspace``; launches
    that share it must not overlap."""
    m, k = a.shape
    _check(a, "a", BF16, (m, k), contiguous=False)
    if a.stride(1) != 1 or m > FUSED_NORM_MAX_M or m == 0:
        raise KernelError(f"gemm_pick takes 1 to {FUSED_NORM_MAX_M} dense bf16 rows")
    _check(plain_of(w), "w", BF16, (None, k))
    n = w.shape[0]
    if not bf16_kernel_takes(a, w):
        raise KernelError("gemm_pick: operands do not fit the MFMA kernel")
    _check(residual, "residual", F32, (m, k), contiguous=False)
    if residual.stride(1) != 1 or (m > 1 and residual.stride(0) % 4):
        raise KernelError("gemm_pick: rows of the residual stream must be dense and start on 16 bytes")
    for t, name in ((tokens, "tokens"), (token_ids, "token_ids"), (positions, "positions"),
                    (ctx_lens, "ctx_lens")):
        _check(t, name, I32, (None,))
        if t.shape[0] < m:
            raise KernelError(f"gemm_pick: {name} is shorter than the batch")
    _check(ring, "ring", I32, (None, None))
    _check(run_counter, "run_counter", I32, (1,))
    if ring.shape[1] < m:
        raise KernelError("gemm_pick: rows of the ring are shorter than the batch")
    _check(embed, "embed", BF16, (None, k))
    if embed.shape[0] < n or k % 8:
        raise KernelError("gemm_pick: the embedding table must hold a row of K elements (a multiple "
                          "of 8) for every column of w")
    part_val, part_idx, ticket = work
    groups = int(_fn("gemm_bf16", "kvf_gemm_bf16_pick_groups", [c_int, c_int])(m, n))
    _check(part_val, "work[0]", F32, (None,))
    _check(part_idx, "work[1]", I32, (None,))
    _check(ticket, "work[2]", I32, (int(_fn("gemm_bf16", "kvf_gemm_bf16_pick_ticket_ints", [])()),))
    if part_val.shape[0] < 16 * groups + 16 * 64 or part_idx.shape[0] < 16 * groups + 16 * 64:
        raise KernelError("gemm_pick: workspace too small for these rows and columns")
    f = _fn("gemm_bf16", "kvf_gemm_bf16_pick",
            [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int] + [c_void_p] * 9
            + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p])
    wp, tiled = _w_args(w)
    _ok(f(a.data_ptr(), wp, tiled, m, n, k, a.stride(0) if m > 1 else k, part_val.data_ptr(),
          part_idx.data_ptr(), ticket.data_ptr(), tokens.data_ptr(), token_ids.data_ptr(),
          positions.data_ptr(), ctx_lens.data_ptr(), ring.data_ptr(), run_counter.data_ptr(),
          ring.shape[1], ring.shape[0], embed.data_ptr(), residual.data_ptr(), k,
          residual.stride(0) if m > 1 else k, _stream()), "gemm_pick")


def set_gemm_waves(waves: int, rows: int = 0) -> None:
    """Measurement aid: force the waves per workgroup and the rows of W per workgroup of the
    MFMA kernel (0 = by shape)."""
    lib = library.load("gemm_bf16")
    for fn, v in ((lib.kvf_gemm_bf16_set_waves, waves), (lib.kvf_gemm_bf16_set_rows, rows)):
        fn.argtypes = [c_int]
        fn.restype = None
        fn(int(v))


# ------------------------------------------------------------------------------ attention
def _attn_common(q, k_pages, v_pages, block_table, cu_q, ctx_lens, out, H, KV, d):
    if d % 16 or d > 256 or d <= 0:
        raise KernelError(f"attention kernels take head sizes in steps of 16 up to 256, got {d}")
    if H % KV:
        raise KernelError(f"query heads ({H}) must be a multiple of kv heads ({KV})")
    _check(q, "q", None, (None, None), contiguous=False)
    if q.stride(1) != 1 or q.shape[1] < H * d:
        raise KernelError("attention: q rows must be dense and hold all query heads")
    _check(k_pages, "k_pages", q.dtype, (None, KV, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", q.dtype, (nb, KV, d, bs))
    _check(block_table, "block_table", I32, (None, None))
    n_seqs = block_table.shape[0]
    _check(cu_q, "cu_q", I32, (None,))
    _check(ctx_lens, "ctx_lens", I32, (None,))
    if cu_q.shape[0] < n_seqs + 1 or ctx_lens.shape[0] < n_seqs:
        raise KernelError("attention: cu_q / ctx_lens shorter than the block table")
    _check(out, "out", q.dtype, (None, H * d))
    if out.shape[0] < q.shape[0]:
        raise KernelError("attention: out has fewer rows than q")
    return n_seqs


def _slopes_ptr(slopes, H: int, like: torch.Tensor):
    """Pointer to the per-head slopes of a bias by distance, or ``None`` for attention without."""
    if slopes is None:
        return None
    _check(slopes, "slopes", F32, (H,))
    if slopes.device != like.device:
        raise KernelError("attention: slopes live on another device than q")
    return slopes.data_ptr()


def attention_on_matrix_cores(dtype: torch.dtype, block_size: int) -> bool:
    """The MFMA attention kernels take bf16 and pages of a multiple of 8 tokens; everything else
    (the true 32-bit path above all) runs the vector-ALU kernel."""
    return dtype == BF16 and block_size % 8 == 0


def prefill_rows_per_item(dtype: torch.dtype, head_dim: int, block_size: int, row_tiles: int = 1) -> int:
    """Rows of (query token, head in group) that one entry of a prefill work list covers.
    ``row_tiles``: 1 or 2 tiles of 16 rows per wave of the matrix-core kernel (two where the head
    size allows them; they pay when the work fills the chip anyway, see ``attn_mfma.hip``)."""
    if attention_on_matrix_cores(dtype, block_size):
        return int(_fn("attn_mfma", "kvf_attn_mfma_rows_per_item", [c_int, c_int])(int(head_dim), int(row_tiles)))
    return int(_fn("attn_generic", "kvf_attn_generic_rows_per_item", [])())


_blocks_per_cu: dict[tuple, int] = {}


def prefill_blocks_per_cu(dtype: torch.dtype, head_dim: int, block_size: int, row_tiles: int = 1) -> int:
    """Workgroups of the kernel for query runs that one compute unit holds at a time (by its
    registers and LDS, asked of the runtime once): what fills the chip is this many times the
    compute units."""
    key = (dtype, int(head_dim), int(block_size) % 8 == 0, int(row_tiles))
    if key not in _blocks_per_cu:
        n = 4
        if attention_on_matrix_cores(dtype, block_size):
            n = int(_fn("attn_mfma", "kvf_attn_mfma_prefill_blocks_per_cu", [c_int, c_int])(int(head_dim), int(row_tiles)))
        _blocks_per_cu[key] = max(1, n)
    return _blocks_per_cu[key]


def attn_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                 block_table: torch.Tensor, cu_q: torch.Tensor, ctx_lens: torch.Tensor,
                 work: torch.Tensor, out: torch.Tensor, num_heads: int, num_kv_heads: int,
                 head_dim: int, scale: float, window: int = 0,
                 slopes: torch.Tensor | None = None, rows_per_item: int | None = None) -> None:
    """Causal attention of query runs over the paged cache.  ``work``: ``[num_work, 3]`` rows
    (sequence row, item, item or -1) where a sequence has ``query_len * H/KV`` rows per kv head,
    an item covers ``rows_per_item`` of them (what ``prefill_rows_per_item`` gave when the rows
    were made; by default its answer for one row tile), and the items of one row are taken by
    one workgroup in turn; rows start in the order given (the longest walks first).  ``v_pages`` are transposed:
    ``[num_blocks, KV, head_dim, block_size]``.  ``slopes``: fp32 ``[H]``; the score of key ``j``
    for a query at position ``p`` of head ``h`` then is ``scale * q.k + slopes[h] * (j - p)``."""
    H, KV, d = num_heads, num_kv_heads, head_dim
    n_seqs = _attn_common(q, k_pages, v_pages, block_table, cu_q, ctx_lens, out, H, KV, d)
    _check(work, "work", I32, (None, 3))
    sl = _slopes_ptr(slopes, H, q)
    nb, _, bs, _ = k_pages.shape
    if rows_per_item is None:
        rows_per_item = prefill_rows_per_item(q.dtype, d, bs)
    if attention_on_matrix_cores(q.dtype, bs):
        f = _fn("attn_mfma", "kvf_attn_mfma_prefill",
                [c_void_p] * 7 + [c_int, c_int] + [c_void_p] + [c_int] * 10 + [c_float, c_void_p, c_void_p])
        _ok(f(q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(),
              cu_q.data_ptr(), ctx_lens.data_ptr(), work.data_ptr(), work.shape[0], int(rows_per_item), out.data_ptr(),
              H, KV, d, bs, nb, block_table.shape[1], q.stride(0), out.stride(0), int(window),
              n_seqs, float(scale), sl, _stream()), "attn_mfma_prefill")
        return
    if rows_per_item != prefill_rows_per_item(q.dtype, d, bs):
        raise KernelError(f"attn_prefill: the 32-bit kernel takes items of "
                          f"{prefill_rows_per_item(q.dtype, d, bs)} rows, got {rows_per_item}")
    if q.stride(0) % 4 or out.stride(0) % 4:
        raise KernelError("attn_prefill: rows of q and out must start on 16 bytes")
    f = _fn("attn_generic", "kvf_attn_generic",
            [c_int] + [c_void_p] * 7 + [c_int] + [c_void_p] + [c_int] * 10
            + [c_float, c_void_p, c_void_p])
    _ok(f(_tcode(q.dtype), q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
          block_table.data_ptr(), cu_q.data_ptr(), ctx_lens.data_ptr(), work.data_ptr(),
          work.shape[0], out.data_ptr(), H, KV, d, bs, nb, block_table.shape[1], q.stride(0),
          out.stride(0), int(window), n_seqs, float(scale), sl, _stream()), "attn_generic")


def attn_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                block_table: torch.Tensor, seq_ids: torch.Tensor | None, num_seqs: int,
                cu_q: torch.Tensor, ctx_lens: torch.Tensor, out: torch.Tensor, num_heads: int,
                num_kv_heads: int, head_dim: int, scale: float, window: int = 0, splits: int = 1,
                workspace: tuple[torch.Tensor, torch.Tensor] | None = None,
                token_is_seq: bool = False, slopes: torch.Tensor | None = None) -> None:
    """Attention of one-token queries: sequence rows ``seq_ids[:num_seqs]`` (or ``0..num_seqs-1``)
    each attend from their token ``cu_q[seq]`` over ``ctx_lens[seq]`` cached keys.  The key
    range may be cut into ``splits`` runs; ``workspace`` then holds fp32 partial accumulators
    (``num_seqs * H * splits * d``) and fp32 (max, sum) pairs (``num_seqs * H * splits * 2``).
    ``token_is_seq``: the caller vouches that ``cu_q[i] == i`` for every sequence (a batch of
    single tokens), which spares the matrix-core kernel a dependent load.  ``slopes``: as in
    ``attn_prefill``."""
    H, KV, d = num_heads, num_kv_heads, head_dim
    n_seqs = _attn_common(q, k_pages, v_pages, block_table, cu_q, ctx_lens, out, H, KV, d)
    sl = _slopes_ptr(slopes, H, q)
    if token_is_seq and seq_ids is not None:
        raise KernelError("attn_decode: token_is_seq is for batches where every sequence decodes")
    if seq_ids is not None:
        _check(seq_ids, "seq_ids", I32, (None,))
        if seq_ids.shape[0] < num_seqs:
            raise KernelError("attn_decode: seq_ids shorter than num_seqs")
    elif num_seqs > n_seqs:
        raise KernelError("attn_decode: more sequences than block-table rows")
    nb, _, bs, _ = k_pages.shape
    if not 1 <= splits <= 64:
        raise KernelError(f"attn_decode: 1 to 64 cuts of the key range, got {splits}")
    pa = pm = None
    if splits > 1:
        if workspace is None:
            raise KernelError("attn_decode: splits > 1 need a workspace")
        pa, pm = workspace[0], workspace[1]
        _check(pa, "workspace[0]", F32)
        _check(pm, "workspace[1]", F32)
        if pa.numel() < num_seqs * H * splits * d or pm.numel() < num_seqs * H * splits * 2:
            raise KernelError("attn_decode: workspace too small")
    if not attention_on_matrix_cores(q.dtype, bs):
        f = _fn("attn_generic", "kvf_attn_generic_decode",
                [c_int] + [c_void_p] * 10 + [c_int] * 12 + [c_float, c_void_p, c_void_p])
        _ok(f(_tcode(q.dtype), q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
              block_table.data_ptr(), seq_ids.data_ptr() if seq_ids is not None else None,
              None if token_is_seq else cu_q.data_ptr(), ctx_lens.data_ptr(), out.data_ptr(),
              pa.data_ptr() if pa is not None else None, pm.data_ptr() if pm is not None else None,
              num_seqs, H, KV, d, bs, nb, block_table.shape[1], q.stride(0), out.stride(0),
              int(window), n_seqs, int(splits), float(scale), sl, _stream()), "attn_generic_decode")
        return
    f = _fn("attn_mfma", "kvf_attn_mfma_decode",
            [c_void_p] * 10 + [c_int] * 12 + [c_float, c_void_p, c_void_p])
    _ok(f(q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(),
          seq_ids.data_ptr() if seq_ids is not None else None,
          None if token_is_seq else cu_q.data_ptr(),
          ctx_lens.data_ptr(), out.data_ptr(), pa.data_ptr() if pa is not None else None,
          pm.data_ptr() if pm is not None else None, num_seqs, H, KV, d, bs, nb,
          block_table.shape[1], q.stride(0), out.stride(0), int(window), n_seqs, int(splits),
          float(scale), sl, _stream()), "attn_mfma_decode")


# ------------------------------------------------------------------------------ sampling
GREEDY_SPLIT_MAX = 16


def sample_work_size(rows: int) -> int:
    """int32 elements of the ``work`` tensor that lets ``sample`` read greedy rows with several
    workgroups each: tickets, then the best value and index of every chunk."""
    return rows * (1 + 2 * GREEDY_SPLIT_MAX)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor | None,
           top_p: torch.Tensor | None, u: torch.Tensor, tokens: torch.Tensor,
           u_step: torch.Tensor | None = None, work: torch.Tensor | None = None) -> None:
    """One token per row of fp32 ``logits``: argmax where ``temperature == 0``, otherwise the
    inverse CDF of the processed distribution at ``u``.  With ``u_step`` (one int32 on the
    device) ``u`` holds several rows of numbers, ``[steps, row stride]``, and row ``u_step[0]``
    is used: a captured launch then serves several decode steps.  ``work`` (int32,
    ``sample_work_size(rows)`` elements, zero when first handed over, not shared with a launch
    that may overlap): greedy rows are then read by several workgroups each, about as many as
    fill the chip; the result is the same."""
    _check(logits, "logits", F32, (None, None), contiguous=False)
    if logits.stride(1) != 1:
        raise KernelError("sample: logits rows must be dense")
    r, v = logits.shape
    _check(temperature, "temperature", F32, (r,))
    stride = 0
    if u_step is None:
        _check(u, "u", F32, (r,))
    else:
        _check(u_step, "u_step", I32, (1,))
        _check(u, "u", F32, (None, None))
        stride = u.shape[1]
        if stride < r:
            raise KernelError("sample: rows of u are shorter than the batch")
    _check(tokens, "tokens", I32, (r,))
    if top_k is not None:
        _check(top_k, "top_k", I32, (r,))
    if top_p is not None:
        _check(top_p, "top_p", F32, (r,))
    splits = 1
    if work is not None:
        _check(work, "work", I32, (None,))
        if work.shape[0] < sample_work_size(r):
            raise KernelError("sample: work is smaller than sample_work_size(rows)")
        # about one workgroup per compute unit, each with at least 4096 logits
        splits = max(1, min(GREEDY_SPLIT_MAX, compute_units(logits.device) // r, v // 4096))
    f = _fn("sampling", "kvf_sample",
            [c_void_p, c_int, c_int, c_int] + [c_void_p] * 5 + [c_int, c_void_p, c_void_p, c_int,
                                                                c_void_p])
    _ok(f(logits.data_ptr(), logits.stride(0) if r > 1 else v, r, v, temperature.data_ptr(),
          top_k.data_ptr() if top_k is not None else None,
          top_p.data_ptr() if top_p is not None else None, u.data_ptr(),
          u_step.data_ptr() if u_step is not None else None, stride, tokens.data_ptr(),
          work.data_ptr() if work is not None else None, splits, _stream()), "sample")


def decode_advance(sampled: torch.Tensor, token_ids: torch.Tensor, positions: torch.Tensor,
                   ctx_lens: torch.Tensor, ring: torch.Tensor, counter: torch.Tensor) -> None:
    """After a step of single tokens: ``ring[counter[0]] = sampled``; for every sequence with a
    context, the sampled token becomes the next input (``token_ids``), ``positions`` and
    ``ctx_lens`` move on by one; ``counter[0] += 1``.  All on the device, in stream order."""
    r = sampled.shape[0]
    for t, name in ((sampled, "sampled"), (token_ids, "token_ids"), (positions, "positions"),
                    (ctx_lens, "ctx_lens")):
        _check(t, name, I32, (r,))
    _check(ring, "ring", I32, (None, None))
    _check(counter, "counter", I32, (1,))
    if ring.shape[1] < r:
        raise KernelError("decode_advance: rows of the ring are shorter than the batch")
    f = _fn("sampling", "kvf_decode_advance", [c_void_p] * 6 + [c_int] * 3 + [c_void_p])
    _ok(f(sampled.data_ptr(), token_ids.data_ptr(), positions.data_ptr(), ctx_lens.data_ptr(),
          ring.data_ptr(), counter.data_ptr(), r, ring.shape[1], ring.shape[0], _stream()),
        "decode_advance")
