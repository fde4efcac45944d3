"""The sampling entry point that allocates nothing (``kvf_sample_static``, declared in
``kvforge_amd/csrc/sampling_static.h``) against ``kvf_sample`` with a work tensor the caller
brings: called through ``ctypes``, twice in a row, the second time with a smaller input, so that
what the first call left in the library's own work memory is what the second one meets."""

from __future__ import annotations

import ctypes
from ctypes import c_int, c_void_p

import pytest
import torch

from kvforge_amd.kernels import library

pytestmark = pytest.mark.gpu

MAX_ROWS = 1024      # KVF_SAMPLE_STATIC_MAX_ROWS
SPLITS = 16


def entry_points():
    lib = ctypes.CDLL(library.build_module("sampling"))
    plain = lib.kvf_sample
    plain.argtypes = [c_void_p, c_int, c_int, c_int] + [c_void_p] * 5 + [c_int, c_void_p, c_void_p,
                                                                         c_int, c_void_p]
    plain.restype = c_int
    static = lib.kvf_sample_static
    static.argtypes = [c_void_p, c_int, c_int, c_int] + [c_void_p] * 5 + [c_int, c_void_p, c_void_p]
    static.restype = c_int
    return plain, static


def case(rows, vocab, seed, drawn_rows=()):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(rows, vocab, generator=g).cuda()
    # equal maxima in some rows: the lowest index has to win in both entry points
    for r in range(0, rows, 3):
        i, j = sorted(torch.randint(0, vocab, (2,), generator=g).tolist())
        logits[r, i] = logits[r, j] = 9.0
    temperature = torch.zeros(rows)
    for r in drawn_rows:
        temperature[r] = 0.8
    u = torch.rand(rows, generator=g)
    return logits, temperature.cuda(), u.cuda()


def run_both(plain, static, logits, temperature, u):
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    work = torch.zeros(rows * (1 + 2 * SPLITS), dtype=torch.int32, device="cuda")
    splits = max(1, min(SPLITS, 256 // rows, vocab // 4096))
    rc = plain(logits.data_ptr(), logits.stride(0), rows, vocab, temperature.data_ptr(), None, None,
               u.data_ptr(), None, 0, want.data_ptr(), work.data_ptr(), splits, stream)
    assert rc == 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    rc = static(logits.data_ptr(), logits.stride(0), rows, vocab, temperature.data_ptr(), None, None,
                u.data_ptr(), None, 0, got.data_ptr(), stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before      # the device's free memory did not move
    return got.cpu(), want.cpu()


def test_static_entry_point_equals_the_one_with_a_work_tensor_twice_in_a_row():
    plain, static = entry_points()
    # first call: 12 rows of a large vocabulary (16 workgroups a row), two rows draw
    logits, temperature, u = case(12, 128256, 0, drawn_rows=(4, 9))
    got, want = run_both(plain, static, logits, temperature, u)
    assert got.tolist() == want.tolist()
    greedy = [r for r in range(12) if r not in (4, 9)]
    assert got[greedy].tolist() == logits[greedy].argmax(-1).cpu().tolist()
    # second call, smaller: fewer rows and a smaller vocabulary, hence another layout of the same
    # work memory (other row count, other number of chunks) over what the first call left
    logits, temperature, u = case(5, 50000, 1)
    got, want = run_both(plain, static, logits, temperature, u)
    assert got.tolist() == want.tolist() == logits.argmax(-1).cpu().tolist()
    # and once more at the first size
    logits, temperature, u = case(12, 128256, 2)
    got, want = run_both(plain, static, logits, temperature, u)
    assert got.tolist() == want.tolist()


def test_static_entry_point_refuses_more_rows_than_its_memory_holds():
    _, static = entry_points()
    rows = MAX_ROWS + 1
    logits = torch.zeros(rows, 8, device="cuda")
    temperature = torch.zeros(rows, device="cuda")
    tokens = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    rc = static(logits.data_ptr(), 8, rows, 8, temperature.data_ptr(), None, None,
                temperature.data_ptr(), None, 0, tokens.data_ptr(),
                torch.cuda.current_stream().cuda_stream)
    assert rc == 1          # hipErrorInvalidValue
    torch.cuda.synchronize()
    assert tokens.eq(-7).all()
