"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes and
compared with the entry point it is a variant of, on two calls in a row."""
import ctypes
import math
from ctypes import c_float, c_int, c_size_t, c_void_p

import pytest
import torch

from braidinfer_amd.csrc import build as _build

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
_P = c_void_p
SCRATCH_FLOATS = 1 << 20        # BR_NO_ALLOC_SCRATCH_FLOATS in csrc/no_alloc.h


def _case(lens, nq, nkv, hd, seed):
    """Sequences of the given lengths scattered over shuffled pages: q, cache, table, slots, ctx."""
    g = torch.Generator().manual_seed(seed)
    page = 64
    n_pages = sum(-(-n // page) for n in lens) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    cache = torch.full((n_pages, 2, nkv, page, hd), 3.0, dtype=torch.bfloat16, device=DEV)
    table = torch.full((len(lens) + 1, max(-(-n // page) for n in lens) + 1), -1, dtype=torch.int32)
    for b, n in enumerate(lens):
        for i in range(-(-n // page)):
            pg = order.pop()
            table[b + 1, i] = pg
            m = min(page, n - i * page)
            cache[pg, 0, :, :m] = torch.randn(nkv, m, hd, generator=g).to(torch.bfloat16).to(DEV)
            cache[pg, 1].view(nkv, hd, page)[:, :, :m] = torch.randn(nkv, hd, m, generator=g).to(torch.bfloat16).to(DEV)
    B = len(lens)
    q = torch.randn(B, nq * hd, generator=g).to(torch.bfloat16).to(DEV)
    slots = torch.arange(1, B + 1, dtype=torch.int32, device=DEV)
    ctx = torch.tensor(lens, dtype=torch.int32, device=DEV)
    return q, cache, table.to(DEV), slots, ctx


def _entry_points():
    lib = _build.load("attention_bf16")
    head = [_P, c_size_t, _P, _P, _P, _P, c_int, _P] + [c_int] * 6 + [c_float, c_int]
    tail = [c_int, c_int, _P, _P, c_int, _P]
    old, new = lib.br_attn_decode_bf16, lib.br_attn_decode_bf16_no_alloc
    old.argtypes, old.restype = head + [_P, _P] + tail, c_int
    new.argtypes, new.restype = head + tail, c_int
    return old, new


def _run(old, new, lens, nq, nkv, hd, nsplit, window, seed):
    q, cache, table, slots, ctx = _case(lens, nq, nkv, hd, seed)
    B = len(lens)
    stream = _P(torch.cuda.current_stream().cuda_stream)
    p = lambda t: _P(t.data_ptr())
    head = (p(q), nq * hd, None, p(slots), p(ctx), p(table), table.shape[1], p(cache), B, nq, nkv, hd, 64, window,
            1 / math.sqrt(hd), nsplit)
    want = torch.full((B, nq * hd), 9.0, dtype=torch.bfloat16, device=DEV)
    part_o = torch.empty(B * nq * nsplit * hd, device=DEV)
    part_ml = torch.empty(B * nq * nsplit * 2, device=DEV)
    rc = old(*head[:2], p(want), *head[3:], p(part_o), p(part_ml), 0, 0, None, None, 1, stream)
    assert rc == 0
    got = torch.full((B, nq * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    print(f"no_alloc case: lens {lens} nq {nq} nkv {nkv} hd {hd} nsplit {nsplit} window {window}", flush=True)
    rc = new(*head[:2], p(got), *head[3:], 0, 0, None, None, 1, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got, want)
    return got


def test_no_alloc_decode_attention_twice_in_a_row_the_second_smaller():
    old, new = _entry_points()
    big = _run(old, new, [700, 64, 1, 333, 2000, 129, 65, 1024], 32, 8, 128, 4, 0, seed=1)
    small = _run(old, new, [130, 900, 5], 8, 2, 64, 2, 100, seed=2)      # what the first call left in the scratch is still there
    assert big.abs().max() > 0 and small.abs().max() > 0
    _run(old, new, [70, 200], 6, 3, 32, 3, 0, seed=3)                    # the kernel that reads operands straight from the cache
    _run(old, new, [300], 4, 4, 64, 1, 0, seed=4)                        # one run: no scratch at all


def test_no_alloc_refuses_what_its_scratch_cannot_hold():
    old, new = _entry_points()
    q, cache, table, slots, ctx = _case([100] * 4, 32, 8, 128, seed=5)
    B, nq, hd, nsplit = 4, 32, 128, 80          # 4 * 32 * 80 * 130 floats > 2^20
    assert B * nq * nsplit * (hd + 2) > SCRATCH_FLOATS
    out = torch.full((B, nq * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    p = lambda t: _P(t.data_ptr())
    rc = new(p(q), nq * hd, p(out), p(slots), p(ctx), p(table), table.shape[1], p(cache), B, nq, 8, hd, 64, 0,
             1 / math.sqrt(hd), nsplit, 0, 0, None, None, 1, _P(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == 3 and bool((out == 7.0).all())          # BR_TOO_LARGE, and nothing was launched
