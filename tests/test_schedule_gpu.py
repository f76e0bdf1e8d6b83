"""The device-side scheduler on its own, through the C ABI: the workspace sba_build_schedule fills is
read back and compared with a plain Python model of what it should hold -- every 128-row query
tile and every 128-key tile of every document exactly once, the key tiles in two groups (first the
tiles that many queries follow, then every tile of a document of at most 256 tokens and the last
tile of every longer one), table areas that do not overlap, and the header counts the kernels and
the launch bounds rely on."""
import ctypes
import random

import pytest
import torch

from stickbreaking_attention import _native as nat
from stickbreaking_attention import _ops
from tests import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HDR, TILE_WORDS = 16, 8


def _schedule(lengths, tokens, fixed_batch=0):
    lib = nat.load()
    if fixed_batch:
        prob = nat.SbaProblem(nat.SBA_BF16, 64, 2, fixed_batch, tokens, 0, tokens, nat.FLAG_FIXED_LENGTH, 0.125, None)
        n_docs, rows = fixed_batch, fixed_batch * tokens
    else:
        cu = helpers.cu_from_lengths(lengths, device=DEV)
        prob = nat.SbaProblem(nat.SBA_BF16, 64, 2, 1, tokens, cu.numel(), max(lengths + [1]), 0, 0.125, cu.data_ptr())
        n_docs, rows = len(lengths), tokens
    nbytes = lib.sba_schedule_bytes(ctypes.byref(prob))
    sched = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    nat.check(lib.sba_build_schedule(ctypes.byref(prob), sched.data_ptr(), sched.numel(), nat.stream_ptr(torch.device(DEV))),
              "sba_build_schedule")
    torch.cuda.synchronize()
    words = sched.view(torch.int32).cpu().tolist()
    n_q_max = rows // 128 + n_docs + 1
    hdr = words[:HDR]
    tile = lambda base, i: tuple(words[base + TILE_WORDS * i: base + TILE_WORDS * i + 5])   # tok_start, doc_len, idx, batch, tab_base
    q_tiles = [tile(HDR, i) for i in range(hdr[1])]
    kv_tiles = [tile(HDR + TILE_WORDS * n_q_max, i) for i in range(hdr[2])]
    return hdr, q_tiles, kv_tiles, rows


def _check(lengths, tokens, fixed_batch=0):
    hdr, q_tiles, kv_tiles, rows = _schedule(lengths, tokens, fixed_batch)
    docs = [(b * 0, tokens, b) for b in range(fixed_batch)] if fixed_batch else []
    if not fixed_batch:
        start = 0
        for n in lengths:
            docs.append((start, n, 0))
            start += n
    cdiv = lambda a, b: -(-a // b)
    tail = lambda n: cdiv(n, 128) if n <= 256 else 1
    assert hdr[0] == 0
    assert hdr[1] == sum(cdiv(n, 128) for _, n, _ in docs)
    assert hdr[2] == sum(cdiv(n, 128) for _, n, _ in docs)
    n_long = sum(cdiv(n, 128) - tail(n) for _, n, _ in docs)
    assert hdr[7] == n_long
    assert hdr[3] == sum(_ops.table_entries(n) for _, n, _ in docs)
    assert hdr[4] == (0 if not docs else (tokens if fixed_batch else sum(lengths)))
    assert hdr[6] == max([n for _, n, _ in docs] + [0])
    # the bound the backward sizes its first-group launch with
    assert n_long <= rows // 128
    # every tile of every document exactly once
    want = sorted((s, n, i, b) for s, n, b in docs for i in range(cdiv(n, 128)))
    assert sorted(t[:4] for t in q_tiles) == want
    assert sorted(t[:4] for t in kv_tiles) == want
    # groups of the key-tile list
    for pos, (s, n, i, b, _) in enumerate(kv_tiles):
        in_tail = i >= cdiv(n, 128) - tail(n)
        assert in_tail == (pos >= n_long), (pos, n, i)
    # table areas: one base per document, areas disjoint and inside the total
    areas = {}
    for s, n, i, b, base in q_tiles + kv_tiles:
        assert areas.setdefault((s, b), (base, n)) == (base, n)
    spans = sorted((base, base + _ops.table_entries(n)) for base, n in areas.values())
    for (a0, a1), (b0, b1) in zip(spans, spans[1:]):
        assert a1 <= b0
    assert not spans or (spans[0][0] >= 0 and spans[-1][1] <= hdr[3])
    # longest documents first (packed input with few enough documents to be ranked)
    if not fixed_batch and len(lengths) <= 4096:
        order = []
        for t in q_tiles:
            if (t[0], t[1]) not in order:
                order.append((t[0], t[1]))
        assert [n for _, n in order] == sorted((n for _, n in order), reverse=True)


@pytest.mark.parametrize("seed", range(6))
def test_random_documents(seed):
    rng = random.Random(seed)
    kind = seed % 3
    if kind == 0:
        lengths = [rng.randint(0, 700) for _ in range(rng.randint(1, 40))]
    elif kind == 1:
        lengths = [rng.choice([0, 1, 31, 32, 33, 127, 128, 129, 255, 256, 257, 383, 384, 385, 1000]) for _ in range(60)]
    else:
        lengths = [rng.randint(1, 40) for _ in range(700)]       # more documents than scheduler threads
    tail_tokens = rng.choice([0, 0, 5, 300])
    _check(lengths, sum(lengths) + tail_tokens)


def test_no_documents_and_fixed_length():
    _check([], 256)
    _check([], 2048, fixed_batch=3)
    _check([], 200, fixed_batch=5)
