"""CPU-only checks of the boundary: the shared library loads, exports every symbol the header
declares, sizes workspaces sensibly and rejects bad arguments without touching a GPU."""
import ctypes
import os
import re

import pytest
import torch

from stickbreaking_attention import _native as nat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "sba.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sba_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = nat.load()
    syms = header_symbols()
    assert len(syms) >= 11
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in include/sba.h but not exported"
    assert sorted(nat.EXPORTS) == syms
    assert lib.sba_version() == 213


def problem(**kw):
    base = dict(dtype=1, head_dim=128, heads=32, batch=1, tokens=16384, n_docs=8, max_doc_len=4096,
                flags=0, inv_temp=0.0884, cu_seqlens=0x1000)
    base.update(kw)
    return nat.SbaProblem(*[base[f[0]] for f in nat.SbaProblem._fields_])


def _entries(L):
    nb = -(-L // 32)
    return sum(32 * nb - 32 * b for b in range(nb)) + 32 * nb      # rows at or below each 32-key block (rounded up to 32), plus one per row


def test_workspace_sizes():
    lib = nat.load()
    p = problem()
    sched = lib.sba_schedule_bytes(ctypes.byref(p))
    # two tile lists (32 B per tile): query tiles and key tiles, each bounded by tokens/128 + docs
    assert 32 * (128 + 8 + 128 + 8) <= sched <= 32 * (128 + 128 + 32) + 1024
    # no lengths: four documents of max_doc_len = 4096 tokens are the worst split of 16384 tokens (+ 31 per document of rounding)
    # (+ 256 bytes at the end of every table: the work counters of the persistent launches)
    assert lib.sba_table_bytes(ctypes.byref(p)) == 32 * (4 * _entries(4096) + _entries(31 * 8)) * 4 + 256
    # exact, from host lengths (the headline workload's documents): under 100 MiB
    lengths = [4026, 2261, 1563, 566, 1189, 615, 3465, 2699]
    arr = (ctypes.c_int64 * len(lengths))(*lengths)
    exact = lib.sba_table_bytes_for_lengths(ctypes.byref(p), arr, len(lengths))
    assert exact == 32 * sum(_entries(n) for n in lengths) * 4 + 256
    assert exact < 100 * 2 ** 20 < lib.sba_table_bytes(ctypes.byref(p))
    # a length beyond the token count is refused
    bad = (ctypes.c_int64 * 1)(20000)
    assert lib.sba_table_bytes_for_lengths(ctypes.byref(p), bad, 1) == 0
    pf = problem(batch=4, heads=16, tokens=2048, n_docs=0, max_doc_len=2048, head_dim=64,
                 flags=nat.FLAG_FIXED_LENGTH, cu_seqlens=None)
    assert lib.sba_table_bytes(ctypes.byref(pf)) == 16 * 4 * _entries(2048) * 4 + 256


def test_undersized_workspaces_are_refused_on_the_host():
    """Every workspace travels with its size; what the host can check comes back as SBA_E_WORKSPACE
    (-6) before anything is launched (no GPU is touched: argument checks come first)."""
    lib = nat.load()
    p = problem()
    need = lib.sba_schedule_bytes(ctypes.byref(p))
    v = nat.SbaView(0x1000, 0, 128 * 16384, 128)
    r = nat.SbaView(0x1000, 0, 16384, 1)
    vs = [ctypes.byref(x) for x in (v, v, v, v, r)]
    sched = ctypes.c_void_p(0x1000)
    assert lib.sba_build_schedule(ctypes.byref(p), sched, need - 1, None) == -6
    assert lib.sba_varlen_fwd(ctypes.byref(p), sched, need - 1, *vs, None, 0, None) == -6
    assert lib.sba_varlen_fwd(ctypes.byref(p), sched, need, *vs, ctypes.c_void_p(0x1000), 0, None) in (-6, -7)
    assert lib.sba_varlen_fwd_weights(ctypes.byref(p), sched, need, *vs, None, 0, ctypes.c_void_p(0x1000), 1024, None) == -6
    bw = [ctypes.byref(x) for x in (v, v, v, v, r)]
    outs = [ctypes.byref(v)] * 3
    assert lib.sba_varlen_bwd(ctypes.byref(p), sched, need - 1, *bw, ctypes.c_void_p(0x1000),
                              ctypes.c_void_p(0x1000), 1 << 30, *outs, None) == -6
    # fixed-length: the table need is known on the host
    pf = problem(batch=4, heads=16, tokens=2048, n_docs=0, max_doc_len=2048, head_dim=64,
                 flags=nat.FLAG_FIXED_LENGTH, cu_seqlens=None)
    needf = lib.sba_schedule_bytes(ctypes.byref(pf))
    tbl = lib.sba_table_bytes(ctypes.byref(pf))
    vf = nat.SbaView(0x1000, 16 * 2048 * 64, 2048 * 64, 64)
    rf = nat.SbaView(0x1000, 16 * 2048, 2048, 1)
    vsf = [ctypes.byref(x) for x in (vf, vf, vf, vf, rf)]
    assert lib.sba_attn_fwd(ctypes.byref(pf), sched, needf, *vsf, ctypes.c_void_p(0x1000), tbl - 4, None) == -6
    assert lib.sba_attn_bwd(ctypes.byref(pf), sched, needf, *vsf, ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1000),
                            tbl - 4, *[ctypes.byref(vf)] * 3, None) == -6


def test_table_only_forward_checks_its_arguments():
    """SBA_TABLE_ONLY: the stick table is required, v / o / rem may be null views, the weights output
    cannot be combined with it; the table of the fixed-length op is still size-checked."""
    lib = nat.load()
    p = problem(flags=nat.FLAG_PRODUCT_SPACE | nat.FLAG_TABLE_ONLY)
    need = lib.sba_schedule_bytes(ctypes.byref(p))
    v = nat.SbaView(0x1000, 0, 128 * 16384, 128)
    null = nat.SbaView(None, 0, 0, 0)
    sched = ctypes.c_void_p(0x1000)
    args = [ctypes.byref(x) for x in (v, v, null, null, null)]
    assert lib.sba_varlen_fwd(ctypes.byref(p), sched, need, *args, None, 0, None) == -1              # no table
    assert lib.sba_varlen_fwd(ctypes.byref(p), sched, need, *[ctypes.byref(x) for x in (v, null, null, null, null)],
                              ctypes.c_void_p(0x1000), 1 << 30, None) == -1                             # k missing
    # everything the host can check is fine: the call gets as far as looking for a gfx950 device
    # (-7 here, where there is none) without having asked for v, o or rem
    # (only where no GPU could take the made-up pointers seriously)
    if not torch.cuda.is_available():
        assert lib.sba_varlen_fwd(ctypes.byref(p), sched, need, *args, ctypes.c_void_p(0x1000), 1 << 30, None) == -7
    pf = problem(batch=4, heads=16, tokens=2048, n_docs=0, max_doc_len=2048, head_dim=64,
                 flags=nat.FLAG_FIXED_LENGTH | nat.FLAG_TABLE_ONLY, cu_seqlens=None)
    vf = nat.SbaView(0x1000, 16 * 2048 * 64, 2048 * 64, 64)
    argsf = [ctypes.byref(x) for x in (vf, vf, null, null, null)]
    assert lib.sba_attn_fwd(ctypes.byref(pf), sched, lib.sba_schedule_bytes(ctypes.byref(pf)), *argsf,
                            ctypes.c_void_p(0x1000), lib.sba_table_bytes(ctypes.byref(pf)) - 4, None) == -6


@pytest.mark.parametrize("kw,code", [
    (dict(head_dim=50), -2), (dict(head_dim=512), -2), (dict(dtype=7), -3), (dict(dtype=2, head_dim=50), -2), (dict(heads=0), -4), (dict(batch=2), -4),
    (dict(cu_seqlens=None), -1),
])
def test_bad_problems_are_rejected_on_the_host(kw, code):
    lib = nat.load()
    p = problem(**kw)
    assert lib.sba_schedule_bytes(ctypes.byref(p)) == 0
    assert lib.sba_build_schedule(ctypes.byref(p), ctypes.c_void_p(0x1000), 1 << 20, None) == code
    v = nat.SbaView(0x1000, 0, 128 * 16384, 128)
    r = nat.SbaView(0x1000, 0, 16384, 1)
    assert lib.sba_varlen_fwd(ctypes.byref(p), ctypes.c_void_p(0x1000), 1 << 20, ctypes.byref(v), ctypes.byref(v),
                              ctypes.byref(v), ctypes.byref(v), ctypes.byref(r), None, 0, None) == code


def test_misaligned_stride_and_null_views_are_rejected():
    lib = nat.load()
    p = problem()
    good = nat.SbaView(0x1000, 0, 128 * 16384, 128)
    bad = nat.SbaView(0x1000, 0, 128 * 16384 + 2, 128)
    null = nat.SbaView(None, 0, 0, 0)
    r = nat.SbaView(0x1000, 0, 16384, 1)
    args = lambda q: (ctypes.byref(p), ctypes.c_void_p(0x1000), 1 << 20, ctypes.byref(q), ctypes.byref(good),
                      ctypes.byref(good), ctypes.byref(good), ctypes.byref(r), None, 0, None)
    assert lib.sba_varlen_fwd(*args(bad)) == -5
    assert lib.sba_varlen_fwd(*args(null)) == -1
    assert b"16-byte" in lib.sba_error_string(-5)


def test_ops_fail_loudly_without_a_gpu():
    from stickbreaking_attention import sb_attn, sb_attn_varlen
    q = torch.zeros(2, 16, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="MI355X"):
        sb_attn_varlen(q, q, q, torch.tensor([16], dtype=torch.int32), 16, zero_start=False)
    with pytest.raises(RuntimeError, match="MI355X"):
        sb_attn(q[None], q[None], q[None])


def test_missing_library_raises(monkeypatch):
    monkeypatch.setattr(nat, "_lib", None)
    monkeypatch.setattr(nat, "LIB_PATH", "/nonexistent/libsba.so")
    with pytest.raises(RuntimeError, match="libsba.so not found"):
        nat.load()


@pytest.mark.parametrize("kw", [
    dict(),                                                           # C3
    dict(head_dim=64, tokens=16384, n_docs=207, max_doc_len=256),     # many short documents
    dict(tokens=65536, n_docs=7, max_doc_len=32768),
    dict(tokens=300, n_docs=1, max_doc_len=300, heads=2),
    dict(tokens=130, n_docs=0, max_doc_len=130, heads=3),
    dict(batch=4, heads=16, tokens=2048, n_docs=0, max_doc_len=2048, head_dim=64, fixed=True),
    dict(batch=2, heads=7, tokens=500, n_docs=0, max_doc_len=500, head_dim=64, fixed=True),
])
def test_python_workspace_formula_matches_the_library(kw):
    # _ops.workspace_sizes restates sba_schedule_bytes / sba_table_bytes so that buffer sizes can
    # be computed while torch.compile traces; the two must never drift apart.
    from stickbreaking_attention import _ops
    lib = nat.load()
    kw = dict(kw)
    fixed = kw.pop("fixed", False)
    if fixed:
        kw.update(flags=nat.FLAG_FIXED_LENGTH, cu_seqlens=None)
    p = problem(**kw)
    sched, table = _ops.workspace_sizes(fixed, p.batch, p.heads, p.tokens, p.n_docs, p.max_doc_len)
    assert sched == lib.sba_schedule_bytes(ctypes.byref(p))
    assert 4 * table == lib.sba_table_bytes(ctypes.byref(p))


def test_operators_are_registered_under_the_upstream_names():
    import torch
    import stickbreaking_attention  # noqa: F401
    for name in ("varlen_fwd", "varlen_bwd", "attn_fwd", "attn_bwd"):
        assert hasattr(torch.ops.stickbreaking_attention, name)


def test_host_copy_of_cu_seqlens_is_cached_per_tensor_object():
    """Host logic only: the values of one cu_seqlens tensor are fetched once and reused until the
    tensor is modified in place or another tensor arrives (upstream reads cu_seqlens[0] back on every
    call for its assertion, sb_varlen/__init__.py:73)."""
    import torch
    from stickbreaking_attention import _ops, sb_varlen
    _ops.release_workspaces()
    cu = torch.tensor([0, 5, 9], dtype=torch.int32)
    assert sb_varlen._starts_at_zero(cu)
    assert _ops._host_cu_cache[-1][0]() is cu and _ops._host_cu_cache[-1][2] == (0, 5, 9)
    n = len(_ops._host_cu_cache)
    assert sb_varlen._starts_at_zero(cu) and len(_ops._host_cu_cache) == n       # served from the cache
    stripped = sb_varlen._strip_leading_zero(cu)
    assert _ops.host_cu_seqlens(stripped, allow_sync=False) == (5, 9)              # carried over to the view
    same_values = torch.tensor([0, 5, 9], dtype=torch.int32)
    assert sb_varlen._starts_at_zero(same_values) and _ops._host_cu_cache[-1][0]() is same_values
    same_values[0] = 2                                                             # in-place write: new version
    assert not sb_varlen._starts_at_zero(same_values)
    assert _ops.host_cu_seqlens(same_values) == (2, 5, 9)
    assert not sb_varlen._starts_at_zero(torch.tensor([1, 4]))
    with pytest.raises(ValueError):
        _ops._doc_lengths((5, 3), 10)          # not monotone
    with pytest.raises(ValueError):
        _ops._doc_lengths((5, 12), 10)         # beyond the token count
    assert _ops._doc_lengths((5, 5, 9), 10) == (5, 0, 4)


def test_leading_zero_check_works_on_inference_tensors():
    """Tensors created under torch.inference_mode() have no version counter: the check must read
    the values every time instead of raising."""
    import torch
    from stickbreaking_attention import _ops, sb_varlen
    _ops.release_workspaces()
    with torch.inference_mode():
        cu = torch.tensor([0, 5, 9], dtype=torch.int32)
        bad = torch.tensor([3, 5, 9], dtype=torch.int32)
        assert sb_varlen._starts_at_zero(cu) and sb_varlen._starts_at_zero(cu)
        assert not sb_varlen._starts_at_zero(bad)
    assert sb_varlen._starts_at_zero(cu)          # also outside the mode, on the inference tensor
    assert all(e[0]() is not cu for e in _ops._host_cu_cache)


def test_python_table_formula_with_lengths_matches_the_library():
    from stickbreaking_attention import _ops
    lib = nat.load()
    p = problem()
    lengths = [4026, 2261, 1563, 566, 1189, 615, 3465, 2699, 0, 1, 33]
    p.tokens = sum(lengths)
    arr = (ctypes.c_int64 * len(lengths))(*lengths)
    _, table = _ops.workspace_sizes(False, 1, p.heads, p.tokens, len(lengths), 0, lengths)
    assert 4 * table == lib.sba_table_bytes_for_lengths(ctypes.byref(p), arr, len(lengths))


# ---------------------------------------------------------------------------------------------
# Launch geometry: every tile descriptor a workgroup can read lies inside the schedule workspace.
# The forward, dq and dk/dv kernels fetch the descriptor of their slot BEFORE they compare the slot
# with the true length of the list (one round trip to memory instead of two), so the grids must
# stay inside the room of the lists whatever the documents are.  The library exports the grids it
# would launch (sba_launch_geometry, the same functions the launchers call).
# ---------------------------------------------------------------------------------------------
def _geometry(**kw):
    lib = nat.load()
    p = problem(**kw)
    g = nat.SbaGeometry()
    rc = lib.sba_launch_geometry(ctypes.byref(p), ctypes.byref(g))
    assert rc == 0, rc
    assert g.schedule_words * 4 == lib.sba_schedule_bytes(ctypes.byref(p))
    return g


def _check_geometry(g, n_docs):
    # the two lists and the per-document arrays behind them fit the workspace
    assert g.query_list_word == 16 and g.tile_words == 8
    assert g.key_list_word == g.query_list_word + g.tile_words * g.query_list_tiles
    lists_end = g.key_list_word + g.tile_words * g.key_list_tiles
    assert lists_end + 6 * n_docs + 2 <= g.schedule_words
    # query-tile-owned kernels: slots 0 .. fwd_tiles-1 of the query list
    assert 0 <= g.fwd_tiles <= g.query_list_tiles and 0 <= g.dq_tiles <= g.query_list_tiles
    # dk/dv main kernel: slots 0 .. dkdv_main_tiles-1 of the key list, read unconditionally
    assert 0 <= g.dkdv_main_tiles <= g.key_list_tiles
    assert g.key_list_word + g.tile_words * g.dkdv_main_tiles <= g.schedule_words
    # (the tail kernel checks its slot against the true list length before reading: any grid is safe)
    assert g.dkdv_tail_tiles >= 0


def _tiles(lengths, rows):
    return sum(-(-n // rows) for n in lengths)


def _tail_tiles(n):
    nkv = -(-n // 128)
    return nkv if n <= 2 * 128 else 1


def test_every_launch_stays_inside_the_schedule_workspace():
    import random
    rng = random.Random(20261125)
    cases = [(0, 0, 0), (128, 0, 0), (128, 1, 128), (1, 1, 1), (2112, 10, 2112), (16384, 8, 4096), (16384, 207, 256),
             (65536, 6, 32768), (5, 9, 1), (100, 300, 0), (4096, 1, 1), (4096, 1, 99999)]
    for _ in range(3000):
        tokens = rng.choice([rng.randint(0, 300), rng.randint(0, 5000), rng.randint(0, 70000)])
        n_docs = rng.choice([0, 1, rng.randint(0, 12), rng.randint(0, 400)])
        mdl = rng.choice([0, 1, rng.randint(0, max(tokens, 1)), tokens, tokens + 7])
        cases.append((tokens, n_docs, mdl))
    for tokens, n_docs, mdl in cases:
        for d in (32, 64, 128, 256):
            g = _geometry(tokens=tokens, n_docs=n_docs, max_doc_len=mdl, head_dim=d, heads=3)
            _check_geometry(g, n_docs)
            # what an earlier version launched at head_dim 128 (both bounds added, no clamp) does NOT stay inside:
            # the test must be able to tell the difference
    g = _geometry(tokens=2112, n_docs=10, max_doc_len=2112, head_dim=128, heads=3)
    assert g.long_tiles_bound + g.tail_tiles_bound > g.key_list_tiles >= g.dkdv_main_tiles
    # fixed length: batch documents of `tokens` tokens each
    for batch, tokens in [(1, 1), (4, 2048), (3, 500), (2, 16384), (7, 129)]:
        for d in (32, 64, 128, 256):
            g = _geometry(batch=batch, tokens=tokens, n_docs=0, max_doc_len=tokens, head_dim=d, heads=2,
                          flags=nat.FLAG_FIXED_LENGTH, cu_seqlens=None)
            _check_geometry(g, batch)
            assert g.fwd_tiles >= batch * -(-tokens // 128)


def test_launch_bounds_cover_every_split_into_documents():
    """The grids are upper bounds: whatever documents fill the token axis, their query tiles, key tiles
    and the two groups of the key-tile list fit what would be launched (no tile is ever dropped)."""
    import random
    rng = random.Random(7)
    for _ in range(1500):
        n_docs = rng.choice([1, 2, rng.randint(1, 10), rng.randint(1, 250)])
        mode = rng.random()
        if mode < 0.3: lengths = [rng.randint(0, 300) for _ in range(n_docs)]
        elif mode < 0.6: lengths = [rng.choice([0, 1, 127, 128, 129, 255, 256, 257, 384, 385, 1000]) for _ in range(n_docs)]
        else: lengths = [int(2 ** rng.uniform(0, 13)) for _ in range(n_docs)]
        tokens = sum(lengths) + rng.choice([0, 0, 5, 300])      # rows behind the last document are allowed
        mdl = max(lengths)
        for d in (64, 128, 256):
            g = _geometry(tokens=tokens, n_docs=n_docs, max_doc_len=mdl, head_dim=d, heads=1)
            assert _tiles(lengths, 128) <= g.fwd_tiles
            n_kv = _tiles(lengths, 128)
            assert n_kv <= g.key_list_tiles
            n_tail = sum(_tail_tiles(n) for n in lengths if n > 0)
            n_long = n_kv - n_tail
            assert n_long <= g.long_tiles_bound and n_tail <= g.tail_tiles_bound
            if d >= 128:
                assert n_kv <= g.dkdv_main_tiles           # one kernel takes both groups
            else:
                assert n_long <= g.dkdv_main_tiles and n_tail <= g.dkdv_tail_tiles


def test_scratch_tables_grow_instead_of_multiplying(monkeypatch):
    """Packed-document training changes the exact table size with every batch: the gradient table is one
    buffer per (device, stream, role) that only grows, not one allocation per size."""
    from types import SimpleNamespace
    from stickbreaking_attention import _ops
    monkeypatch.setattr(torch.cuda, "current_stream", lambda device=None: SimpleNamespace(cuda_stream=0))
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    _ops.release_workspaces()
    allocations = []
    real_empty = torch.empty

    def counting_empty(*a, **kw):
        t = real_empty(*a, **kw)
        allocations.append(t.numel())
        return t
    monkeypatch.setattr(torch, "empty", counting_empty)
    import random
    rng = random.Random(3)
    base = 32 * 90_000     # floats; sizes wander within +-12 % as document lengths change
    ptrs = set()
    for _ in range(20):
        n = int(base * rng.uniform(0.88, 1.12)) // 32 * 32
        t = _ops._scratch_table(n, torch.device("cpu"), "grad")
        assert t.numel() == n and t.data_ptr() % 16 == 0
        ptrs.add(t.data_ptr())
    assert len(allocations) <= 2 and len(ptrs) <= 2, allocations
    assert len(_ops._gtab_cache) == 1
    # another role (the rebuilt stick table) has a buffer of its own; a much larger request replaces, not adds
    _ops._scratch_table(1000, torch.device("cpu"), "stick")
    big = _ops._scratch_table(4 * base, torch.device("cpu"), "grad")
    assert big.numel() == 4 * base and len(_ops._gtab_cache) == 2
    held = sum(b.numel() for b in _ops._gtab_cache.values())
    assert held <= int(4 * base * 1.13) + (1 << 17)
    _ops.release_workspaces()
    assert not _ops._gtab_cache
