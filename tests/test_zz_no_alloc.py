"""The entry point that allocates nothing (sba_varlen_fwd_static) against the ordinary forward
(sba_build_schedule + sba_varlen_fwd), both called through the C ABI: bit-identical o and rem on
two calls in a row, the second on a smaller problem (the static schedule array keeps the first
call's contents), plus the size limit."""
import ctypes

import pytest
import torch

from oracle import sb_oracle as orc
from stickbreaking_attention import _native as nat
from tests import helpers

pytestmark = pytest.mark.gpu


def _problem(q, cu, max_len, inv_temp):
    H, T, d = q.shape
    flags = nat.FLAG_PRODUCT_SPACE | (nat.FLAG_CU_INT64 if cu.dtype == torch.int64 else 0)
    return nat.SbaProblem(nat.SBA_BF16, d, H, 1, T, cu.numel(), max_len, flags, float(inv_temp), cu.data_ptr())


def _forward_pair(lengths, H, d, seed):
    """(o, rem) from the static entry point and from the ordinary one, same inputs."""
    lib = nat.load()
    dev = torch.device("cuda:0")
    T = sum(lengths) + 37          # some tokens belong to no document: both paths must clear them
    q, k, v, _ = (t.to(dev) for t in orc.make_inputs((H, T, d), seed))
    cu = helpers.cu_from_lengths(lengths, device=dev)
    prob = _problem(q, cu, max(lengths), d ** -0.5)
    views = lambda o, rem: [ctypes.byref(nat.view4(t, False)) for t in (q, k, v, o)] + [ctypes.byref(nat.view4(rem, False, per_row=True))]
    stream = nat.stream_ptr(dev)
    # outputs start from different garbage so that equality means both were fully written
    o_a, rem_a = torch.full_like(q, 7.0), torch.full_like(q[..., 0], 7.0)
    o_b, rem_b = torch.full_like(q, -3.0), torch.full_like(q[..., 0], -3.0)
    sched = torch.empty(lib.sba_schedule_bytes(ctypes.byref(prob)), dtype=torch.uint8, device=dev)
    # one call first: the library looks its array's device address up on the first call per device
    nat.check(lib.sba_varlen_fwd_static(ctypes.byref(prob), *views(o_a, rem_a), stream), "sba_varlen_fwd_static")
    torch.cuda.synchronize()
    o_a.fill_(7.0); rem_a.fill_(7.0)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]      # the driver's own count: sees a hipMalloc inside the library too
    nat.check(lib.sba_varlen_fwd_static(ctypes.byref(prob), *views(o_a, rem_a), stream), "sba_varlen_fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before, "sba_varlen_fwd_static changed the device's free memory"
    nat.check(lib.sba_build_schedule(ctypes.byref(prob), sched.data_ptr(), sched.numel(), stream), "sba_build_schedule")
    nat.check(lib.sba_varlen_fwd(ctypes.byref(prob), sched.data_ptr(), sched.numel(), *views(o_b, rem_b), None, 0, stream), "sba_varlen_fwd")
    torch.cuda.synchronize()
    return (q, k, v), (o_a, rem_a), (o_b, rem_b)


def test_static_forward_matches_the_ordinary_forward_twice_in_a_row():
    for lengths, H, d, seed in (([700, 129, 1, 333, 64, 2000], 4, 128, 11), ([45, 200, 17], 3, 64, 12)):
        (q, k, v), (o_a, rem_a), (o_b, rem_b) = _forward_pair(lengths, H, d, seed)
        assert torch.equal(o_a, o_b), f"o differs for lengths {lengths}"
        assert torch.equal(rem_a, rem_b), f"rem differs for lengths {lengths}"
        assert torch.isfinite(o_a.float()).all()
        # and both agree with the oracle on the documents' rows
        T = sum(lengths)
        ro, rrem = orc.sb_varlen(q.float().cpu(), k.float().cpu(), v.float().cpu(), lengths)
        helpers.assert_close("o", o_a[:, :T], ro[:, :T])
        helpers.assert_close("rem", rem_a[:, :T], rrem[:, :T])
        assert (o_a[:, T:] == 0).all() and (rem_a[:, T:] == 0).all()


def test_static_forward_rejects_problems_beyond_its_array():
    lib = nat.load()
    dev = torch.device("cuda:0")
    n_docs = 40000                      # the schedule of this many documents does not fit 512 KiB
    q = torch.zeros(1, n_docs, 64, dtype=torch.bfloat16, device=dev)
    cu = torch.arange(1, n_docs + 1, dtype=torch.int32, device=dev)
    prob = _problem(q, cu, 1, 0.125)
    assert lib.sba_schedule_bytes(ctypes.byref(prob)) > 512 * 1024
    o, rem = torch.empty_like(q), torch.empty_like(q[..., 0])
    vs = [ctypes.byref(nat.view4(t, False)) for t in (q, q, q, o)] + [ctypes.byref(nat.view4(rem, False, per_row=True))]
    assert lib.sba_varlen_fwd_static(ctypes.byref(prob), *vs, nat.stream_ptr(dev)) == -6
