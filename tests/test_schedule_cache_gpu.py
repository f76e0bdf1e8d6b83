"""The scheduler kernel runs once per cu_seqlens tensor, not once per call: the Python layer keeps
the schedule workspace it built for a tensor object (and the view without the leading zero it handed
out) and reuses both while the tensor comes back unmodified."""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from stickbreaking_attention import _native as nat
    assert os.path.exists(nat.LIB_PATH), "libsba.so must be built before the GPU tests run"
    nat.load()


def test_schedule_is_reused_per_cu_seqlens_tensor_and_rebuilt_after_a_change():
    from stickbreaking_attention import _ops, sb_attn_varlen
    dev = torch.device("cuda:0")
    torch.manual_seed(3)
    H, T, d = 2, 384, 64
    q, k, v = (torch.randn(H, T, d, device=dev, dtype=torch.bfloat16) for _ in range(3))
    cu = torch.tensor([0, 100, 230, 384], device=dev, dtype=torch.int32)
    _ops.release_workspaces()
    o1, r1 = sb_attn_varlen(q, k, v, cu, 200)
    n = len(_ops._sched_cache)
    sched1 = _ops._sched_cache[-1][3]
    o2, r2 = sb_attn_varlen(q, k, v, cu, 200)
    assert len(_ops._sched_cache) == n and _ops._sched_cache[-1][3] is sched1      # same workspace, not rebuilt
    assert torch.equal(o1, o2) and torch.equal(r1, r2)
    # same values in a NEW tensor: a new schedule (identity, not contents, is what is remembered)
    cu_b = cu.clone()
    o3, r3 = sb_attn_varlen(q, k, v, cu_b, 200)
    assert _ops._sched_cache[-1][3] is not sched1
    assert torch.equal(o1, o3)
    # an in-place change of the documents is seen through the version counter
    cu[1] = 150
    o4, r4 = sb_attn_varlen(q, k, v, cu, 200)
    ref = torch.tensor([0, 150, 230, 384], device=dev, dtype=torch.int32)
    o5, r5 = sb_attn_varlen(q, k, v, ref, 200)
    assert torch.equal(o4, o5) and torch.equal(r4, r5)
    assert not torch.equal(o4, o1)


def test_fixed_length_schedule_is_reused_per_shape():
    from stickbreaking_attention import _ops, sb_attn
    dev = torch.device("cuda:0")
    torch.manual_seed(4)
    q, k, v = (torch.randn(2, 2, 256, 64, device=dev, dtype=torch.bfloat16) for _ in range(3))
    _ops.release_workspaces()
    o1, r1 = sb_attn(q, k, v)
    sched1 = _ops._sched_cache[-1][3]
    o2, r2 = sb_attn(q, k, v)
    assert _ops._sched_cache[-1][3] is sched1 and torch.equal(o1, o2) and torch.equal(r1, r2)
    q2, k2, v2 = (torch.randn(2, 2, 384, 64, device=dev, dtype=torch.bfloat16) for _ in range(3))
    sb_attn(q2, k2, v2)
    assert _ops._sched_cache[-1][3] is not sched1
    o3, _ = sb_attn(q, k, v)          # the first shape again: still right
    assert torch.equal(o1, o3)
