"""The library only enqueues kernels on the stream it is given (no allocation, no host
synchronisation, no memset nodes), so a forward + backward can be recorded into a HIP graph and
replayed.  Every replay is checked bit-for-bit against eager launches on the same inputs, with
eager work and synchronisations between the replays."""
import os

import pytest
import torch

from oracle import sb_oracle as orc
from tests.helpers import cu_from_lengths

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from stickbreaking_attention import _native as nat
    assert os.path.exists(nat.LIB_PATH), "libsba.so must be built before the GPU tests run"
    nat.load()


@pytest.mark.parametrize("fused", [False, True])
def test_forward_and_backward_replay_from_a_hip_graph(fused):
    from stickbreaking_attention import _ops
    lengths = [300, 77, 410]
    H, T, d = 4, sum(lengths) + 5, 128
    cu = cu_from_lengths(lengths, device=DEV)
    inv_temp = d ** -0.5

    def launch(q, k, v, do):
        o, rem, state = _ops.run_forward(q, k, v, False, cu, max(lengths), inv_temp, False, need_table=True, fused=fused)
        return (o, rem) + _ops.run_backward(q, k, v, do, None, False, state, inv_temp, False, fused=fused)

    def inputs(seed):
        return [t.to(DEV) for t in orc.make_inputs((H, T, d), seed)]

    static = inputs(100)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(*static)                       # warm-up outside the capture (loads the library, fills caches)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = launch(*static)
    # the replays must not lean on anything the Python layer remembers between eager calls (schedule,
    # gradient table): drop all of it and let the allocator hand that memory to someone else
    _ops.release_workspaces()
    junk = [torch.full((1 << 18,), -1, dtype=torch.int32, device=DEV) for _ in range(16)]
    torch.cuda.synchronize()
    for seed in (101, 102, 103):
        fresh = inputs(seed)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        eager = launch(*fresh)
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "rem", "dq", "dk", "dv"), captured, eager):
            assert torch.equal(a, b), f"replay with seed {seed}: {name} differs from the eager launch"
    del junk


def test_capture_with_a_cu_seqlens_tensor_never_seen_in_eager_mode():
    """Under capture nothing may be read back from the device: a cu_seqlens tensor whose values the
    Python layer does not know yet is taken as is (tables sized from max_seqlens, checks on the
    device), and the replays still equal eager launches."""
    from stickbreaking_attention import _ops, sb_attn_varlen
    lengths = [260, 31, 129, 500]
    H, T, d = 2, sum(lengths), 64
    inv_temp = d ** -0.5

    def make_cu():
        return torch.tensor([0] + lengths, dtype=torch.int64).cumsum(0).to(torch.int32).to(DEV)

    def launch(q, k, v, do, cu):
        qg, kg, vg = (t.detach().requires_grad_() for t in (q, k, v))
        o, rem = sb_attn_varlen(qg, kg, vg, cu, max(lengths), inv_temp, zero_start=True)
        return (o, rem) + torch.autograd.grad(o, (qg, kg, vg), do)

    static = [t.to(DEV) for t in orc.make_inputs((H, T, d), 200)]
    warm_cu = make_cu()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(*static, warm_cu)              # loads the library; this tensor object is not the captured one
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    _ops.release_workspaces()
    fresh_cu = make_cu()                      # never passed to the library before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = launch(*static, fresh_cu)
    for seed in (201, 202):
        fresh = [t.to(DEV) for t in orc.make_inputs((H, T, d), seed)]
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        eager = launch(*fresh, make_cu())
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "rem", "dq", "dk", "dv"), captured, eager):
            assert torch.equal(a, b), f"replay with seed {seed}: {name} differs from the eager launch"
