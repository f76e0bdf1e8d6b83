"""GPU parity of the attention-weights debug output (upstream ``return_attention=True``,
sb_varlen_fwd.py:195-202 and :421-425, sb_attn/sb_fwd.py:147-151) against the oracle's dense
weights.  The weights are fp32 values computed from bf16-MFMA logits: tolerance 2e-2 max-abs
like every other output (observed: a few 1e-3)."""
import os

import pytest
import torch

from oracle import sb_oracle as orc
from tests.helpers import assert_close, cu_from_lengths

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from stickbreaking_attention import _native as nat
    assert os.path.exists(nat.LIB_PATH), "libsba.so must be built before the GPU tests run"
    nat.load()


@pytest.mark.parametrize("ac", [False, True])
@pytest.mark.parametrize("d", [32, 64, 128, 256])
@pytest.mark.parametrize("product_space", [False, True])
def test_varlen_attention_weights(ac, d, product_space, monkeypatch):
    from stickbreaking_attention import _ops
    from stickbreaking_attention.sb_varlen import varlen_fwd
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", product_space)
    lengths, tail = [130, 1, 65, 200], 4
    T = sum(lengths) + tail
    q, k, v, _ = orc.make_inputs((3, T, d), 40 + d, dist="upstream")
    cu = cu_from_lengths(lengths, device=DEV)
    o, rem, _state, W = varlen_fwd(q.to(DEV), k.to(DEV), v.to(DEV), cu, max(lengths), d ** -0.5, attend_current=ac,
                                   return_attention=True)
    torch.cuda.synchronize()
    assert W.shape == (3, T, T) and W.dtype == torch.float32
    ref = torch.zeros(3, T, T)
    s = 0
    for n in lengths:
        ref[:, s:s + n, s:s + n] = orc.attention_weights(q[:, s:s + n].float(), k[:, s:s + n].float(), ac)
        s += n
    assert_close("W", W, ref)
    # nothing is written outside the causal triangle of a document
    doc = torch.repeat_interleave(torch.arange(len(lengths) + 1), torch.tensor(lengths + [tail]))
    allowed = (doc[:, None] == doc[None, :]) & (doc[:, None] < len(lengths)) & torch.ones(T, T).tril(0 if ac else -1).bool()
    assert torch.count_nonzero(W.cpu()[:, ~allowed]).item() == 0
    # and the two regular outputs are what the weights imply
    assert_close("o", o, torch.matmul(ref, v.float()))
    assert_close("rem", rem[:, :sum(lengths)], 1.0 - ref.sum(-1)[:, :sum(lengths)])


def test_fixed_length_attention_weights():
    from stickbreaking_attention.sb_attn import _fwd
    B, H, T, d = 2, 2, 200, 64
    q, k, v, _ = orc.make_inputs((B, H, T, d), 12, dist="upstream")
    o, rem, _state, W = _fwd(q.to(DEV), k.to(DEV), v.to(DEV), d ** -0.5, return_attention=True)
    torch.cuda.synchronize()
    assert W.shape == (B, H, T, T)
    ref = orc.attention_weights(q.float(), k.float())
    assert_close("W", W, ref)
    assert_close("rem", rem, 1.0 - ref.sum(-1))
