"""Writes tests/golden/small_cases.npz: inputs and float64 expected outputs of tiny problems.

Expected o and rem come from the oracle's product-form double loop (float64, no log space),
gradients from float64 autograd through the oracle, cross-checked here against the
hand-derived backward before anything is written.  Inputs are stored already rounded to bf16
(as float32) so the device and the oracle see identical values.
Run once:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import sb_oracle as orc  # noqa: E402

CASES = {
    # name: (heads, lengths, head_dim, attend_current, dist)
    "a": (2, [96], 64, False, "normal"),
    "b": (2, [96], 64, True, "normal"),
    "c": (2, [70, 1, 150, 33], 128, False, "upstream"),
    "d": (1, [200], 128, True, "upstream"),
}


def main():
    out = {}
    for name, (H, lengths, d, ac, dist) in CASES.items():
        T = sum(lengths)
        q, k, v, do = (t.float() for t in orc.make_inputs((H, T, d), 4242 + len(name) + T, dist=dist))
        g = torch.Generator().manual_seed(99 + T)
        dr = torch.randn((H, T), generator=g).to(torch.bfloat16).float()
        o, rem, dq, dk, dv = orc.sb_varlen_grads(q.double(), k.double(), v.double(), lengths, do.double(),
                                                 dr.double(), ac)
        start = 0
        for n in lengths:
            for h in range(H):
                sl = slice(start, start + n)
                ob, rb, _ = orc.bruteforce(q[h, sl], k[h, sl], v[h, sl], ac)
                assert torch.allclose(o[h, sl], ob, atol=1e-11) and torch.allclose(rem[h, sl], rb, atol=1e-11)
                aq, ak, av = orc.analytic_backward(q[h, sl], k[h, sl], v[h, sl], do[h, sl], dr[h, sl], ac)
                assert torch.allclose(dq[h, sl], aq, atol=1e-10) and torch.allclose(dk[h, sl], ak, atol=1e-10)
                assert torch.allclose(dv[h, sl], av, atol=1e-10)
            start += n
        for key, t in dict(q=q, k=k, v=v, do=do, dr=dr, o=o, rem=rem, dq=dq, dk=dk, dv=dv).items():
            out[f"{name}_{key}"] = t.numpy().astype(np.float32)
        out[f"{name}_lengths"] = np.array(lengths, dtype=np.int32)
        out[f"{name}_ac"] = np.array([int(ac)], dtype=np.int32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "small_cases.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
