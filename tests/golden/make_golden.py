"""Writes tests/golden/ref_cpp_golden.npz: seeded inputs and the outputs that the
reference's own CPU extension (cpp/l1attn_drv.cpp, cpp/l1attn_sparse_drv.cpp,
cpp/l1attn_sparse_bidi_drv.cpp, compiled by `make -C oracle` into oracle/_ref) returns
for them.  Run in the build container only (the reference tree does not travel):

    python tests/golden/make_golden.py

The edge lists are expanded with the brute-force rank in tests/closed_forms.py, so no
Python file of the reference is imported.  float64 only: the reference's CPU extension
has no other type (cpp/l1attn_drv.cpp:5).
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import oracle  # noqa: E402
from closed_forms import expand_coo_bruteforce  # noqa: E402


def main():
    mods = oracle.ref_modules()
    if mods is None:
        raise SystemExit("oracle/_ref is not built (make -C oracle, needs /root/reference)")
    out = {}
    g = torch.Generator().manual_seed(20241)

    # dense: B=2,T=5,H=3,W=7 (ragged everything) and the reference's check.py shape 1,16,8,64
    for tag, (B, T, H, W) in {"dA": (2, 5, 3, 7), "dB": (1, 16, 8, 64)}.items():
        q = torch.randn(B, T, H, W, generator=g, dtype=torch.float64)
        k = torch.randn(B, T, H, W, generator=g, dtype=torch.float64)
        k[0, 1] = q[0, 2]  # exact ties: sign(0) = 0 must show in the gradients
        da = torch.randn(B, T, T, H, generator=g, dtype=torch.float64)
        (attn,) = mods["l1attn_drv_cpp"].forward(q, k)
        dq, dk = mods["l1attn_drv_cpp"].backward(da, q, k)
        for n, t in dict(q=q, k=k, da=da, attn=attn, dq=dq, dk=dk).items():
            out[f"{tag}_{n}"] = t.numpy()

    # sparse / bidi: check_sparse.py shape B=2,T=3,H=16,W=7 with a permuted cartesian list
    # minus 4 edges, and a ragged random list on T=6 with a dst that has no edge.
    B, T, H, W = 2, 3, 16, 7
    co = torch.cartesian_prod(torch.arange(T), torch.arange(T))
    co = co[torch.randperm(co.shape[0], generator=g)][:-4]
    cases = {"sA": (B, T, H, W, co)}
    co2 = torch.tensor([[0, 1], [0, 3], [2, 2], [5, 0], [0, 5], [2, 1], [4, 4], [5, 5], [5, 1], [0, 0]])
    cases["sB"] = (1, 6, 2, 5, co2)
    for tag, (B, T, H, W, co) in cases.items():
        coo, dmx, smx = expand_coo_bruteforce(co)
        v, q, k, vb, dvo = (torch.randn(B, T, H, W, generator=g, dtype=torch.float64) for _ in range(5))
        out[f"{tag}_co"] = co.numpy()
        out[f"{tag}_coo"] = coo.numpy()
        out[f"{tag}_mx"] = np.array([dmx, smx])
        for n, t in dict(v=v, q=q, k=k, vb=vb, dvo=dvo).items():
            out[f"{tag}_{n}"] = t.numpy()
        for sm in (True, False):
            s = "sm" if sm else "nsm"
            vo, attn = mods["l1attn_sparse_drv"].forward(v, q, k, coo, dmx, sm)
            dv, dq, dk = mods["l1attn_sparse_drv"].backward(dvo, v, q, k, coo, attn, dmx, sm)
            for n, t in dict(vo=vo, attn=attn, dv=dv, dq=dq, dk=dk).items():
                out[f"{tag}_{s}_{n}"] = t.numpy()
            vo, attn = mods["l1attn_sparse_bidi_drv"].forward(v, vb, q, k, coo, dmx, sm)
            dvf, dvb, dq, dk = mods["l1attn_sparse_bidi_drv"].backward(dvo, v, vb, q, k, coo, attn, dmx, sm)
            for n, t in dict(vo=vo, dvf=dvf, dvb=dvb, dq=dq, dk=dk).items():
                out[f"{tag}_{s}_bidi_{n}"] = t.numpy()
    path = os.path.join(HERE, "ref_cpp_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
