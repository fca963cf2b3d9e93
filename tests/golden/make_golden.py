"""Writes tests/golden/kge_small.npz: small seeded inputs for all eight score functions with scores and
dense gradients computed in float64 by torch library operations and autograd (no oracle, no HIP code).

The reference holds no golden vectors for this path (its tests only compare against eager PyTorch at run
time), so these fixtures are generated from the textbook / eager definitions
(apps/kge/test_pytorch.py:21,40,58,74,91 for the reference's five models).  They freeze inputs and
expected outputs as data; tests/test_golden.py checks the CPU oracle and the HIP path against them.

    python tests/golden/make_golden.py        # rewrites the .npz next to this file
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))                   # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))  # repo root

from cuke_amd import synth  # noqa: E402
from test_oracle_pins import ALL, T, torch_score  # noqa: E402


def main():
    out = {}
    for mi, model in enumerate(ALL):
        for p in (1, 2):
            if p == 1 and model not in ("TransE", "TransH", "TransR"):
                continue
            w = synth.custom_workload(model, n_ent=40, n_rel=5, dim=16, batch=16, chunk=8, n_neg=4, sigma=0.3,
                                      ent_zipf=1.1, gamma=3.0, norm_p=p, seed=100 + mi)
            a = w.arrays
            key = f"{model}_p{p}"
            for k in ("E", "R", "A", "h", "r", "t", "neg"):
                if a.get(k) is not None:
                    out[f"{key}/{k}"] = a[k]
            rng = np.random.default_rng(7 + mi)
            dpos = rng.standard_normal(w.batch).astype(np.float32)
            dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32)
            out[f"{key}/dpos"], out[f"{key}/dneg"] = dpos, dneg
            h, r, t = (torch.from_numpy(a[k]) for k in "hrt")
            ids = torch.from_numpy(a["neg"]).view(w.n_chunks, w.n_neg)[torch.arange(w.batch) // w.chunk]  # [B, N]
            for mode in ("tail", "head"):
                E = T(a["E"]).requires_grad_()
                R = T(a["R"]).requires_grad_() if a["R"] is not None and a["R"].size else None
                A = T(a["A"]).requires_grad_() if a["A"] is not None else None
                pos = torch_score(model, E, R, A, h, r, t, p, w.gamma)
                if mode == "tail":
                    neg = torch_score(model, E, R, A, h, r, ids, p, w.gamma)
                else:  # (neg_k, r_b, t_b): score every negative as a head, one column at a time
                    neg = torch.stack([torch_score(model, E, R, A, ids[:, k], r, t, p, w.gamma)
                                       for k in range(w.n_neg)], dim=1)
                (pos * T(dpos)).sum().add((neg * T(dneg)).sum()).backward()
                out[f"{key}/{mode}/pos"] = pos.detach().numpy()
                out[f"{key}/{mode}/neg"] = neg.detach().numpy()
                out[f"{key}/{mode}/gE"] = E.grad.numpy()
                if R is not None and R.grad is not None:
                    out[f"{key}/{mode}/gR"] = R.grad.numpy()
                if A is not None:
                    out[f"{key}/{mode}/gA"] = A.grad.numpy().reshape(w.n_rel, -1)
            out[f"{key}/meta"] = np.array([w.chunk, w.n_neg, p], np.int64)
            out[f"{key}/gamma"] = np.array([w.gamma], np.float64)
    path = os.path.join(HERE, "kge_small.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
