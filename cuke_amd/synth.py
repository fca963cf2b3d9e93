"""Seeded synthetic inputs for the KGE score path.

The reference gets its tables from ``torch.rand`` and its indices from a DGL
edge sampler over a downloaded dataset (apps/kge/data/data_init.py:4-63);
neither is available offline, so every workload here is generated from fixed
seeds with the shapes and distributions the benchmark configurations name:
tables N(0, sigma), uniform or bounded-Zipf indices, per-chunk shared
negative tails, RotatE phases uniform in [-pi, pi), TransH normals of unit
length.  Everything is numpy on the host; callers move arrays to the GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np


def zipf_indices(rng: np.random.Generator, n_rows: int, count: int, s: float) -> np.ndarray:
    """Bounded Zipf(s) over ``n_rows`` ids; rank k has weight k**-s, ranks are
    mapped to ids through a random permutation so hot rows are scattered."""
    w = np.arange(1, n_rows + 1, dtype=np.float64) ** (-s)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    rank = np.searchsorted(cdf, rng.random(count), side="left")
    rank = np.minimum(rank, n_rows - 1)
    perm = rng.permutation(n_rows)
    return perm[rank].astype(np.int64)


def uniform_indices(rng: np.random.Generator, n_rows: int, count: int) -> np.ndarray:
    return rng.integers(0, n_rows, count, dtype=np.int64)


@dataclass
class Workload:
    name: str
    model: str
    n_ent: int
    n_rel: int
    dim: int                 # floats per entity row
    batch: int
    chunk: int = 0           # positives per chunk (0: no shared negatives)
    n_neg: int = 0           # shared negative tails per chunk
    norm_p: int = 2
    gamma: float = 0.0
    margin: float = 1.0
    sigma: float = 0.1
    ent_zipf: float = 0.0    # 0: uniform
    rel_zipf: float = 0.0
    backward: bool = True
    loss: str = "sum"        # "sum": dL/dscore = 1 everywhere; "margin": margin-ranking loss
    lattice: bool = False    # tables on a coarse binary grid: every residual is exact in fp32
    seed: int = 0
    arrays: dict = field(default_factory=dict)

    @property
    def rel_dim(self) -> int:
        return self.dim // 2 if self.model == "RotatE" else self.dim

    @property
    def n_chunks(self) -> int:
        return self.batch // self.chunk if self.chunk else 0

    @property
    def scores_per_step(self) -> int:
        return self.batch * (1 + self.n_neg)


# The five benchmark configurations.  cfg 4 and 5 do not state the chunk size;
# chunk == n_neg is assumed (the reference's own shared-negative layout has
# chunk == n_neg, apps/examples/examples.py:1404-1444).
CONFIGS = {
    "cfg1_transe": dict(model="TransE", n_ent=16384, n_rel=1024, dim=128, batch=1024, norm_p=2,
                        sigma=0.1, backward=False),
    "cfg2_distmult": dict(model="DistMult", n_ent=1_000_000, n_rel=2000, dim=256, batch=4096,
                          chunk=256, n_neg=256, sigma=0.05, ent_zipf=1.1),
    "cfg2_complex": dict(model="ComplEx", n_ent=1_000_000, n_rel=2000, dim=256, batch=4096,
                         chunk=256, n_neg=256, sigma=0.05, ent_zipf=1.1),
    "cfg3_transr": dict(model="TransR", n_ent=40000, n_rel=1345, dim=200, batch=8192, norm_p=2,
                        sigma=0.05, rel_zipf=1.2),
    "cfg4_rotate": dict(model="RotatE", n_ent=40943, n_rel=11, dim=1000, batch=1024, chunk=256,
                        n_neg=256, sigma=0.05, ent_zipf=1.1, gamma=12.0, margin=1.0,
                        loss="margin"),
    "cfg5_transh": dict(model="TransH", n_ent=4_000_000, n_rel=10000, dim=400, batch=16384,
                        chunk=1024, n_neg=1024, norm_p=1, sigma=0.05, ent_zipf=1.05),
}


def make_indices(w: Workload) -> None:
    """h, r, t (and neg) index arrays, int64, from the workload's seed."""
    rng = np.random.default_rng([w.seed, 1])
    draw_e = (lambda n: zipf_indices(rng, w.n_ent, n, w.ent_zipf)) if w.ent_zipf else \
        (lambda n: uniform_indices(rng, w.n_ent, n))
    a = w.arrays
    a["h"] = draw_e(w.batch)
    a["t"] = draw_e(w.batch)
    a["r"] = zipf_indices(rng, w.n_rel, w.batch, w.rel_zipf) if w.rel_zipf else \
        uniform_indices(rng, w.n_rel, w.batch)
    if w.chunk:
        a["neg"] = draw_e(w.n_chunks * w.n_neg)


def make_tables(w: Workload) -> None:
    """E, R and the per-relation auxiliary table (TransH normals / TransR projections)."""
    rng = np.random.default_rng([w.seed, 2])
    a = w.arrays
    a["E"] = rng.standard_normal((w.n_ent, w.dim), dtype=np.float32) * np.float32(w.sigma)
    if w.model == "RotatE":
        a["R"] = rng.uniform(-np.pi, np.pi, (w.n_rel, w.rel_dim)).astype(np.float32)
    else:
        a["R"] = rng.standard_normal((w.n_rel, w.rel_dim), dtype=np.float32) * np.float32(w.sigma)
    a["A"] = None
    if w.model == "TransH":
        wn = rng.standard_normal((w.n_rel, w.dim), dtype=np.float32)
        wn /= np.linalg.norm(wn, axis=1, keepdims=True).astype(np.float32)
        a["A"] = wn
    elif w.model in ("TransR", "RESCAL"):
        a["A"] = rng.standard_normal((w.n_rel, w.dim, w.dim), dtype=np.float32) * np.float32(w.sigma)
    if w.lattice:
        # Multiples of 1/64 in [-1, 1] for E and R, of 1/4 for the TransH normals: sums and
        # products of a few hundred such values fit in 24 bits, so translation-model residuals
        # come out identical whatever the summation order or FMA use.  L1 gradients (a sum of
        # signs of residual elements) can then be compared without sign flips at |u| ~ 1 ulp.
        def grid(x, step):
            return (np.clip(np.rint(x / np.float32(w.sigma) / 3 / step) * step, -1, 1)).astype(np.float32)
        a["E"] = grid(a["E"], 1 / 64)
        if w.model != "RotatE":
            a["R"] = grid(a["R"], 1 / 64)
        if w.model == "TransH":
            a["A"] = (np.clip(np.rint(a["A"] * 4 * 3), -4, 4) / 4).astype(np.float32)


def device_tables(w: Workload, dev):
    """The workload's tables drawn on the GPU from its seed (same distributions as make_tables): tables of
    benchmark size are too large to push through numpy.  Returns torch tensors (E, R, A)."""
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(1000 + w.seed)
    f32 = dict(generator=g, device=dev, dtype=torch.float32)
    E = torch.randn((w.n_ent, w.dim), **f32) * w.sigma
    if w.model == "RotatE":
        R = (torch.rand((w.n_rel, w.rel_dim), **f32) * 2 - 1) * np.pi
    else:
        R = torch.randn((w.n_rel, w.rel_dim), **f32) * w.sigma
    A = None
    if w.model == "TransH":
        A = torch.randn((w.n_rel, w.dim), **f32)
        A = A / A.norm(dim=1, keepdim=True)
    elif w.model in ("TransR", "RESCAL"):
        A = torch.randn((w.n_rel, w.dim, w.dim), **f32) * w.sigma
    return E, R, A


def make_workload(name: str, seed: int = 0, tables: bool = True, **override) -> Workload:
    """Build a named configuration; keyword overrides shrink it for tests."""
    spec = dict(CONFIGS[name])
    spec.update(override)
    w = Workload(name=name, seed=seed, **spec)
    if w.chunk:
        assert w.batch % w.chunk == 0, "batch must be a whole number of chunks"
    make_indices(w)
    if tables:
        make_tables(w)
    return w


def custom_workload(model: str, seed: int = 0, **kw) -> Workload:
    w = Workload(name=f"custom_{model}", model=model, seed=seed, **kw)
    make_indices(w)
    make_tables(w)
    return w
