"""Randomised shapes: every model, forward and backward, against the oracle.

Shapes are drawn to hit the awkward corners: chunk sizes and negative counts that are not
multiples of the tile sizes, a single negative, one chunk, row widths that are not multiples of
4 (scalar-load path), widths below one staging slice, duplicate-heavy and duplicate-free ids."""
import numpy as np
import pytest
import torch

from cuke_amd import synth
from helpers import assert_close, gpu_model

pytestmark = pytest.mark.gpu

NEG_MODELS = ["TransE", "TransH", "DistMult", "ComplEx", "RotatE", "TransF"]


def draw(seed):
    rng = np.random.default_rng(seed)
    model = NEG_MODELS[seed % len(NEG_MODELS)]
    chunk = int(rng.choice([1, 3, 16, 31, 32, 33, 64, 70, 128]))
    n_chunks = int(rng.integers(1, 5))
    n_neg = int(rng.choice([1, 2, 5, 31, 32, 33, 63, 64, 65, 100]))
    dim = int(rng.choice([2, 4, 6, 12, 30, 32, 36, 64, 66, 100, 128, 130]))
    if model in ("ComplEx", "RotatE") and dim % 2:
        dim += 1
    n_ent = int(rng.choice([7, 50, 400, 5000]))
    p = int(rng.choice([1, 2]))
    return dict(model=model, n_ent=n_ent, n_rel=int(rng.integers(1, 9)), dim=dim, batch=chunk * n_chunks,
                chunk=chunk, n_neg=n_neg, norm_p=p, sigma=0.3, gamma=2.0,
                ent_zipf=float(rng.choice([0.0, 1.1])), lattice=(p == 1 and model in ("TransE", "TransH")))


@pytest.mark.parametrize("seed", range(120))
def test_random_shape(oracle, seed):
    spec = draw(seed)
    model = spec.pop("model")
    w = synth.custom_workload(model, seed=seed, **spec)
    a = w.arrays
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    pos, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                             p=w.norm_p, gamma=w.gamma)
    what = f"seed {seed}: {model} {spec}"
    assert_close(fw.pos.cpu().numpy(), pos, what=what + " pos")
    assert_close(fw.neg.cpu().numpy(), negs, what=what + " neg")
    rng = np.random.default_rng(seed + 1000)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32)
    g = m.backward(fw, torch.from_numpy(dpos).cuda(), torch.from_numpy(dneg).cuda())
    ref = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, dpos, dneg,
                          p=w.norm_p)
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids), what
    assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids), what
    out = (1e-5, 4.0) if model == "RotatE" else None
    floor = 0.1 if w.dim < 8 else 0.0
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=what + " entity rows", rows=True, outliers=out, global_floor=floor)
    assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=what + " relation rows", rows=True, outliers=out, global_floor=floor)
    if ref.aux_rows is not None:
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=what + " aux rows", rows=True, global_floor=floor)


def draw_grouped(seed):
    rng = np.random.default_rng(10_000 + seed)
    model = ["TransR", "RESCAL", "TransF"][seed % 3]
    dim = int(rng.choice([4, 8, 12, 16, 20, 36, 48, 64, 68, 100, 128, 132, 200]))
    batch = int(rng.choice([1, 2, 7, 16, 17, 64, 100, 255, 256, 600]))
    n_rel = int(rng.choice([1, 2, 5, 40, 300]))
    p = 2  # L1 gradients need lattice tables; covered in test_gpu_transr.py
    return dict(model=model, n_ent=int(rng.choice([5, 60, 900])), n_rel=n_rel, dim=dim, batch=batch, norm_p=p,
                sigma=0.25, rel_zipf=float(rng.choice([0.0, 1.3])), ent_zipf=float(rng.choice([0.0, 1.1])))


@pytest.mark.parametrize("seed", range(60))
def test_random_shape_relation_grouped(oracle, seed):
    """TransR / RESCAL through the relation-grouped path (and ungrouped), TransF per triple."""
    from cuke_amd.kge import inspect
    spec = draw_grouped(seed)
    model = spec.pop("model")
    w = synth.custom_workload(model, seed=seed, **spec)
    a = w.arrays
    m, ix = gpu_model(w)
    what = f"seed {seed}: {model} {spec}"
    pos, _ = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], p=2)
    rng = np.random.default_rng(seed + 2000)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    ref = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], dpos=dpos, p=2)
    floor = 0.1 if w.dim < 8 else 0.0
    variants = [None] if model == "TransF" else [inspect([ix["r"]], m.n_rel), None]
    for rel in variants:
        tag = what + (" grouped" if rel is not None else " ungrouped")
        fw = m.score(ix["h"], ix["r"], ix["t"], rel_insp=rel)
        assert_close(fw.pos.cpu().numpy(), pos, what=tag + " pos")
        g = m.backward(fw, torch.from_numpy(dpos).cuda())
        assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids), tag
        assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids), tag
        assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=tag + " entity rows", rows=True,
                     global_floor=floor)
        if ref.rel_rows is not None and ref.rel_rows.size:
            assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=tag + " relation rows", rows=True,
                         global_floor=floor)
        if ref.aux_rows is not None:
            assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=tag + " projection rows", rows=True,
                         global_floor=floor)
