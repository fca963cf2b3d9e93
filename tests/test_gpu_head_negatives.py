"""Shared negatives that replace the HEAD of every positive of their chunk (the head batches of
apps/kge/data/sampler.py): scores and sparse gradients against the oracle, whose head mode is
pinned by brute force over explicit (neg, r, t) triples in test_oracle_pins.py."""
import numpy as np
import pytest
import torch

from cuke_amd import synth
from helpers import assert_close, gpu_model

pytestmark = pytest.mark.gpu

NEG_MODELS = ["TransE", "TransH", "DistMult", "ComplEx", "RotatE", "TransF"]


def both(oracle, w, seed=0, neg_mode="head"):
    a = w.arrays
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=neg_mode)
    pos, negs = oracle.score(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                             p=w.norm_p, gamma=w.gamma, neg_mode=neg_mode)
    rng = np.random.default_rng(seed)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32)
    g = m.backward(fw, torch.from_numpy(dpos).cuda(), torch.from_numpy(dneg).cuda())
    ref = oracle.backward(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, dpos, dneg,
                          p=w.norm_p, neg_mode=neg_mode)
    return fw, pos, negs, g, ref


def compare(fw, pos, negs, g, ref, what, outliers=None, floor=0.0):
    assert_close(fw.pos.cpu().numpy(), pos, what=what + " pos")
    assert_close(fw.neg.cpu().numpy(), negs, what=what + " neg")
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids), what
    assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids), what
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=what + " entity rows", rows=True, outliers=outliers,
                 global_floor=floor)
    if ref.rel_rows is not None and ref.rel_rows.size:
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=what + " relation rows", rows=True,
                     outliers=outliers, global_floor=floor)
    if ref.aux_rows is not None:
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=what + " aux rows", rows=True, global_floor=floor)


@pytest.mark.parametrize("model", NEG_MODELS)
@pytest.mark.parametrize("shape", [
    dict(dim=128, batch=256, chunk=64, n_neg=64),
    dict(dim=36, batch=96, chunk=32, n_neg=33),    # ragged tiles
    dict(dim=30, batch=40, chunk=8, n_neg=5),      # dim % 4 != 0: scalar loads
])
@pytest.mark.parametrize("p", [1, 2])
def test_head_negatives(oracle, model, shape, p):
    if p == 1 and model not in ("TransE", "TransH"):
        pytest.skip("norm order only matters for the translation models")
    w = synth.custom_workload(model, n_ent=300, n_rel=9, norm_p=p, sigma=0.3, gamma=4.0, ent_zipf=1.1, seed=p,
                              lattice=(p == 1), **shape)
    out = (1e-5, 4.0) if model == "RotatE" else None
    compare(*both(oracle, w), what=f"{model} {shape} p={p}", outliers=out)


@pytest.mark.parametrize("model", ["TransR", "RESCAL"])
def test_head_negatives_projection_models(oracle, model):
    w = synth.custom_workload(model, n_ent=200, n_rel=7, dim=32, batch=64, chunk=16, n_neg=8, sigma=0.25, seed=4)
    compare(*both(oracle, w), what=model)


@pytest.mark.parametrize("seed", range(30))
def test_head_negatives_random_shapes(oracle, seed):
    from test_gpu_random_shapes import draw
    spec = draw(seed)
    model = spec.pop("model")
    w = synth.custom_workload(model, seed=seed, **spec)
    out = (1e-5, 4.0) if model == "RotatE" else None
    compare(*both(oracle, w, seed=seed), what=f"seed {seed} {model} {spec}", outliers=out,
            floor=0.1 if w.dim < 8 else 0.0)


def test_tail_mode_is_unchanged_by_the_mode_argument(oracle):
    w = synth.custom_workload("TransH", n_ent=300, n_rel=9, dim=64, batch=128, chunk=32, n_neg=32, sigma=0.3, seed=2)
    m, ix = gpu_model(w)
    a = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    b = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode="tail")
    assert torch.equal(a.neg, b.neg) and torch.equal(a.pos, b.pos)
    with pytest.raises(ValueError):
        m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode="both")


@pytest.mark.parametrize("name,over", [("cfg2_distmult", dict(n_ent=100_000, batch=1024)),
                                       ("cfg4_rotate", dict(batch=512))])
def test_train_step_head_mode_graph_replay(oracle, name, over):
    from cuke_amd.kge import TrainStep
    w = synth.make_workload(name, **over)
    a = w.arrays
    m, ix = gpu_model(w)
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, loss="margin" if w.loss == "margin" else "sum",
                     margin=w.margin, neg_mode="head")
    step.run()
    torch.cuda.synchronize()
    pos, negs = oracle.score(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                             p=w.norm_p, gamma=w.gamma, neg_mode="head")
    assert_close(step.pos.cpu().numpy(), pos, what="pos")
    assert_close(step.neg.cpu().numpy(), negs, what="neg")
    eager = step.sparse_grads()
    e_rows = eager.ent_rows.clone()
    step.capture()
    for _ in range(3):
        step.ent_rows.zero_()
        step.replay()
        torch.cuda.synchronize()
        assert torch.equal(step.sparse_grads().ent_rows, e_rows)
