"""Forward parity: HIP kernels (through the C ABI) against the CPU oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from cuke_amd import synth
from helpers import assert_close, gpu_model

pytestmark = pytest.mark.gpu

RESIDUAL = ["TransE", "TransH", "TransR"]
NEG_MODELS = ["TransE", "TransH", "DistMult", "ComplEx", "RotatE", "TransF"]
ALL = ["TransE", "TransH", "TransR", "DistMult", "ComplEx", "RotatE", "TransF", "RESCAL"]


def test_cfg1_transe_residual_bit_exact_and_l2_score(oracle):
    w = synth.make_workload("cfg1_transe")
    a = w.arrays
    m, ix = gpu_model(w)
    got = m.residual(ix["h"], ix["r"], ix["t"]).cpu().numpy()
    want = oracle.residual("TransE", a["E"], a["R"], None, a["h"], a["r"], a["t"])
    assert np.array_equal(got, want)  # two fp32 adds in a fixed order: exact
    pos, _ = oracle.score("TransE", a["E"], a["R"], None, a["h"], a["r"], a["t"], p=2)
    assert_close(m.score(ix["h"], ix["r"], ix["t"]).pos.cpu().numpy(), pos, what="cfg1 L2 score")


def test_reference_shaped_callables(oracle):
    from cuke_amd import kge
    for model in RESIDUAL:
        w = synth.custom_workload(model, n_ent=300, n_rel=17, dim=64, batch=160, sigma=0.2, seed=4)
        a = w.arrays
        dev = torch.device("cuda:0")
        E, R = torch.from_numpy(a["E"]).to(dev), torch.from_numpy(a["R"]).to(dev)
        h, r, t = (torch.from_numpy(a[k]).to(dev) for k in "hrt")
        dummy = torch.zeros(1, device=dev)
        if model == "TransE":
            out = kge.transE(w.batch, w.dim, w.n_ent, E, h, t, w.n_rel, R, r)
        elif model == "TransH":
            P = torch.from_numpy(a["A"]).to(dev)
            out = kge.transH(w.batch, w.dim, w.n_ent, E, h, t, w.n_rel, R, r, dummy, dummy, dummy, P)
        else:
            P = torch.from_numpy(a["A"]).to(dev)
            out = kge.transR(w.batch, w.dim, 0, E, h, t, 0, P, r, dummy, dummy, dummy, R)
        want = oracle.residual(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"])
        assert_close(out.cpu().numpy(), want, what=f"{model} residual")


def test_reference_shaped_scalar_callables(oracle):
    """kge.transF / kge.RESCAL take the reference's positional lists literally
    (apps/kge/test_cuke.py:198,244): (batch, dim, nnodes, E, h, nedges, R | Proj, r, uniq, buf, cnt, t) -- the tail
    ids come LAST, after the three inspector tensors.  h and t are drawn differently, and TransF / RESCAL are not
    symmetric in them, so a slip in the order changes the scores."""
    from cuke_amd import kge
    dev = torch.device("cuda:0")
    for model in ("TransF", "RESCAL"):
        w = synth.custom_workload(model, n_ent=300, n_rel=17, dim=64, batch=160, sigma=0.2, seed=9)
        a = w.arrays
        E = torch.from_numpy(a["E"]).to(dev)
        h, r, t = (torch.from_numpy(a[k]).to(dev) for k in "hrt")
        r_sorted, order = torch.sort(r)  # the reference sorts the batch by relation before its inspector
        uniq, buf, cnt = kge.inspector(r_sorted, w.n_rel)
        if model == "TransF":
            Rm = torch.from_numpy(a["R"]).to(dev)
            out = kge.transF(w.batch, w.dim, w.n_ent, E, h[order], w.n_rel, Rm, r_sorted, uniq, buf, cnt, t[order])
        else:
            Pm = torch.from_numpy(a["A"]).to(dev)
            out = kge.RESCAL(w.batch, w.dim, w.n_ent, E, h[order], w.n_rel, Pm, r_sorted, uniq, buf, cnt, t[order])
        o = order.cpu().numpy()
        want, _ = oracle.score(model, a["E"], a["R"], a["A"], a["h"][o], a["r"][o], a["t"][o])
        assert out.shape == (w.batch,)
        assert_close(out.cpu().numpy(), want, what=f"{model} positional call")
        swapped, _ = oracle.score(model, a["E"], a["R"], a["A"], a["t"][o], a["r"][o], a["h"][o])
        assert np.abs(swapped - want).max() > 1e-3, "the test inputs must tell h from t"


@pytest.mark.parametrize("model", ALL)
@pytest.mark.parametrize("dim", [24, 20, 200])
@pytest.mark.parametrize("p", [1, 2])
def test_positive_scores(oracle, model, dim, p):
    if p == 1 and model not in RESIDUAL:
        pytest.skip("norm order only matters for the translation models")
    if dim == 20 and model in ("ComplEx", "RotatE"):
        dim = 22  # complex rows need an even width; 11 per half exercises the scalar path
    w = synth.custom_workload(model, n_ent=500, n_rel=23, dim=dim, batch=203, norm_p=p, sigma=0.2,
                              gamma=4.0, ent_zipf=1.1, seed=dim + p)
    a = w.arrays
    m, ix = gpu_model(w)
    got = m.score(ix["h"], ix["r"], ix["t"]).pos.cpu().numpy()
    want, _ = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], p=p, gamma=w.gamma)
    assert_close(got, want, what=f"{model} d={dim} p={p}")


@pytest.mark.parametrize("model", NEG_MODELS)
@pytest.mark.parametrize("shape", [
    dict(dim=24, batch=96, chunk=24, n_neg=40),      # ragged tile edges
    dict(dim=22, batch=64, chunk=64, n_neg=7),       # scalar-load path, tiny N
    dict(dim=200, batch=256, chunk=128, n_neg=130),  # several slices, ragged N
])
@pytest.mark.parametrize("p", [1, 2])
def test_shared_negative_scores(oracle, model, shape, p):
    if p == 1 and model not in ("TransE", "TransH"):
        pytest.skip("norm order only matters for the translation models")
    w = synth.custom_workload(model, n_ent=400, n_rel=19, norm_p=p, sigma=0.2, gamma=4.0,
                              ent_zipf=1.1, seed=shape["dim"] + p, **shape)
    a = w.arrays
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    pos, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                             p=p, gamma=w.gamma)
    assert_close(fw.pos.cpu().numpy(), pos, what=f"{model} pos")
    assert_close(fw.neg.cpu().numpy(), negs, what=f"{model} neg {shape}")


@pytest.mark.parametrize("model,dim,p", [("TransE", 640, 1), ("TransE", 520, 2), ("RotatE", 1000, 2), ("RotatE", 512, 2)])
@pytest.mark.parametrize("mode", ["tail", "head"])
def test_small_batch_splits_the_row_over_workgroups(oracle, model, dim, p, mode):
    """A batch that leaves one or two tiles per CU has its reduction axis split over up to four workgroups per
    tile (partial score planes in the forward workspace, a finishing kernel); without the workspace the same
    call runs unsplit.  Both must reproduce the oracle."""
    import ctypes as C
    from cuke_amd import _lib
    w = synth.custom_workload(model, n_ent=400, n_rel=11, dim=dim, batch=96, chunk=32, n_neg=40, norm_p=p, sigma=0.3,
                              gamma=6.0, ent_zipf=1.1, seed=dim + p)
    a = w.arrays
    m, ix = gpu_model(w)
    bat, _ = m._batch(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=mode)
    assert _lib.lib().kge_score_fwd_workspace(C.byref(m._tab), C.byref(bat)) >= 2 * 4 * w.batch * w.n_neg, \
        "this shape is meant to take the split"
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=mode)
    pos, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, p=p, gamma=w.gamma,
                             neg_mode=mode)
    assert_close(fw.neg.cpu().numpy(), negs, what=f"{model} split negatives")
    # the same call without a workspace: one workgroup per tile
    unsplit = torch.empty_like(fw.neg)
    res = torch.empty((w.batch, w.dim), dtype=torch.float32, device=fw.neg.device) if model == "RotatE" else None
    _lib.check(_lib.lib().kge_score_fwd(C.byref(m._tab), C.byref(bat), fw.pos.data_ptr(), unsplit.data_ptr(), None, None,
                                        res.data_ptr() if res is not None else None, None, 0,
                                        C.c_void_p(torch.cuda.current_stream().cuda_stream)), "kge_score_fwd")
    assert_close(unsplit.cpu().numpy(), negs, what=f"{model} unsplit negatives")


@pytest.mark.parametrize("model,p", [("TransE", 1), ("TransE", 2), ("DistMult", 2), ("ComplEx", 2)])
@pytest.mark.parametrize("mode", ["tail", "head"])
@pytest.mark.parametrize("batch,chunk,n_neg,dim", [(130, 26, 7, 64), (96, 32, 40, 640), (1024, 256, 256, 256)])
def test_positives_carried_by_the_tile_launch(oracle, model, p, mode, batch, chunk, n_neg, dim):
    """TransE / DistMult / ComplEx with shared negatives: the positives are scored by workgroups of the tile
    launch (no launch of their own).  Their scores must equal, bit for bit, those of the positives' own kernel
    (a call without negatives), also where the batch is not a multiple of the four positives of a workgroup,
    where the tile launch splits the reduction axis, and where the pair sums stay on the vector ALUs (then the
    dot-product models launch the positives' kernel themselves)."""
    w = synth.custom_workload(model, n_ent=500, n_rel=13, dim=dim, batch=batch, chunk=chunk, n_neg=n_neg, norm_p=p,
                              sigma=0.3, ent_zipf=1.1, seed=batch + dim + p)
    a = w.arrays
    m, ix = gpu_model(w)
    alone = m.score(ix["h"], ix["r"], ix["t"]).pos
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=mode)
    assert torch.equal(fw.pos, alone)
    pos, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, p=p, neg_mode=mode)
    assert_close(fw.pos.cpu().numpy(), pos, what=f"{model} carried positives")
    assert_close(fw.neg.cpu().numpy(), negs, what=f"{model} negatives beside carried positives")
    m.pair_sums = "vector_alus"
    fv = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=mode)
    assert torch.equal(fv.pos, alone)


@pytest.mark.parametrize("name,over", [
    ("cfg2_distmult", dict(n_ent=100_000, batch=1024)),
    ("cfg2_complex", dict(n_ent=100_000, batch=1024)),
    ("cfg4_rotate", dict(batch=512)),
    ("cfg5_transh", dict(n_ent=200_000, batch=2048)),
])
def test_scaled_configs_against_oracle(oracle, name, over):
    # same dim / chunk / negatives / distributions as the benchmark configuration, fewer rows
    w = synth.make_workload(name, **over)
    a = w.arrays
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    pos, negs = oracle.score(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                             p=w.norm_p, gamma=w.gamma)
    assert_close(fw.pos.cpu().numpy(), pos, what=f"{name} pos")
    assert_close(fw.neg.cpu().numpy(), negs, what=f"{name} neg")


@pytest.mark.parametrize("model", NEG_MODELS)
def test_diagonal_property_neg_equals_tails(oracle, model):
    # with neg == t and N == C (the reference's own layout) the k == b % C column is the positive score
    w = synth.custom_workload(model, n_ent=5000, n_rel=50, dim=128, batch=512, chunk=128, n_neg=128,
                              sigma=0.1, gamma=6.0, seed=8)
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["t"], w.chunk)
    diag = fw.neg[torch.arange(w.batch), torch.arange(w.batch) % w.chunk]
    assert_close(diag.cpu().numpy(), fw.pos.cpu().numpy(), what=f"{model} diagonal")


def test_empty_batch_and_bad_arguments():
    from cuke_amd.kge import KGEModel
    dev = torch.device("cuda:0")
    m = KGEModel("TransE", torch.zeros(10, 16, device=dev), torch.zeros(3, 16, device=dev))
    e = torch.zeros(0, dtype=torch.int64, device=dev)
    assert m.score(e, e, e).pos.numel() == 0
    assert m.residual(e, e, e).shape == (0, 16)
    h = torch.zeros(10, dtype=torch.int64, device=dev)
    with pytest.raises(ValueError):
        m.score(h, h, h, h, chunk=3)  # 10 is not a whole number of chunks of 3
    with pytest.raises(ValueError):
        m.score(h, h[:5], h)
    with pytest.raises(TypeError):
        m.score(h.float(), h, h)
